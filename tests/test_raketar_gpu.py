"""The Raketar decoder on the GPU against the plain implementation (tests/plain_raketar.py): each mechanism
alone, then whole models through the engine's step function, cache manager, scheduler and entry point,
however the work is cut."""
import copy
import math
import random

import pytest
import torch

import plain_raketar as plain
from raketar_helpers import (CONFIGS, CUT_TOLERANCE, DTYPES, SINGLE_LAYER_TOLERANCE, TOLERANCE, load_plain, make_model, plain_generate_greedy,
                             row_errors, run_cut)

pytestmark = pytest.mark.gpu
CASES = [(name, dtype) for name in CONFIGS for dtype in DTYPES]
DEVICE = "cuda:0"


def tokens_of(seed, count, vocab, avoid=()):
    rng = random.Random(seed)
    out = []
    while len(out) < count:
        token = rng.randrange(vocab)
        if token not in avoid:
            out.append(token)
    return out


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            folder = make_model(tmp_path_factory.mktemp(f"raketar_{name}"), CONFIGS[name], seed=31)
            raw, weights = load_plain(folder)
            made[name] = {"folder": folder, "raw": raw, "weights": weights, "plain": {}}
        return made[name]
    return get


def plain_logits(setup, tokens):
    key = tuple(tokens)
    if key not in setup["plain"]:
        setup["plain"][key] = plain.forward(setup["raw"], setup["weights"], list(tokens))[0]
    return setup["plain"][key]


def new_engine(setup, dtype, max_tokens=640, page_size=16, max_requests=4, **options):
    from tlie_amd import Engine
    return Engine(setup["folder"], dtype=dtype, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests, **options)


def assert_rows(got, want, tolerance, what):
    errors = row_errors(got, want)
    worst = int(errors.argmax())
    assert float(errors.max()) <= tolerance, f"{what}: row {worst} is off by {float(errors[worst]):.3g} of its largest value (allowed {tolerance})"


def split_product(dense, nsplit, generator):
    """A product as `nsplit` float partial sums that add up to `dense`."""
    from tlie_amd import ops
    if nsplit == 1:
        return ops.Product(dense.to(DEVICE).contiguous(), 1)
    parts = torch.randn(nsplit, *dense.shape, generator=generator)
    parts[0] += dense.float() - parts.sum(0)
    return ops.Product(parts.to(DEVICE).contiguous(), nsplit)


# ---- each mechanism alone ----------------------------------------------------------------------------------
@pytest.mark.parametrize("heads,per_group,dv,nsplit", [(4, 2, 24, 1), (6, 6, 80, 3), (3, 1, 5, 1), (2, 1, 130, 2)])
def test_two_maps_are_combined_normed_and_gated(heads, per_group, dv, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(heads * dv)
    tokens, lam, eps, mult = 7, 0.37, 1e-5, 0.6
    groups = heads // per_group
    first, second = torch.randn(tokens, heads, dv, generator=generator), torch.randn(tokens, heads, dv, generator=generator)
    gate = torch.randn(tokens, 11 + heads * dv, generator=generator)
    # the kernel's order: the query heads of one key head (a group's map) side by side
    a = torch.stack([first.reshape(tokens, groups, per_group, dv), second.reshape(tokens, groups, per_group, dv)], dim=2)
    got = ops.head_combine(a.reshape(tokens, 2 * heads * dv).contiguous().to(DEVICE), heads, dv, eps, torch.float32,
                           pair_group=per_group, pair_lambda=lam, mult=mult, gate=split_product(gate, nsplit, generator), gate_col=11)
    want = plain.unit_rms(first.double() - lam * second.double(), eps) * mult * torch.sigmoid(gate[:, 11:].double()).reshape(tokens, heads, dv)
    assert float((got.cpu().double() - want.reshape(tokens, -1)).abs().max()) < 2e-5
    # a map's result in pieces, each a head of its own of the attention kernel: (key head, piece, query head of the key head)
    for parts in (2, 3, 5):
        if dv % parts == 0:
            pieces = a.reshape(tokens, 2 * groups, per_group, parts, dv // parts).transpose(2, 3).contiguous()
            again = ops.head_combine(pieces.reshape(tokens, -1).to(DEVICE), heads, dv, eps, torch.float32, pair_group=per_group,
                                     pair_lambda=lam, mult=mult, gate=split_product(gate, 1, generator), gate_col=11, parts=parts)
            assert float((again - got).abs().max()) < 1e-6
    # one result a head, with a weight, in bfloat16 out
    weight = torch.randn(heads * dv, generator=generator)
    got = ops.head_combine(first.reshape(tokens, -1).contiguous().to(DEVICE), heads, dv, eps, torch.bfloat16, weight=weight.to(DEVICE))
    want = (plain.unit_rms(first.double(), eps).reshape(tokens, -1) * weight.double())
    assert float((got.cpu().double() - want).abs().max()) < 3e-2


@pytest.mark.parametrize("tokens,inner,outputs,top,dtype", [(5, 96, 6, 0, torch.float32), (3, 1000, 16, 0, torch.bfloat16),
                                                            (9, 64, 5, 2, torch.float32), (4, 200, 70, 70, torch.bfloat16),
                                                            (6, 130, 130, 3, torch.float32), (2, 32, 3, 1, torch.bfloat16)])
def test_products_with_few_outputs_and_the_router(tokens, inner, outputs, top, dtype):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(inner + outputs)
    x = torch.randn(tokens, inner, generator=generator).to(dtype)
    weight = (torch.randn(outputs, inner, generator=generator) / math.sqrt(inner)).to(dtype)        # (scores that do not saturate)
    bias = torch.randn(outputs, generator=generator).to(dtype)
    sums = x.double() @ weight.double().T
    if top == 0:
        got = ops.few_outputs(x.to(DEVICE), weight.to(DEVICE), bias.to(DEVICE))
        assert float((got.cpu().double() - (sums + bias.double())).abs().max()) < 1e-4 * math.sqrt(inner)
        return
    got = ops.few_outputs(x.to(DEVICE), weight.to(DEVICE), top=top).cpu().double()
    scores = torch.sigmoid(sums)
    want = torch.zeros_like(scores)
    picked = torch.topk(scores, top, dim=1).indices
    want.scatter_(1, picked, scores.gather(1, picked))
    assert (got != 0).sum(1).tolist() == [top] * tokens
    assert float((got - want).abs().max()) < 1e-5


def test_the_router_takes_the_lower_index_of_equal_scores():
    from tlie_amd import ops
    x = torch.ones(1, 8, device=DEVICE)
    weight = torch.zeros(6, 8, device=DEVICE)
    weight[1], weight[4], weight[5] = 0.25, 0.25, 0.1
    got = ops.few_outputs(x, weight, top=2).cpu()
    assert (got[0] != 0).tolist() == [False, True, False, False, True, False]
    got = ops.few_outputs(x, weight, top=1).cpu()
    assert (got[0] != 0).tolist() == [False, True, False, False, False, False]


@pytest.mark.parametrize("tokens,experts,block,shared,nsplit", [(5, 4, 6, 10, 1), (3, 7, 24, 0, 2), (18, 2, 3, 5, 1)])
def test_routed_gate_scales_an_experts_columns(tokens, experts, block, shared, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(experts * block)
    inter = experts * block + shared
    gate, up = torch.randn(tokens, inter, generator=generator), torch.randn(tokens, inter, generator=generator)
    scale = torch.rand(tokens, experts, generator=generator) * (torch.rand(tokens, experts, generator=generator) < 0.5)
    per_column = torch.cat([scale.repeat_interleave(block, dim=1), torch.ones(tokens, shared)], dim=1).double()
    want = plain.silu(per_column * gate.double()) * (per_column * up.double())
    product = split_product(torch.stack([gate, up], dim=2).reshape(tokens, 2 * inter), nsplit, generator)
    got = ops.routed_gate(product, scale.to(DEVICE).contiguous(), block, torch.float32)
    assert float((got.cpu().double() - want).abs().max()) < 2e-5


@pytest.mark.parametrize("tokens,width,nsplit,second", [(6, 96, 1, True), (3, 200, 2, True), (20, 64, 1, False)])
def test_residual_update_adds_both_results_and_leaves_a_copy(tokens, width, nsplit, second):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(width)
    mult = 0.45
    x, a, b = (torch.randn(tokens, width, generator=generator) for _ in range(3))
    summed = x.double() + mult * (a.double() + (b.double() if second else 0.0))
    residual = x.clone().to(DEVICE)
    assert ops.residual_update(residual, split_product(a, nsplit, generator), split_product(b, nsplit, generator) if second else None, mult) is None
    assert float((residual.cpu().double() - summed).abs().max()) < 1e-5
    residual = x.clone().to(DEVICE)
    copy = ops.residual_update(residual, split_product(a, nsplit, generator), split_product(b, nsplit, generator) if second else None, mult,
                               copy_dtype=torch.bfloat16)
    assert copy.dtype == torch.bfloat16 and torch.equal(copy, residual.to(torch.bfloat16))


@pytest.mark.parametrize("tokens,side_dim,nsplit", [(6, 10, 1), (3, 3, 2), (20, 24, 1)])
def test_the_token_inputs_gate(tokens, side_dim, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(side_dim)
    vocab, layers, layer = 30, 3, 1
    pre = torch.randn(tokens, side_dim, generator=generator) * 2.0
    ids = torch.randint(0, vocab, (tokens,), generator=generator)
    table = torch.randn(vocab, layers * side_dim, generator=generator)
    want = plain.gelu_tanh(pre.double()) * table.double()[ids][:, layer * side_dim:(layer + 1) * side_dim]
    got = ops.side_gate(split_product(pre, nsplit, generator), ids.to(torch.int32).to(DEVICE), table.to(DEVICE), layer * side_dim, torch.float32)
    assert float((got.cpu().double() - want).abs().max()) < 1e-5


def test_residual_inject_adds_the_embedding_and_a_vector():
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(9)
    table, vector, x = torch.randn(12, 40, generator=generator), torch.randn(40, generator=generator), torch.randn(5, 40, generator=generator)
    ids = torch.tensor([3, 0, 11, 3, 7], dtype=torch.int32)
    residual = x.clone().to(DEVICE)
    ops.residual_inject(residual, ids.to(DEVICE), table.to(DEVICE), vector.to(DEVICE))
    assert torch.allclose(residual.cpu(), x + table[ids.long()] + vector, atol=1e-6)
    residual = x.clone().to(DEVICE)
    ops.residual_inject(residual, None, None, vector.to(DEVICE))
    assert torch.allclose(residual.cpu(), x + vector, atol=1e-6)


SHORT_STEPS = ([23, 9], [(1, 4), (5, 0), (2, 1), (1, 1), (14, 3)])
LONG_STEPS = ([150, 41], [(70, 1), (1, 30), (60, 0), (18, 9), (1, 1)])


@pytest.mark.parametrize("heads,dim,vdim,cap,plan,nsplit", [(3, 24, 40, 10.0, SHORT_STEPS, 1), (2, 72, 130, 4.0, SHORT_STEPS, 2),
                                                            (1, 160, 16, 15.0, LONG_STEPS, 1), (2, 8, 70, 6.0, LONG_STEPS, 1),
                                                            (4, 32, 64, 15.0, SHORT_STEPS, 1), (1, 256, 5, 2.0, SHORT_STEPS, 1)])
def test_the_matrix_memory_carries_its_state(heads, dim, vdim, cap, plan, nsplit):
    """Two sequences of unequal length in steps of unequal portions (down to one token), in slots that are not in order,
    against the plain function on each whole sequence; gates that let the memory grow for a long time and gates that
    forget at once are both among them."""
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(dim + vdim)
    (lengths, steps), slots = plan, [2, 0]
    width = 2 * heads * dim + heads * vdim + 5                       # q | k | v | columns of someone else's
    fused = [torch.randn(length, width, generator=generator) for length in lengths]
    pre = [torch.randn(length, 2 * heads, generator=generator) * 2.0 for length in lengths]
    pre[0][:, heads:] += 8.0                                          # the first sequence forgets next to nothing
    pre[1][:, heads:] += 2.0
    scale = dim ** -0.5
    want = []
    for x, gates in zip(fused, pre):
        q = x[:, :heads * dim].double().reshape(-1, heads, dim) * scale
        k = x[:, heads * dim:2 * heads * dim].double().reshape(-1, heads, dim)
        v = x[:, 2 * heads * dim:2 * heads * dim + heads * vdim].double().reshape(-1, heads, vdim)
        gate_i, gate_f = plain.log_gates(gates[:, :heads].double(), gates[:, heads:].double(), cap)
        want.append(plain.mlstm_memory(q, k, v, gate_i, gate_f)[0].reshape(-1, heads * vdim))
    state = torch.zeros(3, *ops.mlstm_state_shape(heads, dim, vdim), device=DEVICE)
    state[1] = 5.0                                                    # a slot that belongs to nobody stays as it is
    got, at = [[], []], [0, 0]
    for counts in steps:
        live = [s for s in (0, 1) if counts[s] > 0]
        rows = torch.cat([fused[s][at[s]:at[s] + counts[s]] for s in live])
        gates = torch.cat([pre[s][at[s]:at[s] + counts[s]] for s in live]).to(DEVICE).contiguous()
        starts = [0]
        for s in live:
            starts.append(starts[-1] + counts[s])
        # one sequence more than live ones, without a slot: a sequence that pads a recorded step
        seq_start = torch.tensor(starts + [starts[-1]], dtype=torch.int32, device=DEVICE)
        seq_slot = torch.tensor([slots[s] for s in live] + [-1], dtype=torch.int32, device=DEVICE)
        out = ops.mlstm_scan(split_product(rows, nsplit, generator), 0, heads * dim, 2 * heads * dim, gates, state, seq_start, seq_slot,
                             heads, dim, vdim, cap, scale)
        for i, s in enumerate(live):
            got[s].append(out[starts[i]:starts[i + 1]].cpu())
            at[s] += counts[s]
    assert at == lengths
    for s in (0, 1):
        error = (torch.cat(got[s]).double() - want[s]).abs().max() / want[s].abs().max()
        assert float(error) < 1e-4, f"sequence {s}"           # (the quotient's denominator is a sum with cancellation)
    assert float((state[1] - 5.0).abs().max()) == 0.0


def _attend_shared_values(q, k, v, scale, page_size, cuts, dtype):
    """q [T, nq, d], k [T, nk, d], v [T, nv, dv] of one sequence through `qkv_place` and the plain attention kernel in
    portions of the sizes `cuts`, on pages that are not in order: nk / nv key heads in a row read one value head."""
    from tlie_amd import ops
    T, nq, d = q.shape
    nk, nv, dv = k.shape[1], v.shape[1], v.shape[2]
    blocks = (T + page_size - 1) // page_size
    order = list(range(blocks + 3))
    random.Random(T).shuffle(order)
    table = torch.tensor([order[:blocks]], dtype=torch.int32, device=DEVICE)
    cache = torch.zeros(blocks + 3, nv, page_size * (nk // nv * d + dv), dtype=dtype, device=DEVICE)
    fused = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1), torch.full((T, 7), 1e4)], dim=1)
    out, at, index = [], 0, 0
    while at < T:
        count = min(cuts[index % len(cuts)], T - at)
        positions = torch.arange(at, at + count, dtype=torch.int32, device=DEVICE)
        slots = torch.tensor([order[p // page_size] * page_size + p % page_size for p in range(at, at + count)], dtype=torch.int32, device=DEVICE)
        product = ops.Product(fused[at:at + count].to(dtype).to(DEVICE).contiguous(), 1)
        placed = ops.qkv_place(product, positions, slots, None, 0, cache, nq, nk, d, dv, dtype, value_heads=nv, extra_cols=7)
        token_seq = torch.zeros(count, dtype=torch.int32, device=DEVICE)
        seq_start = torch.tensor([0, count], dtype=torch.int32, device=DEVICE)
        for tiled in ((0, 1) if max(d, dv) <= 64 and count >= 4 else (0,)):
            got = ops.attention_generic(placed, cache, table, token_seq, positions, nq, nk, d, None, scale, tiled=tiled,
                                        seq_start=seq_start, value_dim=dv, value_heads=nv, float_out=True)
            assert got.dtype == torch.float32
            if tiled == 0:
                out.append(got.cpu())
            else:
                assert torch.equal(got.cpu(), out[-1])
        at += count
        index += 1
    return torch.cat(out).reshape(T, nq, dv)


@pytest.mark.parametrize("nq,nk,nv,d,dv,page_size,dtype", [(8, 4, 2, 16, 24, 16, torch.float32), (12, 2, 1, 8, 80, 16, torch.float32),
                                                           (6, 6, 3, 6, 5, 4, torch.float32), (4, 4, 2, 32, 32, 16, torch.bfloat16)])
def test_attention_whose_key_heads_share_value_heads(nq, nk, nv, d, dv, page_size, dtype):
    generator = torch.Generator().manual_seed(nq * d)
    T, scale = 150, 0.3
    q, k, v = (torch.randn(T, n, e, generator=generator).to(dtype).float() for n, e in ((nq, d), (nk, d), (nv, dv)))
    want = torch.zeros(T, nq, dv, dtype=torch.float64)
    for head in range(nq):
        key_head = head // (nq // nk)
        want[:, head] = plain.causal_softmax_attention(q[:, head].double(), k[:, key_head].double(), v[:, key_head // (nk // nv)].double(), scale)
    for cuts in ([T], [1], [40, 2, 1, 17]):
        got = _attend_shared_values(q, k, v, scale, page_size, cuts, dtype)
        assert float((got.double() - want).abs().max()) < (2e-5 if dtype == torch.float32 else 2e-2), f"cuts {cuts}"


# ---- single layers through the engine: a mixer's result from its input, and inputs made so that a fault shows ---------
def _single_layer(tmp_path, layer, seed, vocab=97, width=48, changes=None):
    raw = {"architecture": "Raketar", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
           "layers": [layer]}
    folder = make_model(tmp_path, raw, seed=seed)
    config, weights = load_plain(folder)
    if changes is not None:
        from tlie_amd.weights.safetensors_io import write_safetensors
        import os
        changes(weights)
        write_safetensors(os.path.join(folder, "model.safetensors"), {name: tensor.to(torch.bfloat16) for name, tensor in weights.items()})
        config, weights = load_plain(folder)
    return folder, config, weights


def _mixer_alone(folder, tokens, dtype, cuts):
    """The mixer's input and result of every token, from the traces of steps of the sizes `cuts`."""
    from tlie_amd import Engine, StepEntry
    engine = Engine(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=2)
    engine.admit("a")
    inputs, results, at, index = [], [], 0, 0
    while at < len(tokens):
        count = min(cuts[index % len(cuts)], len(tokens) - at)
        trace = {}
        engine.step([StepEntry("a", tokens[at:at + count], [count - 1])], trace=trace)
        inputs.append(trace["layer0.input_norm"].cpu())
        results.append(trace["layer0.attention_output"].cpu())
        at += count
        index += 1
    return torch.cat(inputs).double(), torch.cat(results).double()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer", [
    {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "diff": 0.3, "rot": {"base": 1000.0, "dims": 8, "scaling": {"factor": 2.0}}},
    {"heads": 3, "kv_heads": 1, "dim": 6, "vdim": 70, "scale": 0.5, "diff": 0.7, "rot": {"base": 20.0, "dims": 6}},
    {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.2, "diff": 0.5, "rot": {"base": 250000.0, "dims": 32, "scaling": {"factor": 4.0}}},
    {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 48, "scale": 0.25, "diff": 0.2, "rot": {"base": 300.0, "dims": 8}},
    {"heads": 6, "kv_heads": 1, "dim": 64, "vdim": 128, "scale": 0.125, "diff": 0.5, "rot": {"base": 10000.0, "dims": 64}},
])
def test_differential_attention_alone(tmp_path, mixer, dtype):
    folder, config, weights = _single_layer(tmp_path, {"type": "attention", "mixer": mixer, "mlp": None}, seed=5)
    tokens = tokens_of(6, 300, 97)             # (long enough for the keys to be cut into parts that are merged)
    for cuts in ([300], [33, 1, 2, 20, 150], [280] + [1] * 20):
        h, got = _mixer_alone(folder, tokens, dtype, cuts)
        want = plain.differential_attention(mixer, weights, "l0.mix.", h, torch.arange(len(tokens)), 1e-5)
        assert_rows(got, want, 2e-5 if dtype == "float32" else 3e-2, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer", [{"heads": 3, "dim": 24, "vdim": 40, "gate_cap": 10.0}, {"heads": 2, "dim": 72, "vdim": 130, "gate_cap": 4.0},
                                   {"heads": 1, "dim": 160, "vdim": 16, "gate_cap": 15.0}])
def test_the_memory_layer_alone(tmp_path, mixer, dtype):
    folder, config, weights = _single_layer(tmp_path, {"type": "mlstm", "mixer": mixer, "mlp": None}, seed=7)
    tokens = tokens_of(8, 75, 97)
    for cuts in ([75], [30, 1, 2, 9], [1]):
        h, got = _mixer_alone(folder, tokens, dtype, cuts)
        want = plain.mlstm(mixer, weights, "l0.mix.", h, 1e-5)[0]
        assert_rows(got, want, 3e-5 if dtype == "float32" else 3e-2, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far", [0, 15, 16, 17, 31, 32, 250])
def test_one_far_key_among_hundreds_decides_the_result(tmp_path, dtype, far):
    """The first map of one head is made to look at one position only: token B's key and token A's query are large in a
    dim that does not turn, so that B's value decides what A's head gives.  B stands at a page's first or last row, in
    the sequence's first tokens, or hundreds of positions back; A comes last, in a prompt's portion and decoded alone."""
    A, B, length = 95, 96, 300
    mixer = {"heads": 2, "kv_heads": 1, "dim": 12, "vdim": 20, "scale": 0.3, "diff": 0.4, "rot": {"base": 100.0, "dims": 8}}

    def boost(weights):
        h = {t: plain.rms_norm(weights["embed"][t], weights["l0.norm1"], 1e-5) for t in (A, B)}
        weights["l0.mix.q"][0 * 2 * 12 + 10] = 14.0 * h[A] / (h[A] @ h[A])          # head 0, map 1, dim 10 (past the rotated 8)
        weights["l0.mix.k"][10] = 14.0 * h[B] / (h[B] @ h[B])
    folder, config, weights = _single_layer(tmp_path, {"type": "attention", "mixer": mixer, "mlp": None}, seed=11, changes=boost)
    tokens = tokens_of(12, length, 97, avoid=(A, B))
    tokens[far], tokens[-1] = B, A
    other = list(tokens)
    other[far] = tokens[far + 1]
    want = plain_logits({"raw": config, "weights": weights, "plain": {}}, tokens)
    lost = plain_logits({"raw": config, "weights": weights, "plain": {}}, other)
    assert float(row_errors(lost[-1:], want[-1:])) > 0.2                             # the test shows a key that is lost
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=640, page_size=16, max_requests=2)
    for cuts in ([length], [length - 1, 1], [7, 64, 2]):
        got = run_cut(engine, "a", tokens, cuts)
        assert_rows(got[-1:], want[-1:], SINGLE_LAYER_TOLERANCE[dtype], f"B at {far}, cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_what_the_memory_took_in_long_ago_is_still_there(tmp_path, dtype):
    """Forget gates close to 1 and a key written at the third token that only the last token asks for: a state that is
    lost or zeroed on the way (between steps, in a slot that is used again) changes the last token's result."""
    A, B, length = 95, 96, 260
    mixer = {"heads": 2, "dim": 8, "vdim": 12, "gate_cap": 12.0}

    def boost(weights):
        h = {t: plain.rms_norm(weights["embed"][t], weights["l0.norm1"], 1e-5) for t in (A, B)}
        weights["l0.mix.q"][3] = 20.0 * h[A] / (h[A] @ h[A])
        weights["l0.mix.k"][3] = 20.0 * h[B] / (h[B] @ h[B])
        weights["l0.mix.f.b"][:] = 11.0
        weights["l0.mix.i.b"][:] = 0.0
    folder, config, weights = _single_layer(tmp_path, {"type": "mlstm", "mixer": mixer, "mlp": None}, seed=13, changes=boost)
    tokens = tokens_of(14, length, 97, avoid=(A, B))
    tokens[2], tokens[-1] = B, A
    other = list(tokens)
    other[2] = tokens[3]
    want = plain_logits({"raw": config, "weights": weights, "plain": {}}, tokens)
    lost = plain_logits({"raw": config, "weights": weights, "plain": {}}, other)
    assert float(row_errors(lost[-1:], want[-1:])) > 0.05
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=640, page_size=16, max_requests=1)      # one slot: used again by every cut
    for cuts in ([length], [length - 40] + [1] * 40, [5, 64, 2, 1]):
        got = run_cut(engine, "a", tokens, cuts)
        assert_rows(got[-1:], want[-1:], SINGLE_LAYER_TOLERANCE[dtype], f"cuts {cuts[:4]}")


# ---- whole models through the engine -----------------------------------------------------------------------
@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompt_matches_the_plain_implementation(setups, name, dtype):
    setup = setups(name)
    tokens = tokens_of(1, 150, CONFIGS[name]["vocab"])
    engine = new_engine(setup, dtype)
    got = run_cut(engine, "a", tokens, [len(tokens)])
    assert_rows(got, plain_logits(setup, tokens), TOLERANCE[dtype], f"{name} {dtype}")
    engine.cache.check()


@pytest.mark.parametrize("name", list(CONFIGS))
def test_every_layer_matches_the_plain_implementation(setups, name):
    """The residual after every layer run, in 32-bit: a fault shows in the first run it touches."""
    from tlie_amd import StepEntry
    setup = setups(name)
    tokens = tokens_of(2, 61, CONFIGS[name]["vocab"])
    layers = plain.forward(setup["raw"], setup["weights"], tokens)[1]
    engine = new_engine(setup, "float32")
    engine.admit("a")
    trace = {}
    engine.step([StepEntry("a", tokens, [len(tokens) - 1])], trace=trace)
    assert len(layers) == len(engine.spec.runs)
    for index, want in enumerate(layers):
        assert_rows(trace[f"layer{index}.output"], want, TOLERANCE["float32"], f"{name}: the residual after run {index}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_cuts_agree_with_each_other_and_with_the_plain_implementation(setups, name, dtype):
    """Token by token from the first token on; portions of changing sizes down to two tokens and one; most of a
    prompt and then a long run of single tokens over several page borders."""
    setup = setups(name)
    tokens = tokens_of(3, 131, CONFIGS[name]["vocab"])
    want = plain_logits(setup, tokens)
    engine = new_engine(setup, dtype)
    whole = run_cut(engine, "w", tokens, [len(tokens)])
    for cuts in ([1], [2], [7, 2, 33, 1, 16, 3], [40] + [1] * 200):
        got = run_cut(engine, ("c", tuple(cuts[:3])), tokens, cuts)
        assert_rows(got, want, TOLERANCE[dtype], f"{name} {dtype} cut {cuts[:6]}")
        assert_rows(got, whole, CUT_TOLERANCE[dtype], f"{name} {dtype} cut {cuts[:6]} against the whole prompt")
    engine.cache.check()


@pytest.mark.parametrize("name,dtype", CASES)
def test_batches_of_unequal_requests_with_pages_and_slots_used_again(setups, name, dtype):
    """Up to three live requests of unequal lengths in three slots more than once: portions of some beside single
    tokens of others, requests that pause for a step, a pool that only holds what is live."""
    from tlie_amd import StepEntry
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    lengths = {"a": 70, "b": 9, "c": 41, "d": 1, "e": 55, "f": 30}
    prompts = {key: tokens_of(10 + index, length, vocab) for index, (key, length) in enumerate(lengths.items())}
    engine = new_engine(setup, dtype, max_tokens=192, max_requests=3)
    rng = random.Random(5)
    waiting, live, at, rows = list(prompts), [], {}, {key: [] for key in prompts}
    steps = 0
    while waiting or live:
        while waiting and len(live) < 3 and sum((lengths[key] + 15) // 16 * 16 for key in live + [waiting[0]]) <= 192:
            key = waiting.pop(0)
            engine.admit(key)
            live.append(key)
            at[key] = 0
        entries, counts = [], {}
        for key in live:
            if len(live) > 1 and rng.random() < 0.25:
                continue                                              # left out of this step
            count = min(lengths[key] - at[key], rng.choice([1, 1, 2, 3, 9, 30]))
            entries.append(StepEntry(key, prompts[key][at[key]:at[key] + count], list(range(count))))
            counts[key] = count
        if not entries:
            continue
        logits = engine.step(entries)
        row = 0
        for entry in entries:
            rows[entry.request].append(logits[row:row + counts[entry.request]].clone())
            row += counts[entry.request]
            at[entry.request] += counts[entry.request]
            if at[entry.request] == lengths[entry.request]:
                engine.finish(entry.request)
                live.remove(entry.request)
        engine.cache.check()
        steps += 1
    assert steps > 12
    for key, tokens in prompts.items():
        assert_rows(torch.cat(rows[key]), plain_logits(setup, tokens), TOLERANCE[dtype], f"{name} {dtype} request {key}")


@pytest.mark.parametrize("name", list(CONFIGS))
def test_recorded_steps_equal_launched_steps_bit_for_bit(setups, name):
    """Steps replayed from recordings (padded to the recording's size, with padding tokens and sequences that belong to
    no request) against the same steps launched kernel by kernel: the same bits, also for the layers that carry state."""
    from tlie_amd import StepEntry
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(40 + index, length, vocab) for index, length in enumerate((37, 20, 50))]
    results = []
    for capture in (True, False):
        engine = new_engine(setup, "bfloat16", capture_graphs=capture)
        assert engine.runner.use_graphs
        rows = []
        for key in range(3):
            engine.admit(key)
        at = [0, 0, 0]
        for counts in [(5, 3, 0), (1, 1, 1), (1, 1, 1), (6, 2, 9), (1, 1, 1), (5, 3, 0), (1, 1, 1), (6, 0, 9), (1, 1, 1), (1, 0, 1)]:
            entries = [StepEntry(key, prompts[key][at[key]:at[key] + count], [count - 1]) for key, count in enumerate(counts) if count]
            rows.append(engine.step(entries).clone())
            for key, count in enumerate(counts):
                at[key] += count
        results.append(torch.cat(rows))
    assert torch.equal(results[0], results[1])
    assert bool(torch.isfinite(results[0]).all())


@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_generation_through_the_scheduler(setups, name):
    """The engine's own entry point: prompts of unequal lengths together under the scheduler, prompts cut into
    portions, greedy tokens equal to the plain implementation's in 32-bit."""
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(70 + index, length, vocab) for index, length in enumerate((45, 3, 18))]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 10) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=256)
    assert engine.generate(prompts, max_tokens=10, chunk_size=16, max_tokens_per_step=24) == want
    assert engine.generate([prompts[1]], max_tokens=10) == [want[1]]
    engine.cache.check()
    assert len(new_engine(setup, "bfloat16").generate(prompts, max_tokens=5)[2]) == 5


def test_a_preempted_request_is_recomputed_from_a_state_of_zero(setups):
    """A pool too small for all requests at once: the scheduler preempts and recomputes; a recomputed request must not
    see the memory its earlier admission left in a slot."""
    setup = setups("R")
    prompts = [tokens_of(90 + index, 40, CONFIGS["R"]["vocab"]) for index in range(4)]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 16) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=176, max_requests=4)
    assert engine.generate(prompts, max_tokens=16, admit_partial=True) == want
    engine.cache.check()


def test_long_decoding_keeps_to_the_plain_implementation(setups):
    """A short prompt and then hundreds of single tokens through recorded steps, in bfloat16 and in 32-bit."""
    setup = setups("S")
    tokens = tokens_of(55, 330, CONFIGS["S"]["vocab"])
    want = plain_logits(setup, tokens)
    for dtype in DTYPES:
        engine = new_engine(setup, dtype)
        got = run_cut(engine, "a", tokens, [6] + [1] * 400)
        assert_rows(got, want, TOLERANCE[dtype], f"{dtype}")


def test_the_command_line_and_the_replay_program_run_the_design(setups, tmp_path):
    """`generate` and `logits` of the framework's command line, and a trace of steps through `bin/trace_run` (a portion
    beside a single token, a request that ends and whose slot and pages are used again), on a model of this design."""
    import json
    import os
    import subprocess
    import sys
    import numpy
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    setup = setups("T")
    vocab = CONFIGS["T"]["vocab"]
    tokens, other = tokens_of(61, 40, vocab), tokens_of(62, 21, vocab)
    prompt = "ids:" + ",".join(str(token) for token in tokens[:9])
    cli = [sys.executable, os.path.join(root, "bin", "tinyllama_amd")]
    run = subprocess.run(cli + ["generate", setup["folder"], prompt, "6", "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert json.loads(run.stdout)["generated_tokens"] == plain_generate_greedy(setup["raw"], setup["weights"], tokens[:9], 6)
    run = subprocess.run(cli + ["logits", setup["folder"], prompt, "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert_rows(torch.tensor(json.loads(run.stdout)["logits"])[None], plain_logits(setup, tokens[:9])[-1:], TOLERANCE["float32"], "logits")
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[30:31], "want": [0]}, {"id": "b", "tokens": other, "want": [20]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "c", "tokens": other[:7], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": tokens[31:], "want": [8]}, {"id": "c", "tokens": other[7:], "want": [13]}], "end": ["a", "c"]}]
    for dtype in DTYPES:
        out = tmp_path / dtype
        run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", setup["folder"], "--dtype", dtype,
                              "--out", str(out), "--max-tokens", "128", "--max-requests", "2"],
                             input="".join(json.dumps(line) + "\n" for line in lines), capture_output=True, text=True, timeout=300)
        assert run.returncode == 0 and run.stdout.split() == ["done", "0", "done", "1", "done", "2", "done", "3"], run.stderr
        assert not (out / "2.f32").exists()
        read = lambda step: torch.from_numpy(numpy.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, vocab))
        want, want_other = plain_logits(setup, tokens), plain_logits(setup, other)
        assert_rows(read(0), want[[0, 29]], TOLERANCE[dtype], f"{dtype} step 0")
        assert_rows(read(1), torch.stack([want[30], want_other[20]]), TOLERANCE[dtype], f"{dtype} step 1")
        assert_rows(read(3), torch.stack([want[39], want_other[20]]), TOLERANCE[dtype], f"{dtype} step 3")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["memory_only", "attention_only"])
def test_models_of_one_kind_of_layer_and_odd_sizes(tmp_path, which, dtype):
    """A model without any attention layer (no page group at all) at a width that is no multiple of 8, and one without
    any memory layer (no state area) whose loop runs once and ends with the model's last layer."""
    if which == "memory_only":
        raw = {"architecture": "Raketar", "vocab": 77, "width": 100, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
               "token_side": {"dim": 5}, "loop": {"start": 0, "stop": 2, "times": 2},
               "layers": [{"type": "mlstm", "mixer": {"heads": 2, "dim": 20, "vdim": 30, "gate_cap": 8.0}, "mlp": {"kind": "dense", "ff": 52}},
                          {"type": "mlstm", "mixer": {"heads": 5, "dim": 4, "vdim": 7, "gate_cap": 20.0}, "mlp": None}]}
    else:
        rot = {"base": 5000.0, "dims": 16, "scaling": {"factor": 3.0}}
        raw = {"architecture": "Raketar", "vocab": 90, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 1.5,
               "loop": {"start": 1, "stop": 2, "times": 1},
               "layers": [{"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.25, "diff": 0.0, "rot": rot},
                           "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 70, "top": 4}, "shared": {"ff": 8}}},
                          {"type": "attention", "mixer": {"heads": 8, "kv_heads": 2, "dim": 16, "vdim": 64, "scale": 0.25, "diff": 0.9, "rot": rot},
                           "mlp": None}]}
    folder = make_model(tmp_path, raw, seed=17)
    config, weights = load_plain(folder)
    tokens = tokens_of(19, 140, raw["vocab"])
    want = plain.forward(config, weights, tokens)[0]
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=320, page_size=16, max_requests=2)
    for cuts in ([140], [100] + [1] * 40, [3, 64, 2, 1]):
        assert_rows(run_cut(engine, "a", tokens, cuts), want, TOLERANCE[dtype], f"{which} {dtype} cuts {cuts[:4]}")
    engine.cache.check()
    assert engine.generate([tokens[:12], tokens[20:25]], max_tokens=4, chunk_size=8) is not None
