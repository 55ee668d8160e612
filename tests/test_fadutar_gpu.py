"""The Fadutar decoder on the GPU against the plain implementation (tests/plain_fadutar.py): each
mechanism alone, then whole models through the engine's step function, cache manager, scheduler
and entry point, however the work is cut."""
import math
import random

import pytest
import torch

from fadutar_helpers import CONFIGS, CUT_TOLERANCE, DTYPES, TOLERANCE, load_plain, make_model, row_errors, run_cut
from plain_fadutar import (plain_block_gate, plain_causal_conv, plain_forward, plain_gated_recurrence,
                           plain_gelu_tanh, plain_generate_greedy, plain_offset_norm, plain_sink_attention)

pytestmark = pytest.mark.gpu
CASES = [(name, dtype) for name in CONFIGS for dtype in DTYPES]
DEVICE = "cuda:0"


def tokens_of(seed, count, vocab):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(count)]


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            folder = make_model(tmp_path_factory.mktemp(f"fadutar_{name}"), CONFIGS[name], seed=23)
            raw, weights = load_plain(folder)
            made[name] = {"folder": folder, "raw": raw, "weights": weights, "plain": {}}
        return made[name]
    return get


def plain_logits(setup, tokens):
    key = tuple(tokens)
    if key not in setup["plain"]:
        setup["plain"][key] = plain_forward(setup["raw"], setup["weights"], list(tokens))
    return setup["plain"][key]


def new_engine(setup, dtype, max_tokens=640, page_size=16, max_requests=4, **options):
    from tlie_amd import Engine
    return Engine(setup["folder"], dtype=dtype, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests, **options)


def assert_rows(got, want, tolerance, what):
    errors = row_errors(got, want)
    worst = int(errors.argmax())
    assert float(errors.max()) <= tolerance, f"{what}: row {worst} is off by {float(errors[worst]):.3g} of its largest value (allowed {tolerance})"


# ---- each mechanism alone ----------------------------------------------------------------------------------
@pytest.mark.parametrize("rows,hidden,nsplit", [(5, 96, 1), (3, 200, 3), (17, 1000, 2)])
def test_norm_of_a_result_joins_the_residual_and_the_sum_is_normed(rows, hidden, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(hidden)
    residual = torch.randn(rows, hidden, generator=generator)
    parts = torch.randn(nsplit, rows, hidden, generator=generator)
    post, weight = 0.1 * torch.randn(hidden, generator=generator), 0.1 * torch.randn(hidden, generator=generator)
    want_residual = residual.double() + plain_offset_norm(parts.double().sum(0), post, 1e-5)
    want_out = plain_offset_norm(want_residual, weight, 1e-6)
    on_device = residual.to(DEVICE)
    out = ops.norm_add_rmsnorm(on_device, ops.Product(parts.to(DEVICE), nsplit), (1 + post).to(DEVICE), 1e-5, (1 + weight).to(DEVICE),
                               1e-6, torch.float32)
    assert_rows(on_device, want_residual, 1e-6, "the residual")
    assert_rows(out, want_out, 1e-6, "the normed sum")
    # only some rows, the residual left as it was
    picked = torch.tensor([rows - 1, 0], dtype=torch.int32, device=DEVICE)
    before = residual.to(DEVICE)
    some = ops.norm_add_rmsnorm(before, ops.Product(parts.to(DEVICE), nsplit), (1 + post).to(DEVICE), 1e-5, (1 + weight).to(DEVICE),
                                1e-6, torch.float32, rows=picked)
    assert torch.equal(before.cpu(), residual)
    assert_rows(some, want_out[[rows - 1, 0]], 1e-6, "the picked rows")


@pytest.mark.parametrize("limit,alpha", [(1.0, 1.702), (0.4, 1.702), (3.0, 1.0)])
def test_clamped_gate(limit, alpha):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(3)
    rows, inter = 7, 44
    gate, up = 2 * torch.randn(rows, inter, generator=generator), 2 * torch.randn(rows, inter, generator=generator)
    g, u = gate.double().clamp(max=limit), up.double().clamp(-limit, limit)
    want = g * torch.sigmoid(alpha * g) * (u + 1)
    both = torch.stack([gate, up], dim=2).reshape(rows, 2 * inter).to(DEVICE)
    got = ops.silu_mul(ops.Product(both, 1), torch.float32, interleaved=True, gate="clamped_swish", alpha=alpha, limit=limit)
    assert float((got.cpu().double() - want).abs().max()) < 1e-6
    assert float(want.abs().max()) > 0.2                      # (the clamps were at work and the values are not all tiny)


@pytest.mark.parametrize("rows,blocks,inner,outer", [(1, 3, 8, 16), (19, 2, 130, 70), (33, 5, 7, 3)])
def test_block_diagonal_product(rows, blocks, inner, outer):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(rows)
    # x lies inside a wider array (a head's first dims), the result goes into a wider one too
    x_wide, out_wide = inner + 5, outer + 3
    x = torch.randn(rows, blocks, x_wide, generator=generator)
    weight = torch.randn(blocks, outer, inner, generator=generator)             # [out, in] per block, as stored
    bias = torch.randn(blocks, outer, generator=generator)
    want = torch.einsum("tbi,boi->tbo", x[:, :, 2:2 + inner].double(), weight.double()) + bias.double()
    out = torch.full((rows, blocks, out_wide), 7.0, device=DEVICE)
    ops.block_linear(x.to(DEVICE), 2, blocks * x_wide, x_wide, weight.transpose(1, 2).contiguous().to(DEVICE), bias.to(DEVICE),
                     out, 1, blocks * out_wide, out_wide, rows)
    assert float((out[:, :, 1:1 + outer].cpu().double() - want).abs().max()) < 1e-4
    assert float((out[:, :, 0] - 7.0).abs().max()) == 0.0 and float((out[:, :, 1 + outer:] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("rows,blocks,inner,outer,wide", [(17, 3, 32, 16, False), (200, 2, 96, 70, True), (129, 5, 64, 3, False), (300, 1, 256, 512, True)])
def test_block_diagonal_product_on_the_matrix_cores(rows, blocks, inner, outer, wide):
    """bfloat16 weights, x in bfloat16 or (wide) in float, many rows: against float64 on the same rounded operands."""
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(rows + inner)
    x_wide, out_wide = inner + 8, outer + 3
    x = torch.randn(rows, blocks, x_wide, generator=generator).bfloat16()
    weight = (torch.randn(blocks, outer, inner, generator=generator) / inner ** 0.5).bfloat16()
    bias = torch.randn(blocks, outer, generator=generator).bfloat16()
    want = torch.einsum("tbi,boi->tbo", x[:, :, 8:8 + inner].double(), weight.double()) + bias.double()
    given = (x.float() if wide else x).to(DEVICE)
    out = torch.full((rows, blocks, out_wide), 7.0, device=DEVICE, dtype=torch.float32)
    ops.block_linear(given, 8, blocks * x_wide, x_wide, weight.transpose(1, 2).contiguous().to(DEVICE), bias.to(DEVICE),
                     out, 1, blocks * out_wide, out_wide, rows, weight=weight.to(DEVICE))
    assert float((out[:, :, 1:1 + outer].cpu().double() - want).abs().max()) < 1e-4
    assert float((out[:, :, 0] - 7.0).abs().max()) == 0.0 and float((out[:, :, 1 + outer:] - 7.0).abs().max()) == 0.0
    # and the same rows through the plain kernel: the two routes agree to the sums' rounding
    plain = torch.full((rows, blocks, out_wide), 7.0, device=DEVICE, dtype=torch.float32)
    ops.block_linear(given, 8, blocks * x_wide, x_wide, weight.transpose(1, 2).contiguous().to(DEVICE), bias.to(DEVICE),
                     plain, 1, blocks * out_wide, out_wide, rows)
    assert float((out - plain).abs().max()) < 1e-4


def _attend(q, k, v, sink, scale, chunk, page_size, cuts, dtype=torch.float32):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence through the placing kernel and the attention
    kernel, in steps of the sizes `cuts`, with the sequence's pages in a scrambled order."""
    from tlie_amd import ops
    tokens, heads, d = q.shape
    groups, dv = k.shape[1], v.shape[2]
    blocks = (tokens + page_size - 1) // page_size
    order = list(range(blocks + 3))
    random.Random(blocks).shuffle(order)
    shape = (blocks + 3, 2, groups, page_size * d) if d == dv else (blocks + 3, groups, page_size * (d + dv))
    cache = torch.zeros(shape, dtype=dtype, device=DEVICE)
    table = torch.tensor([order[:blocks]], dtype=torch.int32, device=DEVICE)
    outs, at, index = [], 0, 0
    while at < tokens:
        count = min(cuts[index % len(cuts)], tokens - at)
        index += 1
        positions = torch.arange(at, at + count, dtype=torch.int32, device=DEVICE)
        slots = torch.tensor([order[p // page_size] * page_size + p % page_size for p in range(at, at + count)], dtype=torch.int32, device=DEVICE)
        fused = torch.cat([q[at:at + count].reshape(count, -1), k[at:at + count].reshape(count, -1), v[at:at + count].reshape(count, -1)], dim=1)
        placed = ops.qkv_place(ops.Product(fused.to(DEVICE).contiguous(), 1), positions, slots, None, 0, cache, heads, groups, d, dv, dtype)
        seq = torch.zeros(count, dtype=torch.int32, device=DEVICE)
        start = torch.tensor([0, count], dtype=torch.int32, device=DEVICE)
        for tiled in ((0, 1) if max(d, dv) <= 64 else (0,)):
            out = ops.attention_generic(placed, cache, table, seq, positions, heads, groups, d, None, scale, tiled=tiled, seq_start=start,
                                        value_dim=dv, chunk=chunk, sink=sink.to(DEVICE) if sink is not None else None)
            if tiled:
                assert torch.equal(out, outs[-1]), "the two forms of the attention kernel differ in bits"
            else:
                outs.append(out)
        at += count
    return torch.cat(outs, dim=0).reshape(tokens, heads, dv)


@pytest.mark.parametrize("heads,groups,d,dv,chunk,page_size", [(4, 2, 16, 24, 24, 16), (3, 3, 9, 5, 7, 4), (2, 1, 72, 8, None, 16),
                                                               (4, 1, 56, 40, 60, 16), (2, 2, 8, 80, 33, 8)])
def test_attention_with_sink_and_chunks(heads, groups, d, dv, chunk, page_size):
    generator = torch.Generator().manual_seed(d * dv)
    tokens = 150
    q, k, v = (torch.randn(tokens, n, size, generator=generator) for n, size in ((heads, d), (groups, d), (groups, dv)))
    sink = torch.randn(heads, generator=generator)
    want = plain_sink_attention(q, k, v, sink, 0.31, chunk)
    for cuts in ([tokens], [1], [37, 2, 5, 1]):
        got = _attend(q, k, v, sink, 0.31, chunk, page_size, cuts)
        assert float((got.cpu().double() - want).abs().max()) < 2e-5, f"cut {cuts}"


def _attend_matrix_cores(q, k, v, sink, scale, chunk, page_size, cuts):
    """The same through the kernel on the matrix cores (bfloat16, one head size), launched as the part
    launches it: a work list for steps of several tokens, none for single tokens, keys cut into parts
    as the kernel's own policy says."""
    from types import SimpleNamespace
    import numpy as np
    from tlie_amd import ops
    tokens, heads, d = q.shape
    groups = k.shape[1]
    blocks = (tokens + page_size - 1) // page_size
    order = list(range(blocks + 3))
    random.Random(blocks).shuffle(order)
    cache = torch.zeros((blocks + 3, 2, groups, page_size * d), dtype=torch.bfloat16, device=DEVICE)
    table = torch.tensor([order[:blocks]], dtype=torch.int32, device=DEVICE)
    outs, at, index = [], 0, 0
    while at < tokens:
        count = min(cuts[index % len(cuts)], tokens - at)
        index += 1
        positions = torch.arange(at, at + count, dtype=torch.int32, device=DEVICE)
        slots = torch.tensor([order[p // page_size] * page_size + p % page_size for p in range(at, at + count)], dtype=torch.int32, device=DEVICE)
        fused = torch.cat([q[at:at + count].reshape(count, -1), k[at:at + count].reshape(count, -1), v[at:at + count].reshape(count, -1)], dim=1)
        placed = ops.qkv_place(ops.Product(fused.to(DEVICE).contiguous(), 1), positions, slots, None, 0, cache, heads, groups, d, d, torch.bfloat16)
        host = {"seq_start": np.asarray([0, count], dtype=np.int32), "seq_len": np.asarray([at + count], dtype=np.int32)}
        ctx = SimpleNamespace(max_new=count, num_seqs=1, num_tokens=count, max_context=at + count, scratch={}, tile_owner=None,
                              compute_units=256, host=host, tokens=positions)
        tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, heads // groups, groups, d)
        outs.append(ops.attention_mfma(placed, cache, table, tiles, positions, heads, groups, d, None, scale, nsplit, split_len, col_tiles,
                                       waves, shared, chunk=chunk, sink=sink.to(DEVICE) if sink is not None else None))
        at += count
    return torch.cat(outs, dim=0).reshape(tokens, heads, d)


@pytest.mark.parametrize("heads,groups,d,chunk,page_size,tokens", [(4, 2, 32, 48, 16, 300), (8, 1, 64, 100, 16, 1000), (2, 2, 16, 33, 32, 200),
                                                                   (6, 3, 128, None, 16, 300), (4, 4, 80, 72, 16, 900)])
def test_attention_on_the_matrix_cores_with_sink_and_chunks(heads, groups, d, chunk, page_size, tokens):
    generator = torch.Generator().manual_seed(d + tokens)
    q, k, v = (torch.randn(tokens, n, d, generator=generator).bfloat16().float() for n in (heads, groups, groups))
    sink = torch.randn(heads, generator=generator) + 1.0
    want = plain_sink_attention(q, k, v, sink, 0.2, chunk)
    for cuts in ([tokens], [1], [tokens - 40] + [1] * 40, [37, 2, 5, 1, 130]):
        if cuts == [1] and tokens > 300:
            continue
        got = _attend_matrix_cores(q, k, v, sink, 0.2, chunk, page_size, cuts)
        assert float((got.float().cpu().double() - want).abs().max()) < 3e-2, f"cut {cuts[:5]}"
    # the sink taken away changes the result by far more than that: it is not a detail within the tolerance
    assert float((plain_sink_attention(q, k, v, sink - 30.0, 0.2, chunk) - want).abs().max()) > 0.2


def test_a_sink_that_is_left_out_and_a_key_past_the_chunk_edge_show():
    """Weights made so that faults show: one query and one key are scaled so that their score towers over
    all others; just inside the query's chunk that key takes nearly all the weight, just outside it none;
    and a large sink takes nearly all the weight from the keys."""
    heads, groups, d, dv, chunk, page_size = 2, 1, 16, 16, 20, 16
    generator = torch.Generator().manual_seed(1)
    tokens = 101
    q, k, v = (0.1 * torch.randn(tokens, n, size, generator=generator) for n, size in ((heads, d), (groups, d), (groups, dv)))
    sink = torch.tensor([-30.0, -30.0])
    query = 99                                                        # its chunk is 80 .. 99
    for target, inside in ((80, True), (79, False), (99, True), (60, False)):
        qq, kk = q.clone(), k.clone()
        qq[query, :, 0], kk[target, :, 0] = 30.0, 30.0
        got = _attend(qq, kk, v, sink, 1.0, chunk, page_size, [97, 1, 1, 1, 1])[query].cpu()
        near = float((got - v[target, 0]).abs().max())
        assert (near < 1e-3) == inside, f"key {target} for the query at {query}: distance {near}"
        assert float((got.double() - plain_sink_attention(qq, kk, v, sink, 1.0, chunk)[query]).abs().max()) < 1e-5
    # the first tokens: position 0 sees itself and the sink only
    strong = torch.tensor([4.0, -4.0])
    got = _attend(q, k, v, strong, 1.0, chunk, page_size, [1])[0].cpu().double()
    score = (q[0].double() @ k[0, 0].double())
    share = torch.exp(score) / (torch.exp(score) + torch.exp(strong.double()))
    assert float((got - share[:, None] * v[0, 0].double()).abs().max()) < 1e-6
    assert float(share[0]) < 0.03 < 0.9 < float(share[1])


SHORT_STEPS = ([23, 9], [(1, 4), (5, 0), (2, 1), (1, 1), (14, 3)])
LONG_STEPS = ([300, 101], [(130, 1), (1, 70), (100, 0), (68, 29), (1, 1)])        # portions long enough for the sliced form


@pytest.mark.parametrize("width,blocks,taps,plan", [(64, 1, 1, SHORT_STEPS), (48, 3, 5, SHORT_STEPS), (130, 2, 4, SHORT_STEPS),
                                                    (48, 3, 5, LONG_STEPS), (130, 1, 2, LONG_STEPS)])
def test_convolution_and_recurrence_carry_their_state(width, blocks, taps, plan):
    """Two sequences of unequal length in steps of unequal portions (down to one token), in slots that are
    not in order, against the plain functions on each whole sequence."""
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(width)
    (lengths, steps), slots = plan, [2, 0]
    inside = width // blocks
    conv, conv_bias = torch.randn(width, taps, generator=generator), torch.randn(width, generator=generator)
    gate_r, gate_i = (torch.randn(blocks, inside, inside, generator=generator) / math.sqrt(inside) for _ in range(2))
    bias_r, bias_i = torch.randn(blocks, inside, generator=generator), torch.randn(blocks, inside, generator=generator)
    lam = torch.randn(width, generator=generator) - 2.0               # decays close to 1 among them
    fused = [torch.randn(length, 2 * width, generator=generator) for length in lengths]      # gate branch | inputs
    want = []
    for x in fused:
        u = plain_causal_conv(x[:, width:], conv, conv_bias)
        states = plain_gated_recurrence(u, plain_block_gate(u, gate_r, bias_r), plain_block_gate(u, gate_i, bias_i), lam)
        want.append(states * plain_gelu_tanh(x[:, :width]))
    gates_t = torch.cat([gate_r.transpose(1, 2), gate_i.transpose(1, 2)], dim=2).contiguous().to(DEVICE)
    gate_bias = torch.cat([bias_r, bias_i], dim=1).contiguous().to(DEVICE)
    state = torch.zeros(3, taps, width, device=DEVICE)
    state[1] = 5.0                                                    # a slot that belongs to nobody stays as it is
    got = [[], []]
    at = [0, 0]
    for step, counts in enumerate(steps):
        live = [s for s in (0, 1) if counts[s] > 0]
        rows = torch.cat([fused[s][at[s]:at[s] + counts[s]] for s in live]).to(DEVICE).contiguous()
        seq_start = torch.tensor([0] + list(torch.tensor([counts[s] for s in live]).cumsum(0)), dtype=torch.int32, device=DEVICE)
        token_seq = torch.tensor([i for i, s in enumerate(live) for _ in range(counts[s])], dtype=torch.int32, device=DEVICE)
        seq_slot = torch.tensor([slots[s] for s in live], dtype=torch.int32, device=DEVICE)
        token_slot = seq_slot[token_seq.long()].contiguous()
        product = ops.Product(rows, 1)
        u = ops.causal_conv(product, width, conv.to(DEVICE), conv_bias.to(DEVICE), state, token_seq, token_slot, seq_start)
        gates = torch.empty(rows.shape[0], 2 * width, device=DEVICE)
        ops.block_linear(u, 0, width, inside, gates_t, gate_bias, gates, 0, 2 * width, 2 * inside, rows.shape[0])
        out = ops.gated_recurrence(product, width, 0, u, gates, lam.to(DEVICE), 8.0, state, seq_start, seq_slot, inside, torch.float32,
                                   max_new=max(counts))
        for i, s in enumerate(live):
            got[s].append(out[int(seq_start[i]):int(seq_start[i + 1])].cpu())
            at[s] += counts[s]
    assert at == lengths
    for s in (0, 1):
        assert float((torch.cat(got[s]).double() - want[s]).abs().max()) < 2e-5, f"sequence {s}"
    assert float((state[1] - 5.0).abs().max()) == 0.0


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
    """The residual after every layer, in 32-bit: a fault shows in the first layer it touches."""
    from tlie_amd import StepEntry
    setup = setups(name)
    tokens = tokens_of(2, 61, CONFIGS[name]["vocab"])
    layers = []
    plain_forward(setup["raw"], setup["weights"], tokens, layers)
    engine = new_engine(setup, "float32")
    engine.admit("a")
    trace = {}
    engine.step([StepEntry("a", tokens, [len(tokens) - 1])], trace=trace)
    for index, want in enumerate(layers):
        assert_rows(trace[f"layer{index}.output"], want, 1e-5, f"{name}: the residual after layer {index}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_cuts_agree_with_each_other_and_with_the_plain_implementation(setups, name, dtype):
    """Token by token from the first token on; portions of changing sizes down to two tokens and one;
    most of a prompt and then a long run of single tokens over several chunk and page borders."""
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
    """Up to three live requests of unequal lengths in two slots more than once: portions of some beside
    single tokens of others, requests that pause for a step, a pool that only holds what is live."""
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
            left = lengths[key] - at[key]
            count = min(left, rng.choice([1, 1, 2, 3, 9, 30]))
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
    """Steps replayed from recordings (padded to the recording's size, with padding tokens and sequences
    that belong to no request) against the same steps launched kernel by kernel: the same bits, also
    for the mixers that carry state."""
    from tlie_amd import StepEntry
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(40 + index, length, vocab) for index, length in enumerate((37, 20, 50))]
    results = []
    for capture in (True, False):
        engine = new_engine(setup, "bfloat16", capture_graphs=capture)
        rows = []
        for key in range(3):
            engine.admit(key)
        at = [0, 0, 0]
        # the same shapes come several times, so that recordings are replayed, not only made
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
    """The engine's own entry point: prompts of unequal lengths together under the scheduler, prompts cut
    into portions, greedy tokens equal to the plain implementation's in 32-bit."""
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(70 + index, length, vocab) for index, length in enumerate((45, 3, 18))]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 12) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=256)
    assert engine.generate(prompts, max_tokens=12, chunk_size=16, max_tokens_per_step=24) == want
    # again on the same engine (slots and pages of the first call are back), one request alone, in bfloat16 only the length
    assert engine.generate([prompts[1]], max_tokens=12) == [want[1]]
    engine.cache.check()
    assert len(new_engine(setup, "bfloat16").generate(prompts, max_tokens=5)[2]) == 5


def test_a_preempted_request_is_recomputed_from_a_state_of_zero(setups):
    """A pool too small for all requests at once: the scheduler preempts and recomputes; a recomputed
    request must not see the state its earlier admission left in a slot."""
    setup = setups("Q")
    prompts = [tokens_of(90 + index, 40, CONFIGS["Q"]["vocab"]) for index in range(4)]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 20) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=176, max_requests=4)
    stats = {}
    assert engine.generate(prompts, max_tokens=20, stats=stats, admit_partial=True) == want
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_attention_with_keys_wider_than_a_head_size(tmp_path, dtype):
    """A latent vector and rotated part that together pass the widest head the attention kernels take: the
    cache then keeps values of rank rows only and the plain kernel reads it."""
    raw = {"architecture": "Fadutar", "vocab": 64, "width": 32, "norm": {"eps": 1e-5}, "layers": [
        {"type": "latent_attention", "mixer": {"heads": 2, "dim": 8, "rot_dim": 12, "vdim": 8, "kv_rank": 250, "scale": 0.2,
                                               "rot": {"base": 100.0, "dims": 12}}, "mlp": None}]}
    folder = make_model(tmp_path, raw, seed=4)
    config, weights = load_plain(folder)
    tokens = tokens_of(8, 50, 64)
    want = plain_forward(config, weights, tokens)
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=128, page_size=16, max_requests=2)
    assert not engine.model.blocks[0].mixer.wide_values
    for cuts in ([50], [1], [20, 3, 1]):
        assert_rows(run_cut(engine, "a", tokens, cuts), want, TOLERANCE[dtype], f"cut {cuts}")
