"""The Raketar configuration on the CPU: config.json -> the model as data, the tensors it expects, what it
refuses; and properties of the plain implementation's own pieces."""
import copy
import math

import pytest
import torch

import plain_raketar as plain
from raketar_helpers import CONFIG_R, CONFIG_S, CONFIG_T
from tlie_amd.errors import EngineError
from tlie_amd.models.builder import expected_tensors
from tlie_amd.registry import config_from_dict


def test_the_architecture_is_found_by_its_name_and_turned_into_data():
    spec = config_from_dict(CONFIG_R).to_spec()
    assert spec.architecture == "Raketar" and spec.max_positions is None
    assert [layer.block for layer in spec.layers] == ["parallel"] * 4
    assert [layer.mixer.kind for layer in spec.layers] == ["differential_attention", "mlstm", "differential_attention", "mlstm"]
    assert [None if layer.feed_forward is None else layer.feed_forward.kind for layer in spec.layers] == [
        "gated_mlp", "routed_mlp", None, "gated_mlp"]
    assert all(layer.residual_scale == 0.7 for layer in spec.layers)
    assert [layer.layer_input["offset"] for layer in spec.layers] == [0, 10, 20, 30]
    # layers 1 and 2 run three times in a row; every run owns its cache or state
    assert [run.layer for run in spec.runs] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [run.cache_of for run in spec.runs] == list(range(8))
    assert [run.add_embedding for run in spec.runs] == [False, False, False, True, False, True, False, False]
    assert [run.add_vector for run in spec.runs] == [None, ("loop.step", 0), None, ("loop.step", 1), None, ("loop.step", 2), None, None]
    rotary = spec.layers[0].mixer["position"]
    assert (rotary["rot_dim"], rotary["head_dim"], rotary["linear_factor"], rotary["theta"]) == (8, 16, 2.0, 1000.0)
    assert spec.layers[2].mixer["position"]["linear_factor"] == 1.0
    routed = spec.layers[1].feed_forward
    assert (routed["experts"], routed["top"], routed["expert_size"], routed["shared_size"]) == (5, 2, 24, 40)


def test_a_model_without_a_loop_or_a_token_input():
    spec = config_from_dict(CONFIG_T).to_spec()
    assert [(run.layer, run.cache_of, run.add_embedding, run.add_vector) for run in spec.runs] == [(0, 0, False, None), (1, 1, False, None)]
    assert "loop.step" not in {tensor.name for tensor in expected_tensors(spec)}
    spec = config_from_dict(CONFIG_S).to_spec()
    assert all(layer.layer_input is None for layer in spec.layers)
    assert [run.layer for run in spec.runs] == [0, 0, 1, 2] and spec.runs[1].add_embedding and not spec.runs[0].add_embedding
    assert spec.layers[0].feed_forward["shared_size"] == 0
    assert "side.embed" not in {tensor.name for tensor in expected_tensors(spec)}


def test_expected_tensors_follow_the_layers():
    names = {tensor.name: tuple(tensor.shape) for tensor in expected_tensors(config_from_dict(CONFIG_R).to_spec())}
    assert names["embed"] == (211, 96) and names["head"] == (211, 96) and names["final.norm"] == (96,)
    assert names["loop.step"] == (3, 96) and names["side.embed"] == (211, 40)
    assert names["l0.mix.q"] == (4 * 2 * 16, 96) and names["l0.mix.k"] == (2 * 2 * 16, 96) and names["l0.mix.v"] == (2 * 24, 96)
    assert names["l0.mix.g"] == (4 * 24, 96) and names["l0.mix.o"] == (96, 4 * 24) and names["l0.mix.lq1"] == (16,)
    assert names["l1.mix.q"] == (72, 96) and names["l1.mix.v"] == (120, 96) and names["l1.mix.i"] == (3, 96) and names["l1.mix.f.b"] == (3,)
    assert names["l1.mix.norm"] == (120,) and names["l1.mlp.router"] == (5, 96)
    assert names["l1.mlp.e4.gate"] == (24, 96) and names["l1.mlp.e0.down"] == (96, 24) and names["l1.mlp.shared.up"] == (40, 96)
    assert "l1.mlp.e5.gate" not in names and "l2.mlp.gate" not in names and "l1.norm2" not in names
    assert names["l3.side.gate"] == (10, 96) and names["l3.side.proj"] == (96, 10) and names["l3.side.norm"] == (96,)


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "experts"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "kind"),
    (lambda c: c["loop"].update(stop=5), "stretch"),
    (lambda c: c["loop"].update(start=3, stop=3), "stretch"),
    (lambda c: c.pop("residual_mult"), "residual_mult"),
    (lambda c: c["layers"][3]["mixer"].pop("gate_cap"), "gate_cap"),
])
def test_what_the_configuration_refuses(change, what):
    raw = copy.deepcopy(CONFIG_R)
    change(raw)
    with pytest.raises(EngineError) as caught:
        config_from_dict(raw).to_spec()
    assert what in str(caught.value)


def test_a_memory_head_beyond_the_kernels_registers_is_refused_where_the_model_is_built():
    from tlie_amd.parts.mlstm import MLSTM
    spec = config_from_dict(CONFIG_R).to_spec().layers[1].mixer
    with pytest.raises(EngineError):
        MLSTM(type(spec)("mlstm", {**spec.params, "head_dim": 300}), torch.float32, "cpu")


# ---- the plain implementation's own pieces ---------------------------------------------------------------
def test_plain_rotation_turns_pairs_of_neighbours_and_leaves_the_rest():
    x = torch.arange(1, 13, dtype=torch.float64).reshape(1, 2, 6).repeat(3, 1, 1)
    out = plain.rotate_interleaved(x, torch.tensor([0, 1, 5]), 4, 100.0, 2.0)
    assert torch.equal(out[0], x[0])                                  # position 0: nothing turns
    assert torch.equal(out[:, :, 4:], x[:, :, 4:])                    # the dims past rot.dims pass
    angle = 5 * 100.0 ** (-2.0 / 4) / 2.0                             # pair 1 at position 5
    u, v = x[2, 0, 2], x[2, 0, 3]
    assert math.isclose(float(out[2, 0, 2]), float(u * math.cos(angle) - v * math.sin(angle)), rel_tol=1e-12)
    assert math.isclose(float(out[2, 0, 3]), float(v * math.cos(angle) + u * math.sin(angle)), rel_tol=1e-12)
    assert torch.allclose(out.pow(2).sum(-1), x.pow(2).sum(-1))


def test_plain_memory_carries_its_state_and_starts_its_maximum_at_zero():
    generator = torch.Generator().manual_seed(3)
    mixer = {"heads": 2, "dim": 4, "vdim": 6, "gate_cap": 5.0}
    w = {"q": torch.randn(8, 10, generator=generator), "k": torch.randn(8, 10, generator=generator),
         "v": torch.randn(12, 10, generator=generator), "g": torch.randn(12, 10, generator=generator),
         "o": torch.randn(10, 12, generator=generator), "norm": torch.ones(12), "i": torch.randn(2, 10, generator=generator),
         "i.b": torch.full((2,), -30.0), "f": torch.randn(2, 10, generator=generator), "f.b": torch.randn(2, generator=generator)}
    w = {name: tensor.double() for name, tensor in w.items()}
    h = torch.randn(9, 10, generator=generator, dtype=torch.float64)
    whole, state = plain.mlstm(mixer, w, "", h, 1e-6)
    first, carried = plain.mlstm(mixer, w, "", h[:4], 1e-6)
    second, end = plain.mlstm(mixer, w, "", h[4:], 1e-6, carried)
    assert torch.allclose(torch.cat([first, second]), whole, atol=1e-12) and torch.allclose(end[0], state[0], atol=1e-12)
    # input gates at their floor of -cap: the running maximum stays at its start, 0, minus what is forgotten, never -cap
    assert float(state[2].max()) <= 0.0 and float(state[2].min()) > -5.0 * 9


def test_plain_router_feeds_the_chosen_experts_with_their_scores():
    generator = torch.Generator().manual_seed(4)
    mlp = {"kind": "moe", "expert": {"ff": 3}, "router": {"experts": 4, "top": 2}}
    w = {"router": torch.zeros(4, 5, dtype=torch.float64)}
    w["router"][:, 0] = torch.tensor([3.0, -1.0, 0.5, 2.0], dtype=torch.float64)
    for e in range(4):
        for name, shape in (("gate", (3, 5)), ("up", (3, 5)), ("down", (5, 3))):
            w[f"e{e}.{name}"] = torch.randn(shape, generator=generator, dtype=torch.float64)
    h = torch.zeros(1, 5, dtype=torch.float64)
    h[0, 0], h[0, 1] = 1.0, 0.7
    out = plain.routed_feed_forward(mlp, w, "", h)
    want = sum(plain.gated_feed_forward(w, f"e{e}.", torch.sigmoid(torch.tensor(z, dtype=torch.float64)) * h) for e, z in ((0, 3.0), (3, 2.0)))
    assert torch.allclose(out, want, atol=1e-12)


def test_plain_forward_runs_the_loop_with_its_own_inputs():
    raw = copy.deepcopy(CONFIG_T)
    raw["loop"] = {"start": 0, "stop": 2, "times": 2}
    assert [(layer, t, first) for layer, t, first in plain.layer_runs(raw)] == [(0, 0, True), (1, 0, False), (0, 1, True), (1, 1, False)]
    assert plain.layer_runs(CONFIG_R)[:4] == [(0, None, False), (1, 0, True), (2, 0, False), (1, 1, True)]
