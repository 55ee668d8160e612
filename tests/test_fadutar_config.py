"""The Fadutar configuration on the CPU: config.json -> the model as data, the tensors it expects, what it
refuses; and properties of the plain implementation's own pieces."""
import copy
import json
import math
import os

import pytest
import torch

from fadutar_helpers import CONFIG_P, CONFIG_Q, make_model
from plain_fadutar import (plain_causal_conv, plain_clamped_feed_forward, plain_forward, plain_gated_recurrence, plain_rotate_half, plain_sink_softmax,
                           plain_visible)
from tlie_amd.errors import EngineError
from tlie_amd.models.builder import expected_tensors
from tlie_amd.registry import config_from_dict
from tlie_amd.weights.store import WeightStore


def test_the_architecture_is_found_by_its_name_and_turned_into_data():
    spec = config_from_dict(CONFIG_P).to_spec()
    assert spec.architecture == "Fadutar" and spec.max_positions is None
    assert [layer.block for layer in spec.layers] == ["sandwich_norm"] * 7
    assert [layer.mixer.kind for layer in spec.layers] == ["gated_recurrence", "attention", "attention", "latent_attention",
                                                          "attention", "attention", "attention"]
    assert [layer.feed_forward is None for layer in spec.layers] == [True, False, False, False, True, False, True]
    # the layer that reads another layer's keys and values runs on that layer's cache and owns none
    assert [(run.layer, run.cache_of) for run in spec.runs] == [(0, 0), (1, 1), (2, 1), (3, 3), (4, 4), (5, 5), (6, 5)]
    # a cache whose reader sees every earlier position keeps its pages for good, whatever its owner's chunks
    assert spec.layers[5].mixer["chunk"] == 48 and spec.layers[5].mixer["cache_window"] is None
    owner, reader, free = spec.layers[1].mixer, spec.layers[2].mixer, spec.layers[4].mixer
    assert owner["chunk"] == 24 and reader["chunk"] == 40 and free["chunk"] is None
    assert owner["cache_window"] == 40          # kept for as long as the reader's wider chunks reach
    assert free["cache_window"] is None and reader["reads_other_cache"] and not owner["reads_other_cache"]
    assert spec.layers[1].feed_forward["limit"] == 0.75 and spec.layers[2].feed_forward["limit"] == 2.0


def test_expected_tensors_follow_the_layers():
    names = {tensor.name: tuple(tensor.shape) for tensor in expected_tensors(config_from_dict(CONFIG_P).to_spec())}
    assert names["embed"] == (300, 96) and names["head"] == (300, 96) and names["final.norm"] == (96,)
    assert names["l0.mix.ra"] == (2, 64, 64) and names["l0.mix.conv"] == (128, 3) and names["l0.mix.o"] == (96, 128)
    assert "l0.norm2" not in names and "l0.mlp.gate" not in names and names["l0.norm1b"] == (96,)
    assert names["l1.mix.k"] == (48, 96) and names["l1.mix.v"] == (72, 96) and names["l1.mix.o"] == (96, 144)
    assert "l2.mix.k" not in names and "l2.mix.v" not in names and names["l2.mix.q"] == (96, 96) and names["l2.mix.sink"] == (6,)
    assert names["l3.mix.q"] == (96, 96) and names["l3.mix.dkv"] == (48, 96) and names["l3.mix.dkv.norm"] == (40,)
    assert names["l3.mix.uk"] == (72, 40) and names["l3.mix.uv"] == (48, 40) and names["l3.mix.o"] == (96, 48)
    assert names["l1.mlp.gate.b"] == (160,) and names["l1.mlp.down.b"] == (96,)


@pytest.mark.parametrize("change,message", [
    (lambda raw: raw["layers"][2]["mixer"].update(kv_from=2), "earlier layer"),
    (lambda raw: raw["layers"][2]["mixer"].update(kv_from=0), "no keys and values"),
    (lambda raw: raw["layers"][2]["mixer"].update(dim=8), "differs"),
    (lambda raw: raw["layers"][1]["mixer"].update(kv_heads=4), "multiple"),
    (lambda raw: raw["layers"][0].update(type="lstm"), "not one of"),
    (lambda raw: raw["layers"][0]["mixer"].update(blocks=3), "multiple of blocks"),
    (lambda raw: raw["layers"][3]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda raw: raw["layers"][3]["mixer"]["rot"].update(dims=3), "rot.dims"),
    (lambda raw: raw["layers"][1]["mlp"].update(kind="routed"), "dense"),
    (lambda raw: raw["norm"].pop("eps"), "eps"),
    (lambda raw: raw.pop("vocab"), "vocab"),
])
def test_what_the_configuration_refuses(change, message):
    raw = copy.deepcopy(CONFIG_P)
    change(raw)
    with pytest.raises(EngineError, match=message):
        config_from_dict(raw)


def test_a_folder_of_random_weights_is_written_and_validated(tmp_path):
    folder = make_model(tmp_path, CONFIG_Q, seed=3)
    with open(os.path.join(folder, "config.json")) as handle:
        stored = json.load(handle)
    spec = config_from_dict(stored).to_spec()
    WeightStore(folder).validate(expected_tensors(spec))
    logits = plain_forward(stored, {name: WeightStore(folder).get(name).double() for name in WeightStore(folder).names()}, [5, 9, 2])
    assert logits.shape == (3, 131) and bool(torch.isfinite(logits).all())


def test_pieces_of_the_plain_implementation():
    # a token sees its own chunk up to itself, chunks counted from position 0
    assert plain_visible(9, 12, 4).tolist() == [False] * 8 + [True, True] + [False, False]
    assert plain_visible(8, 12, 4).tolist() == [False] * 8 + [True] + [False] * 3
    assert plain_visible(3, 5, None).tolist() == [True, True, True, True, False]
    # the sink takes weight and gives nothing: the weights sum to less than one
    weights = plain_sink_softmax(torch.tensor([0.0, 0.0, 5.0]), torch.tensor([True, True, False]), 0.0)
    assert weights.tolist() == pytest.approx([1 / 3, 1 / 3, 0.0])
    # rotation by position 0 changes nothing, and keeps lengths at any position
    x = torch.randn(3, 2, 8)
    assert torch.allclose(plain_rotate_half(x, torch.zeros(3, dtype=torch.long), 100.0)[0], x[0].double())
    assert torch.allclose(plain_rotate_half(x, torch.tensor([0, 5, 77]), 100.0).norm(dim=-1), x.double().norm(dim=-1))
    # the convolution's last tap is the current token's; before the start there are zeros
    out = plain_causal_conv(torch.tensor([[1.0], [10.0], [100.0]]), torch.tensor([[3.0, 2.0]]), torch.tensor([0.5]))
    assert out[:, 0].tolist() == [2.5, 23.5, 230.5]
    # r = 0 holds the state, whatever comes in
    held = plain_gated_recurrence(torch.tensor([[1.0], [5.0]]), torch.tensor([[1.0], [0.0]]), torch.ones(2, 1), torch.zeros(1))
    assert float(held[1]) == pytest.approx(float(held[0]))


def test_clamped_feed_forward_formula_of_the_oracle():
    """The oracle's own feed-forward against the formula written out for single numbers."""
    w = {"gate": torch.tensor([[2.0]]), "gate.b": torch.tensor([0.5]), "up": torch.tensor([[-3.0]]), "up.b": torch.tensor([0.25]),
         "down": torch.tensor([[1.0]]), "down.b": torch.tensor([0.125])}
    for h in (-2.0, 0.1, 3.0):
        g, u = min(2 * h + 0.5, 0.75), max(-0.75, min(0.75, -3 * h + 0.25))
        want = g / (1 + math.exp(-1.702 * g)) * (u + 1) + 0.125
        assert abs(float(plain_clamped_feed_forward(torch.tensor([[h]], dtype=torch.float64), w, "", 0.75)) - want) < 1e-12
