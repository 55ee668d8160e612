"""What the Fadutar tests share: two small configurations of their own, model folders of random weights,
and the comparison with the plain implementation.

The two configurations differ from each other in every size and option, and use values that make
faults visible: head sizes that differ between keys and values, chunk sizes that are no multiple of the
page size (and differ between a layer and the layer whose keys it reads), a latent rank that differs from
every head size, a recurrence narrower and wider than the model, one and several blocks and taps, layers
without a feed-forward, a limit other than 1, inner sizes that are no multiple of 8.
"""
import json
import os

import torch
from safetensors.torch import load_file

from plain_fadutar import plain_forward


def _mlp(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


CONFIG_P = {
    "architecture": "Fadutar", "vocab": 300, "width": 96, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "rglru", "mixer": {"width": 128, "blocks": 2, "conv": 3}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 3, "dim": 16, "vdim": 24, "scale": 0.3, "mask": {"size": 24}},
         "mlp": _mlp(160, 0.75)},
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 3, "dim": 16, "vdim": 24, "scale": 0.2, "mask": {"size": 40},
                                        "kv_from": 1}, "mlp": _mlp(64, 2.0)},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 24, "rot_dim": 8, "vdim": 16, "kv_rank": 40, "scale": 0.17,
                                               "rot": {"base": 10000.0, "dims": 8}}, "mlp": _mlp(160, 0.75)},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 72, "vdim": 8, "scale": 0.1}, "mlp": None},
        # one head size for keys and values, a multiple of 16: in bfloat16 these two take the kernel on the matrix cores
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.2, "mask": {"size": 48}},
         "mlp": _mlp(64, 2.0)},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.15, "kv_from": 5}, "mlp": None},
    ],
}
CONFIG_Q = {
    "architecture": "Fadutar", "vocab": 131, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "latent_attention", "mixer": {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 80, "kv_rank": 16, "scale": 0.25,
                                               "rot": {"base": 500.0, "dims": 4}}, "mlp": None},
        {"type": "rglru", "mixer": {"width": 64, "blocks": 1, "conv": 1}, "mlp": _mlp(40, 0.5)},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 1, "dim": 9, "vdim": 5, "scale": 0.4, "mask": {"size": 7}},
         "mlp": _mlp(72, 1.5)},
        {"type": "rglru", "mixer": {"width": 48, "blocks": 3, "conv": 5}, "mlp": _mlp(40, 0.5)},
        # of the rotated part's 12 dims only the first 8 turn
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 16, "rot_dim": 12, "vdim": 8, "kv_rank": 20, "scale": 0.2,
                                               "rot": {"base": 50.0, "dims": 8}}, "mlp": _mlp(40, 0.5)},
    ],
}
CONFIGS = {"P": CONFIG_P, "Q": CONFIG_Q}
DTYPES = ["float32", "bfloat16"]
# a row's largest error relative to the row's largest value, against float64 on the same stored weights
TOLERANCE = {"float32": 3e-5, "bfloat16": 3e-2}
# two cuts of the same request through the same engine
CUT_TOLERANCE = {"float32": 2e-6, "bfloat16": 4e-2}


def make_model(folder, raw_config, seed, std=0.08, norm_std=0.1):
    """Weights are stored in bfloat16, as the design's files are: a float32 run widens the same values."""
    from tlie_amd import write_random_model
    from tlie_amd.registry import config_from_dict
    write_random_model(str(folder), config_from_dict(raw_config), seed, std=std, norm_std=norm_std, dtype=torch.bfloat16)
    return str(folder)


def load_plain(folder):
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        raw = json.load(handle)
    weights = {name: tensor.double() for name, tensor in load_file(os.path.join(folder, "model.safetensors")).items()}
    return raw, weights


def plain_logits(folder, tokens):
    raw, weights = load_plain(folder)
    return plain_forward(raw, weights, list(tokens))


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).abs().amax(dim=-1) / want.abs().amax(dim=-1)


def run_cut(engine, request, tokens, cuts, want_all=True):
    """The request's tokens in portions of the sizes `cuts` (repeated as needed); returns logits [T, vocab]."""
    from tlie_amd import StepEntry
    engine.admit(request)
    rows, at, index = [], 0, 0
    while at < len(tokens):
        count = min(cuts[index % len(cuts)], len(tokens) - at)
        rows.append(engine.step([StepEntry(request, tokens[at:at + count], list(range(count)))]).clone())
        at += count
        index += 1
    engine.finish(request)
    return torch.cat(rows, dim=0)
