"""What the Raketar tests share: configurations of their own, model folders of random weights, and the
comparison with the plain implementation.

The configurations differ from each other in every size and option, and use values that make faults visible:
fewer key/value groups than heads, value heads below and above 64 dims and of no multiple of 64, rotations over
a part of a head and over all of it, with and without a scaling factor, memory heads of 24, 72 and 160 query dims,
several experts a token (up to all of them), with and without a shared expert, layers without a feed-forward,
a loop that starts after the first layer and runs three times, one of a single layer, and no loop at all, a model
without the per-layer token input, inner sizes that are no multiple of 8.
"""
import json
import os

import torch
from safetensors.torch import load_file

import plain_raketar


def _attention(heads, groups, dim, vdim, scale, diff, rot):
    return {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff, "rot": rot}


def _moe(experts, top, ff, shared):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


CONFIG_R = {
    "architecture": "Raketar", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
    "token_side": {"dim": 10}, "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "attention", "mixer": _attention(4, 2, 16, 24, 0.3, 0.3, {"base": 1000.0, "dims": 8, "scaling": {"factor": 2.0}}),
         "mlp": {"kind": "dense", "ff": 72}},
        {"type": "mlstm", "mixer": {"heads": 3, "dim": 24, "vdim": 40, "gate_cap": 10.0}, "mlp": _moe(5, 2, 24, 40)},
        {"type": "attention", "mixer": _attention(6, 1, 8, 80, 0.25, 0.8, {"base": 50.0, "dims": 8}), "mlp": None},
        {"type": "mlstm", "mixer": {"heads": 2, "dim": 72, "vdim": 130, "gate_cap": 4.0}, "mlp": {"kind": "dense", "ff": 36}},
    ],
}
CONFIG_S = {
    "architecture": "Raketar", "vocab": 150, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "loop": {"start": 0, "stop": 1, "times": 2},
    "layers": [
        {"type": "mlstm", "mixer": {"heads": 1, "dim": 160, "vdim": 16, "gate_cap": 15.0}, "mlp": _moe(3, 3, 16, 0)},
        {"type": "attention", "mixer": _attention(2, 2, 32, 32, 0.18, 0.5, {"base": 250000.0, "dims": 32, "scaling": {"factor": 8.0}}),
         "mlp": _moe(8, 1, 12, 20)},
        {"type": "attention", "mixer": _attention(3, 3, 6, 5, 0.4, 0.1, {"base": 10.0, "dims": 2}), "mlp": {"kind": "dense", "ff": 40}},
    ],
}
CONFIG_T = {        # no loop; a single layer of each kind
    "architecture": "Raketar", "vocab": 64, "width": 32, "norm": {"eps": 1e-5}, "residual_mult": 0.25, "token_side": {"dim": 3},
    "layers": [
        {"type": "mlstm", "mixer": {"heads": 2, "dim": 8, "vdim": 70, "gate_cap": 6.0}, "mlp": None},
        # values twice as wide as the keys, both multiples of 16: in bfloat16 this layer takes the kernel on the matrix cores
        {"type": "attention", "mixer": _attention(4, 2, 16, 32, 0.3, 0.6, {"base": 100.0, "dims": 4, "scaling": {"factor": 1.5}}),
         "mlp": _moe(4, 2, 8, 8)},
    ],
}
CONFIGS = {"R": CONFIG_R, "S": CONFIG_S, "T": CONFIG_T}
DTYPES = ["float32", "bfloat16"]
# a row's largest error relative to the row's largest value, against float64 on the same stored weights.  A memory
# layer divides by max(|n . q|, exp(-m)), a sum with cancellation: one rounding of such a layer's input to bfloat16
# alone moves a row of these models' logits by up to 2e-2, and rounding every norm's output by up to 3e-2 (measured
# on the plain implementation); the engine rounds five times a sublayer.  The sharp comparison is the 32-bit one.
TOLERANCE = {"float32": 3e-5, "bfloat16": 1.5e-1}
SINGLE_LAYER_TOLERANCE = {"float32": 3e-5, "bfloat16": 2e-2}
# two cuts of the same request through the same engine (in bfloat16 a step of few rows takes other product kernels
# than a step of many, whose results are rounded to bfloat16 where the others' stay float partial sums)
# (in 32-bit too a cut changes the order of sums: a sequence that brings many tokens takes the memory's sliced walk)
CUT_TOLERANCE = {"float32": 1e-5, "bfloat16": 1.5e-1}


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


def plain_generate_greedy(config, weights, prompt, count):
    tokens, out = list(prompt), []
    for _ in range(count):
        token = int(torch.argmax(plain_raketar.forward(config, weights, tokens)[0][-1]))
        out.append(token)
        tokens.append(token)
    return out


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).abs().amax(dim=-1) / want.abs().amax(dim=-1)


def run_cut(engine, request, tokens, cuts):
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
