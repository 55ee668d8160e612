"""A per-layer token input: after a layer's sublayers, something that depends on the token itself joins the
residual x (float).  With e = table[token][offset .. offset + dim), this layer's part of a table that all layers share:
    g = gelu_tanh(W_gate x) * e,   y = W_proj g,   x += scale * y / sqrt(mean(y^2) + eps) * norm
The two products are the framework's products (the first reads the residual, in a bfloat16 run its copy in that
type); y is not added here: it waits, with its norm's weight (times `scale`), as a `NormedDelta`, and whoever
norms the residual next norms it, adds it and norms the sum in one kernel."""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
from ..weights.arena import keep_in
from .base import Part
from .linear import Linear


@register("layer_input", "token_side")
class TokenSide(Part):
    """spec: hidden_size, dim, table (the shared table's full name; the model's spec lists it), table_width, offset (the
    layer's first column of it), eps, scale, names (gate, proj, norm after the prefix).
    Tensors: gate [dim, hidden], proj [hidden, dim], norm [hidden]."""
    graph_safe = True
    NAMES = {"gate": "gate.weight", "proj": "proj.weight", "norm": "norm.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden, self.dim = int(spec["hidden_size"]), int(spec["dim"])
        self.offset, self.eps, self.scale = int(spec["offset"]), float(spec["eps"]), float(spec.get("scale", 1.0))
        if self.dim <= 0 or self.offset < 0 or self.offset + self.dim > int(spec["table_width"]):
            raise invalid_config("token_side: the layer's columns do not lie in the table")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.table = self.gate = self.proj = self.weight = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, dim = int(spec["hidden_size"]), int(spec["dim"])
        return [TensorSpec(prefix + names["gate"], (dim, hidden)), TensorSpec(prefix + names["proj"], (hidden, dim)),
                TensorSpec(prefix + names["norm"], (hidden,), init="norm")]

    def load(self, weights, prefix):
        names, keep = self.names, partial(keep_in, weights)
        self.table = keep(weights[str(self.spec["table"])].contiguous())       # (kept once, under its name, for all layers)
        self.gate = Linear(weights[prefix + names["gate"]], None, self.dtype, keep=keep)
        self.proj = Linear(weights[prefix + names["proj"]], None, self.dtype, keep=keep)
        stored = weights[prefix + names["norm"]]
        # the factor joins the norm's weight once, formed in float and kept in the weight's type (so that the norm that
        # follows, whose weight has that type, can take both in one kernel)
        self.weight = keep((stored.float() * self.scale).to(stored.dtype).contiguous())

    def copy_dtype(self):
        """The type in which `forward` wants the residual: None, the float residual itself; else a copy in that type."""
        return None if self.dtype == torch.float32 else self.dtype

    def forward(self, residual, copy, ctx):
        """residual: float [T, hidden], up to date; copy: the same in `copy_dtype()` (or None).  Returns what joins
        the residual, to be normed first: an `ops.NormedDelta`."""
        pre = ops.as_product(self.gate(copy if copy is not None else residual))
        gated = ops.side_gate(pre, ctx.tokens, self.table, self.offset, self.dtype)
        return ops.NormedDelta(ops.as_product(self.proj(gated)), self.weight, self.eps)
