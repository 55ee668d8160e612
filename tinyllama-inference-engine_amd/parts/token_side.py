"""A per-layer token input: after a layer's sublayers, something that depends on the token itself joins the
residual x (float).  With e = table[token][offset .. offset + dim), this layer's part of a table that all layers share:
    g = gelu_tanh(W_gate x) * e,   y = W_proj g,   x += scale * y / sqrt(mean(y^2) + eps) * norm
It runs inside the kernel that brings the residual up to date with the sublayers' results (`ops.residual_update`),
so the part only holds its tensors and hands them over."""
from __future__ import annotations

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
from ..weights.arena import keep_in
from .base import Part


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
        self.offset, self.eps = int(spec["offset"]), float(spec["eps"])
        if self.dim <= 0 or self.offset < 0 or self.offset + self.dim > int(spec["table_width"]):
            raise invalid_config("token_side: the layer's columns do not lie in the table")
        if self.hidden > ops.RESIDUAL_UPDATE_MAX_WIDTH:
            raise invalid_config(f"token_side: widths up to {ops.RESIDUAL_UPDATE_MAX_WIDTH}")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.side = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, dim = int(spec["hidden_size"]), int(spec["dim"])
        return [TensorSpec(prefix + names["gate"], (dim, hidden)), TensorSpec(prefix + names["proj"], (hidden, dim)),
                TensorSpec(prefix + names["norm"], (hidden,), init="norm")]

    def load(self, weights, prefix):
        names = self.names
        table = keep_in(weights, weights[str(self.spec["table"])].contiguous())       # (kept once, under its name, for all layers)
        tensors = [keep_in(weights, weights[prefix + names[role]].to(table.dtype).contiguous()) for role in ("gate", "proj", "norm")]
        self.side = ops.SideInput(table, self.offset, self.dim, *tensors, self.eps)
