"""A routed feed-forward: a router scores the experts for every token, the token uses the `top` best, and an
expert that every token uses may run beside them.

    z = W_router x (float sums),  s = sigmoid(z)
    the `top` experts with the largest s are the token's; each is fed with s_e * x:
    out = sum over them of down_e(silu(gate_e(s_e x)) * up_e(s_e x))  +  shared(x)
(the scores are not renormalized, and weigh the expert's input, not its result).

All experts' gate and up matrices are one matrix, their rows side by side expert by expert (g0 u0 g1 u1 ...), the
shared expert's last, and all down matrices are one matrix along the inner index: the feed-forward is then two
products around a gate kernel that multiplies an expert's columns by the token's score for it, which is zero for an
expert that the token does not use (silu(0) * 0 adds nothing to the second product, exactly).  Since the products
are linear, s (W x) stands for W (s x).
"""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
from ..weights.arena import keep_in
from .base import FeedForward
from .linear import Linear


@register("feed_forward", "routed_mlp")
class RoutedMLP(FeedForward):
    """spec: hidden_size, experts, top, expert_size, shared_size (0: no shared expert), score ("sigmoid"),
    renormalize (False), weigh ("input"), names (router, expert: a pattern with {} for the expert's number, shared,
    gate, up, down).
    Tensors: router [experts, hidden]; per expert and for the shared one gate, up [size, hidden], down [hidden, size]."""
    graph_safe = True
    NAMES = {"router": "router.weight", "expert": "experts.{}.", "shared": "shared_expert.", "gate": "gate_proj.weight",
             "up": "up_proj.weight", "down": "down_proj.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.experts, self.top = int(spec["experts"]), int(spec["top"])
        self.expert_size, self.shared_size = int(spec["expert_size"]), int(spec.get("shared_size", 0))
        if min(self.experts, self.top, self.expert_size) <= 0 or self.top > self.experts or self.shared_size < 0:
            raise invalid_config("routed_mlp: experts, top (at most experts) and expert_size must be positive")
        if spec.get("score", "sigmoid") != "sigmoid" or spec.get("renormalize", False) or spec.get("weigh", "input") != "input":
            raise invalid_config("routed_mlp: implemented are sigmoid scores that are not renormalized and weigh the expert's input")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.router = self.gate_up = self.down = None

    @classmethod
    def _prefixes(cls, spec, prefix, names):
        places = [prefix + names["expert"].format(e) for e in range(int(spec["experts"]))]
        sizes = [int(spec["expert_size"])] * len(places)
        if int(spec.get("shared_size", 0)) > 0:
            places.append(prefix + names["shared"])
            sizes.append(int(spec["shared_size"]))
        return list(zip(places, sizes))

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden = int(spec["hidden_size"])
        specs = [TensorSpec(prefix + names["router"], (int(spec["experts"]), hidden))]
        for place, size in cls._prefixes(spec, prefix, names):
            specs += [TensorSpec(place + names["gate"], (size, hidden)), TensorSpec(place + names["up"], (size, hidden)),
                      TensorSpec(place + names["down"], (hidden, size))]
        return specs

    def load(self, weights, prefix):
        names, keep = self.names, partial(keep_in, weights)
        self.router = keep(weights[prefix + names["router"]].contiguous())
        rows, columns = [], []
        for place, size in self._prefixes(self.spec, prefix, names):
            gate, up = weights[place + names["gate"]], weights[place + names["up"]]
            rows.append(torch.stack([gate, up], dim=1).reshape(2 * size, self.hidden))
            columns.append(weights[place + names["down"]])
        self.gate_up = Linear(torch.cat(rows, dim=0).contiguous(), None, self.dtype, keep=keep)
        self.down = Linear(torch.cat(columns, dim=1).contiguous(), None, self.dtype, keep=keep)

    def forward(self, x, ctx, into=None):
        scale = ops.few_outputs(x, self.router, top=self.top)
        hidden = ops.routed_gate(ops.as_product(self.gate_up(x)), scale, self.expert_size, self.dtype)
        return self.down(hidden)
