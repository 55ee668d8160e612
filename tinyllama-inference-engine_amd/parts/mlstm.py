"""The mLSTM mixer: a matrix memory per head, written with an input gate and forgotten with a forget gate, both
exponential and kept in range by a running maximum.

Per token and head, from the mixer's input x (dim = head_dim, vdim = value_dim):
    q = W_q x * dim^(-1/2),  k = W_k x,  v = W_v x
    i = cap * tanh((W_i x + b_i) / cap)                       log input gate
    f = logsigmoid(cap * tanh((W_f x + b_f) / cap))           log forget gate
    m' = max(f + m, i)                                        m = 0 before the first token
    S' = exp(f + m - m') S + exp(i - m') k v^T                S = 0 before the first token (dim x vdim)
    n' = exp(f + m - m') n + exp(i - m') k                    n = 0 before the first token
    o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
    out = W_o (o / sqrt(mean(o^2) + eps) (per head) * norm * sigmoid(W_g x))
What a request carries from token to token is S, n and m of every head: a row of floats in the cache manager's
state area, zero when the request is admitted.  q, k, v and the output gate are one product; the two gates'
pre-activations are a product with float sums of their own, and the gates, the memory and the heads' norm are
float whatever the activation type.
"""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
from ..weights.arena import keep_in
from .base import Binding, Mixer, StateNeed
from .linear import Linear


@register("mixer", "mlstm")
class MLSTM(Mixer):
    """spec: hidden_size, num_heads, head_dim, value_dim, gate_cap, norm_eps, names (the tensors' names after the
    prefix, by role).
    Tensors: q and k [heads * head_dim, hidden]; v and gate [heads * value_dim, hidden]; input_gate and forget_gate
    [heads, hidden] with biases [heads]; norm [heads * value_dim]; o [hidden, heads * value_dim]."""
    graph_safe = True
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "gate": "ogate_proj.weight",
             "o": "out_proj.weight", "norm": "outnorm.weight", "input_gate": "igate.weight", "input_gate_bias": "igate.bias",
             "forget_gate": "fgate.weight", "forget_gate_bias": "fgate.bias"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.heads, self.d, self.dv = int(spec["num_heads"]), int(spec["head_dim"]), int(spec["value_dim"])
        self.cap, self.eps = float(spec["gate_cap"]), float(spec["norm_eps"])
        if min(self.heads, self.d, self.dv) <= 0 or not self.cap > 0.0:
            raise invalid_config("mlstm: heads, head_dim, value_dim and gate_cap must be positive")
        if self.d > ops.MLSTM_MAX_DIM:
            raise invalid_config(f"mlstm: head_dim {self.d} is beyond what the kernel keeps in registers ({ops.MLSTM_MAX_DIM})")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.fused = self.o = self.gates = self.gate_bias = self.norm = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, heads, d, dv = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"]), int(spec["value_dim"])
        shapes = (("q", (heads * d, hidden)), ("k", (heads * d, hidden)), ("v", (heads * dv, hidden)),
                  ("gate", (heads * dv, hidden)), ("o", (hidden, heads * dv)), ("input_gate", (heads, hidden)),
                  ("forget_gate", (heads, hidden)))
        specs = [TensorSpec(prefix + names[role], shape) for role, shape in shapes]
        specs += [TensorSpec(prefix + names["input_gate_bias"], (heads,), init="zeros"),
                  TensorSpec(prefix + names["forget_gate_bias"], (heads,), init="forget_bias")]
        specs.append(TensorSpec(prefix + names["norm"], (heads * dv,), init="norm"))
        return specs

    def load(self, weights, prefix):
        names, keep = self.names, partial(keep_in, weights)

        def get(role):
            return weights[prefix + names[role]]
        self.fused = Linear(torch.cat([get("q"), get("k"), get("v"), get("gate")], dim=0).contiguous(), None, self.dtype, keep=keep)
        # both gates' pre-activations as one product of 2 * heads outputs: the input gates, then the forget gates
        self.gates = keep(torch.cat([get("input_gate"), get("forget_gate")], dim=0).contiguous())
        self.gate_bias = keep(torch.cat([get("input_gate_bias"), get("forget_gate_bias")], dim=0).to(self.gates.dtype).contiguous())
        self.norm = keep(get("norm").contiguous())
        self.o = Linear(get("o"), None, self.dtype, keep=keep)

    def state_need(self):
        return StateNeed(ops.mlstm_state_shape(self.heads, self.d, self.dv), torch.float32)

    def forward(self, x, ctx, binding: Binding, into=None):
        fused = ops.as_product(self.fused(x))
        gates = ops.few_outputs(x, self.gates, self.gate_bias)
        keys, values = self.heads * self.d, self.heads * self.dv
        memory = ops.mlstm_scan(fused, 0, keys, 2 * keys, gates, binding.state, ctx.seq_start, ctx.seq_slot, self.heads, self.d,
                                self.dv, self.cap, float(self.d) ** -0.5, max_new=ctx.max_new)
        normed = ops.head_combine(memory, self.heads, self.dv, self.eps, self.dtype, weight=self.norm, gate=fused,
                                  gate_col=2 * keys + values)
        return self.o(normed)
