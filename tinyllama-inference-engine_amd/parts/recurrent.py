"""A recurrent mixer: a gated linear recurrence behind a short causal convolution, beside a gate branch.

Per token, from the mixer's input h, with `width` channels:
    y = gelu_tanh(W_y h + b_y)                                  the gate branch
    u = conv(W_x h + b_x)                                       causal, per channel, `taps` taps, zeros before the start
    r = sigmoid(R u + b_r),  i = sigmoid(I u + b_i)             R and I block-diagonal: the channels in `blocks` parts
    a = exp(-decay * r * softplus(lambda))
    S_t = a * S_(t-1) + sqrt(1 - a^2) * (i * u)                 S = 0 before the first token
    out = W_o (S * y)
What a request carries from token to token is S and the convolution's last taps - 1 inputs: a row of
[taps, width] floats in the cache manager's state area, zeroed when the request is admitted.  The two
projections are one product; the convolution, the gates' sigmoids, the decay and the state are float whatever
the activation type.  The gates' products have float sums; in a bfloat16 step of many rows they run on the matrix
cores, whose operands are bfloat16 (u is rounded as it becomes one; the u that drives the state stays float).
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


@register("mixer", "gated_recurrence")
class GatedRecurrence(Mixer):
    """spec: hidden_size, width (channels), blocks (of the gates' matrices), taps (of the convolution),
    decay (the constant in log a = -decay * r * softplus(lambda)), names (the tensors' names after the
    prefix, by role).
    Tensors: gate_branch and input [width, hidden] with biases [width]; conv [width, taps], conv_bias [width];
    recurrence_gate and input_gate [blocks, width / blocks, width / blocks] ([out, in] per block) with biases
    [blocks, width / blocks]; decay (lambda) [width]; o [hidden, width]."""
    graph_safe = True
    NAMES = {"gate_branch": "linear_y.weight", "gate_branch_bias": "linear_y.bias", "input": "linear_x.weight",
             "input_bias": "linear_x.bias", "conv": "conv_1d.weight", "conv_bias": "conv_1d.bias",
             "recurrence_gate": "rg_lru.recurrent_gate_weight", "recurrence_gate_bias": "rg_lru.recurrent_gate_bias",
             "input_gate": "rg_lru.input_gate_weight", "input_gate_bias": "rg_lru.input_gate_bias",
             "decay": "rg_lru.recurrent_param", "o": "linear_out.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.width = int(spec["width"])
        self.blocks = int(spec["blocks"])
        self.taps = int(spec["taps"])
        self.decay = float(spec.get("decay", 8.0))
        if min(self.width, self.blocks, self.taps) <= 0 or self.width % self.blocks != 0:
            raise invalid_config("gated_recurrence: width must be a positive multiple of blocks, taps positive")
        self.block_width = self.width // self.blocks
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.first = self.o = self.conv = self.conv_bias = self.gates_t = self.gate_bias = self.lam = self.gates_rows = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, width, blocks, taps = int(spec["hidden_size"]), int(spec["width"]), int(spec["blocks"]), int(spec["taps"])
        inside = width // blocks
        shapes = (("gate_branch", (width, hidden)), ("gate_branch_bias", (width,)), ("input", (width, hidden)),
                  ("input_bias", (width,)), ("conv", (width, taps)), ("conv_bias", (width,)),
                  ("recurrence_gate", (blocks, inside, inside)), ("recurrence_gate_bias", (blocks, inside)),
                  ("input_gate", (blocks, inside, inside)), ("input_gate_bias", (blocks, inside)),
                  ("decay", (width,)), ("o", (hidden, width)))
        return [TensorSpec(prefix + names[role], shape) for role, shape in shapes]

    def load(self, weights, prefix):
        names, keep = self.names, partial(keep_in, weights)

        def get(role):
            return weights[prefix + names[role]]
        # one product for both branches: the gate branch's columns first, then the convolution's inputs
        self.first = Linear(torch.cat([get("gate_branch"), get("input")], dim=0),
                            torch.cat([get("gate_branch_bias"), get("input_bias")], dim=0), self.dtype, keep=keep)
        self.conv, self.conv_bias = keep(get("conv").contiguous()), keep(get("conv_bias").contiguous())
        # both gates of a block as one matrix [inner, 2 * inside]: r's outputs, then i's (stored [out, in] per block)
        self.gates_t = keep(torch.cat([get("recurrence_gate").transpose(1, 2), get("input_gate").transpose(1, 2)], dim=2).contiguous())
        self.gate_bias = keep(torch.cat([get("recurrence_gate_bias"), get("input_gate_bias")], dim=1).contiguous())
        # and as the product on the matrix cores wants them (steps of many rows, bfloat16): [2 * inside, inner] a block
        self.gates_rows = None
        if self.dtype == torch.bfloat16 and self.gates_t.dtype == torch.bfloat16:
            self.gates_rows = keep(torch.cat([get("recurrence_gate"), get("input_gate")], dim=1).contiguous())
        self.lam = keep(get("decay").contiguous())
        self.o = Linear(get("o"), None, self.dtype, keep=keep)

    def state_need(self):
        """Rows 0 .. taps-2: the convolution's last inputs, oldest first; row taps-1: S."""
        return StateNeed((self.taps, self.width), torch.float32)

    def forward(self, x, ctx, binding: Binding, into=None):
        fused = ops.as_product(self.first(x))
        tokens, width = fused.rows, self.width
        u = ops.causal_conv(fused, width, self.conv, self.conv_bias, binding.state, ctx.token_seq, ctx.token_slot, ctx.seq_start)
        gates = torch.empty((tokens, 2 * width), dtype=torch.float32, device=u.device)
        ops.block_linear(u, 0, width, self.block_width, self.gates_t, self.gate_bias,
                         gates, 0, 2 * width, 2 * self.block_width, tokens, weight=self.gates_rows)
        mixed = ops.gated_recurrence(fused, width, 0, u, gates, self.lam, self.decay, binding.state, ctx.seq_start, ctx.seq_slot,
                                     self.block_width, self.dtype, max_new=ctx.max_new)
        return self.o(mixed)
