"""Differential attention over the paged cache: every head holds two maps of attention over the same values,
and what the head gives is their difference.

Per head h (with key/value group g = h // (heads / groups)), from the mixer's input x:
    q1, q2 = two queries of `head_dim`, k1, k2 = two keys of the group, v = one value of `value_dim` of the group
    a_m = softmax over the visible keys of (q_m . k_m) * scale, times v                (m = 1, 2; causal)
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff                                    (one number for the layer)
    o = a_1 - lambda * a_2,  o / sqrt(mean(o^2) + eps) * (1 - diff)                    (no weight)
    out = W_o (concat(o) * sigmoid(W_g x))                                             (the gate is optional)
q and k are rotated (if the layer has a rotation table) before they are used or cached.

The two maps are two heads of an ordinary attention whose key heads come in pairs that read one value head: the
layer runs as an attention of 2 * heads query heads over 2 * groups key heads and `groups` value heads, through
the attention kernel, and a kernel of its own forms the difference, the norm and the gate.  Its results leave the
attention kernel as floats, because their difference is normed.  A page of the cache holds the 2 * groups
planes of keys [row][dim] and after them the `groups` planes of values, transposed, [dim][row].  In bfloat16,
with values a multiple of the keys' size, the kernel on the matrix cores reads the same pages: it takes a value
head as so many pieces of the keys' size, each a head of its own whose scores are those of its map.  The four
projections (q, k, v and the gate) are one product.
"""
from __future__ import annotations

import math
from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import lookup, register
from ..weights.arena import keep_in
from .base import Binding, CacheNeed, Mixer
from .linear import Linear


@register("mixer", "differential_attention")
class DifferentialAttention(Mixer):
    """spec: hidden_size, num_heads, num_kv_heads, head_dim (of a query or key of one map), value_dim, scale (default
    1 / sqrt(head_dim)), diff, norm_eps, output_gate (bool), position (a PartSpec: a rotation table or none), pairing
    ("interleaved": dims 2i and 2i + 1 of a rotated part turn together; "halves": dims i and i + rot_dim / 2), names.
    Tensors: q [heads * 2 * head_dim, hidden] and k [kv_heads * 2 * head_dim, hidden], head by head [map 1, map 2];
    v [kv_heads * value_dim, hidden]; gate [heads * value_dim, hidden] (if output_gate); o [hidden, heads * value_dim];
    lambda_q1, lambda_k1, lambda_q2, lambda_k2 [head_dim]."""
    graph_safe = True
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "gate": "g_proj.weight",
             "lambda_q1": "lambda_q1", "lambda_k1": "lambda_k1", "lambda_q2": "lambda_q2", "lambda_k2": "lambda_k2"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.heads, self.groups = int(spec["num_heads"]), int(spec["num_kv_heads"])
        self.d, self.dv = int(spec["head_dim"]), int(spec["value_dim"])
        if self.heads <= 0 or self.groups <= 0 or self.heads % self.groups != 0:
            raise invalid_config("differential_attention: num_heads must be a positive multiple of num_kv_heads")
        if not 0 < self.d <= 4096 or not 0 < self.dv <= ops.ATTENTION_MAX_HEAD_DIM:
            raise invalid_config(f"differential_attention: value heads of 1 to {ops.ATTENTION_MAX_HEAD_DIM} dims")
        self.scale = float(spec["scale"]) if spec.get("scale") is not None else 1.0 / math.sqrt(float(self.d))
        self.diff = float(spec["diff"])
        self.eps = float(spec["norm_eps"])
        self.output_gate = bool(spec.get("output_gate", False))
        self.pairing = spec.get("pairing", "halves")
        if self.pairing not in ("interleaved", "halves"):
            raise invalid_config(f"differential_attention: pairing '{self.pairing}' is not 'interleaved' or 'halves'")
        if not (self.scale > 0.0 and math.isfinite(self.scale)):
            raise invalid_config("differential_attention: the scale of the scores must be positive")
        position = spec.get("position") or PartSpec("none")
        self.position = lookup("position_encoding", position.kind)(position, dtype, device)
        if self.position.rotary_table() is None and position.kind != "none":
            raise invalid_config("differential_attention: positions are a rotation table or none")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.per_group = self.heads // self.groups
        self.fused = self.o = None
        self.pair_lambda = 0.0

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, heads, groups = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["num_kv_heads"])
        d, dv = int(spec["head_dim"]), int(spec["value_dim"])
        shapes = [("q", (heads * 2 * d, hidden)), ("k", (groups * 2 * d, hidden)), ("v", (groups * dv, hidden))]
        if spec.get("output_gate", False):
            shapes.append(("gate", (heads * dv, hidden)))
        shapes.append(("o", (hidden, heads * dv)))
        shapes += [(role, (d,)) for role in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2")]
        return [TensorSpec(prefix + names[role], shape) for role, shape in shapes]

    def _row_order(self):
        """The order in which the stored rows of q and of k go into the fused matrix.  Queries: those of one key head
        (a group's map) side by side, which is how the attention kernel finds a query head's key head.  Within a
        head, interleaved rotation pairs are brought to the kernels' order, first elements, then second elements:
        a score is a sum over dims and does not change when q and k are reordered alike."""
        d = self.d
        table = self.position.rotary_table()
        inside = list(range(d))
        if table is not None and self.pairing == "interleaved":
            rot = table[1]
            inside = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, d))
        q_rows = []
        for group in range(self.groups):
            for which in range(2):
                for i in range(self.per_group):
                    head = group * self.per_group + i
                    q_rows += [(head * 2 + which) * d + e for e in inside]
        k_rows = [key_head * d + e for key_head in range(2 * self.groups) for e in inside]
        return torch.tensor(q_rows, dtype=torch.long), torch.tensor(k_rows, dtype=torch.long)

    def load(self, weights, prefix):
        names, keep = self.names, partial(keep_in, weights)

        def get(role):
            return weights[prefix + names[role]]
        q_rows, k_rows = self._row_order()
        parts = [get("q")[q_rows.to(self.device)], get("k")[k_rows.to(self.device)], get("v")]
        if self.output_gate:
            parts.append(get("gate"))
        self.fused = Linear(torch.cat(parts, dim=0).contiguous(), None, self.dtype, keep=keep)
        self.o = Linear(get("o"), None, self.dtype, keep=keep)
        # one number for the layer, formed once, in float
        first = float((get("lambda_q1").float() * get("lambda_k1").float()).sum().item())
        second = float((get("lambda_q2").float() * get("lambda_k2").float()).sum().item())
        self.pair_lambda = math.exp(first) - math.exp(second) + self.diff

    def cache_need(self):
        return CacheNeed((self.groups,), 2 * self.d + self.dv, None)

    def forward(self, x, ctx, binding: Binding, into=None):
        pages = ctx.groups[binding.group]
        fused = ops.as_product(self.fused(x))
        table = self.position.rotary_table()
        inv_freq, rot_dim = table if table is not None else (None, 0)
        heads, key_heads = 2 * self.heads, 2 * self.groups
        gate_cols = self.heads * self.dv if self.output_gate else 0
        q = ops.qkv_place(fused, ctx.positions, pages.slot_map if binding.writes else ctx.no_slots, inv_freq, rot_dim,
                          binding.cache, heads, key_heads, self.d, self.dv, self.dtype, value_heads=self.groups,
                          extra_cols=gate_cols)
        page_size = binding.cache.shape[2] // (2 * self.d + self.dv)
        parts = 1
        if self.dv % self.d == 0 and self.dv // self.d <= 64 and ops.attention_mfma_takes(self.dtype, self.d, page_size):
            # bfloat16, values a multiple of the keys' size: the kernel on the matrix cores.  A value head's pieces of
            # the keys' size are kv heads of that kernel: key head k and piece p make kv head k * parts + p, which reads
            # key plane k and, with its map's partner, the group's value planes
            parts = self.dv // self.d
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, self.per_group, key_heads * parts, self.d)
            attended = ops.attention_mfma(q, binding.cache, pages.block_table, tiles, ctx.positions, heads * parts, key_heads * parts,
                                          self.d, None, self.scale, nsplit, split_len, col_tiles, waves, shared,
                                          planes=(parts, 2 * parts, parts), float_out=True)
        else:
            attended = ops.attention_generic(q, binding.cache, pages.block_table, ctx.token_seq, ctx.positions, heads, key_heads,
                                             self.d, None, self.scale, tiled=ops.attention_generic_plan(ctx, self.d, self.dv),
                                             seq_start=ctx.seq_start, value_dim=self.dv, value_heads=self.groups, float_out=True)
        combined = ops.head_combine(attended, self.heads, self.dv, self.eps, self.dtype, pair_group=self.per_group,
                                    pair_lambda=self.pair_lambda, mult=1.0 - self.diff,
                                    gate=fused if self.output_gate else None, gate_col=fused.cols - gate_cols, parts=parts)
        return self.o(combined)
