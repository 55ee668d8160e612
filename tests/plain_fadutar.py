"""A plain, slow implementation of the Fadutar decoder, used only as the tests' oracle.

Every function works on one whole sequence, keeps no cache and no state between calls, and shares
no code with the engine: one function per mechanism, each straight from its equation.  Arithmetic
is float64, except the rotation's angle, which is formed in 32-bit (position times frequency, the
frequency a 32-bit power) and only then widened: the angle is what the formula means.

The design in short.  A layer is x += post1(mixer(pre1(x))), then, if it has a feed-forward,
x += post2(ff(pre2(x))); all four norms are RMS norms whose stored weight w acts as (1 + w).
Mixers: softmax attention with a learned sink per head in the denominator, either grouped-query
attention without positions inside chunks of positions (a layer may read another layer's keys and
values), or latent attention (keys and values expanded from one low-rank vector per position, plus
one rotated key part shared by all heads); and a gated linear recurrence behind a short causal
convolution.  The feed-forward is a clamped, gated one with biases.
"""
from __future__ import annotations

import math

import torch


# ---- norms ----------------------------------------------------------------------------------------
def plain_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = x.double()
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def plain_offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose weight is stored around zero: rms(x) * (1 + w)."""
    return plain_rms(x, eps) * (1.0 + w.double())


def plain_weight_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm with a plain weight: rms(x) * w."""
    return plain_rms(x, eps) * w.double()


# ---- small functions --------------------------------------------------------------------------------
def plain_gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    z = z.double()
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def plain_sink_softmax(scores: torch.Tensor, visible: torch.Tensor, sink: float) -> torch.Tensor:
    """Weights over the keys of one query row.  scores [keys], visible [keys] bool; the
    denominator holds exp(sink) once more than the visible keys' exponentials."""
    scores = scores.double()
    top = max(float(scores[visible].max()) if bool(visible.any()) else -math.inf, float(sink))
    weights = torch.where(visible, torch.exp(scores - top), torch.zeros_like(scores))
    return weights / (weights.sum() + math.exp(float(sink) - top))


def plain_rotate_half(x: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """x [T, ..., dims]: element i pairs with i + dims/2; the pair (u, v) at position p turns by
    p * base^(-2i/dims)."""
    dims = x.shape[-1]
    half = dims // 2
    frequency = torch.pow(torch.tensor(base, dtype=torch.float32), -2.0 * torch.arange(half, dtype=torch.float32) / dims)
    angle = (positions.to(torch.float32)[:, None] * frequency[None, :]).double()
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(angle).reshape(shape), torch.sin(angle).reshape(shape)
    x = x.double()
    u, v = x[..., :half], x[..., half:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin], dim=-1)


def plain_linear(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None = None) -> torch.Tensor:
    out = x.double() @ w.double().T
    return out if b is None else out + b.double()


# ---- attention --------------------------------------------------------------------------------------
def plain_visible(query: int, keys: int, chunk: int | None) -> torch.Tensor:
    """Which of the positions 0..keys-1 the query at position `query` sees: those not after it,
    and, with chunks, only those of its own chunk (chunks counted from position 0)."""
    j = torch.arange(keys)
    seen = j <= query
    if chunk is not None:
        seen &= (j // chunk) == (query // chunk)
    return seen


def plain_sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sink: torch.Tensor, scale: float,
                         chunk: int | None = None) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv], sink [H] -> [T, H, dv].  Query head h reads key/value
    head h // (H / G)."""
    tokens, heads, _ = q.shape
    per_group = heads // k.shape[1]
    out = torch.zeros((tokens, heads, v.shape[-1]), dtype=torch.float64)
    q, k, v = q.double(), k.double(), v.double()
    for t in range(tokens):
        seen = plain_visible(t, tokens, chunk)
        for h in range(heads):
            g = h // per_group
            weights = plain_sink_softmax((k[:, g] @ q[t, h]) * scale, seen, float(sink[h]))
            out[t, h] = weights @ v[:, g]
    return out


def plain_keys_values(h: torch.Tensor, w: dict, prefix: str, kv_heads: int, dim: int, vdim: int):
    """The keys and values a chunked-attention layer makes of its input (no positions enter)."""
    tokens = h.shape[0]
    return (plain_linear(h, w[prefix + "k"]).reshape(tokens, kv_heads, dim),
            plain_linear(h, w[prefix + "v"]).reshape(tokens, kv_heads, vdim))


def plain_attention_mixer(h: torch.Tensor, w: dict, prefix: str, mixer: dict, keys_values=None):
    """Returns (output [T, width], (k, v)): `keys_values` given, the layer uses them (another layer's)
    with its own queries, mask, sink and output projection."""
    tokens = h.shape[0]
    heads, dim, vdim = mixer["heads"], mixer["dim"], mixer["vdim"]
    if keys_values is None:
        keys_values = plain_keys_values(h, w, prefix, mixer["kv_heads"], dim, vdim)
    q = plain_linear(h, w[prefix + "q"]).reshape(tokens, heads, dim)
    chunk = (mixer.get("mask") or {}).get("size")
    mixed = plain_sink_attention(q, keys_values[0], keys_values[1], w[prefix + "sink"], mixer["scale"], chunk)
    return plain_linear(mixed.reshape(tokens, heads * vdim), w[prefix + "o"]), keys_values


def plain_latent_mixer(h: torch.Tensor, w: dict, prefix: str, mixer: dict, eps: float) -> torch.Tensor:
    """Latent attention, written the long way: every position's keys and values are expanded from
    its latent vector, and the scores are sums over the unrotated and the rotated part."""
    tokens = h.shape[0]
    heads, dim, rot, vdim, rank = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"], mixer["kv_rank"]
    base, turn = mixer["rot"]["base"], mixer["rot"]["dims"]            # of the rot dims the first `turn` are rotated
    positions = torch.arange(tokens)

    def rotated(part):
        return torch.cat([plain_rotate_half(part[..., :turn], positions, base), part[..., turn:].double()], dim=-1)
    q = plain_linear(h, w[prefix + "q"]).reshape(tokens, heads, dim + rot)
    q_plain, q_turned = q[..., :dim], rotated(q[..., dim:])
    down = plain_linear(h, w[prefix + "dkv"])
    latent = plain_weight_norm(down[:, :rank], w[prefix + "dkv.norm"], eps)
    k_turned = rotated(down[:, rank:])                                             # [T, rot], one for all heads
    k_plain = plain_linear(latent, w[prefix + "uk"]).reshape(tokens, heads, dim)
    values = plain_linear(latent, w[prefix + "uv"]).reshape(tokens, heads, vdim)
    out = torch.zeros((tokens, heads, vdim), dtype=torch.float64)
    for t in range(tokens):
        seen = plain_visible(t, tokens, None)
        for head in range(heads):
            scores = (k_plain[:, head] @ q_plain[t, head] + k_turned @ q_turned[t, head]) * mixer["scale"]
            out[t, head] = plain_sink_softmax(scores, seen, float(w[prefix + "sink"][head])) @ values[:, head]
    return plain_linear(out.reshape(tokens, heads * vdim), w[prefix + "o"])


# ---- the gated linear recurrence ---------------------------------------------------------------------
def plain_causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: out[t, c] = bias[c] + sum_j taps[c, n-1-j] * x[t-j, c], zeros before
    the start (the last tap is the current token's)."""
    tokens, n = x.shape[0], taps.shape[1]
    x, taps = x.double(), taps.double()
    out = bias.double().expand(tokens, -1).clone()
    for j in range(min(n, tokens)):                 # (a tap further back than the sequence is long meets zeros only)
        out[j:] += taps[:, n - 1 - j] * x[:tokens - j]
    return out


def plain_block_gate(u: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """sigmoid of a block-diagonal product: u [T, C] cut into w.shape[0] equal parts, part k
    multiplied by the square matrix w[k] ([out, in]) plus b[k]."""
    tokens, blocks = u.shape[0], w.shape[0]
    parts = u.double().reshape(tokens, blocks, -1)
    return torch.sigmoid(torch.einsum("tbi,boi->tbo", parts, w.double()) + b.double()).reshape(tokens, -1)


def plain_gated_recurrence(u: torch.Tensor, r: torch.Tensor, i: torch.Tensor, lam: torch.Tensor) -> torch.Tensor:
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t from S = 0, with a_t = exp(-8 r_t softplus(lam))."""
    a = torch.exp(-8.0 * r.double() * torch.nn.functional.softplus(lam.double()))
    drive = torch.sqrt(1.0 - a * a) * i.double() * u.double()
    state = torch.zeros(u.shape[1], dtype=torch.float64)
    out = torch.zeros_like(drive)
    for t in range(u.shape[0]):
        state = a[t] * state + drive[t]
        out[t] = state
    return out


def plain_recurrent_mixer(h: torch.Tensor, w: dict, prefix: str) -> torch.Tensor:
    gate_branch = plain_gelu_tanh(plain_linear(h, w[prefix + "y"], w[prefix + "y.b"]))
    u = plain_causal_conv(plain_linear(h, w[prefix + "x"], w[prefix + "x.b"]), w[prefix + "conv"], w[prefix + "conv.b"])
    r = plain_block_gate(u, w[prefix + "ra"], w[prefix + "ra.b"])
    i = plain_block_gate(u, w[prefix + "ri"], w[prefix + "ri.b"])
    states = plain_gated_recurrence(u, r, i, w[prefix + "lam"])
    return plain_linear(states * gate_branch, w[prefix + "o"])


# ---- feed-forward --------------------------------------------------------------------------------------
def plain_clamped_feed_forward(h: torch.Tensor, w: dict, prefix: str, limit: float) -> torch.Tensor:
    g = torch.clamp(plain_linear(h, w[prefix + "gate"], w[prefix + "gate.b"]), max=limit)
    u = torch.clamp(plain_linear(h, w[prefix + "up"], w[prefix + "up.b"]), min=-limit, max=limit)
    return plain_linear(g * torch.sigmoid(1.702 * g) * (u + 1.0), w[prefix + "down"], w[prefix + "down.b"])


# ---- the whole model -------------------------------------------------------------------------------------
def plain_forward(config: dict, w: dict, tokens: list[int], layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of one whole sequence.  layers_out: a list that receives the
    residual stream after every layer."""
    eps = config["norm"]["eps"]
    x = w["embed"].double()[torch.tensor(tokens, dtype=torch.long)]
    kept = {}
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        h = plain_offset_norm(x, w[p + "norm1"], eps)
        kind, mixer = layer["type"], layer["mixer"]
        if kind == "attention":
            source = mixer.get("kv_from")
            mixed, kept[index] = plain_attention_mixer(h, w, p + "mix.", mixer, kept[source] if source is not None else None)
        elif kind == "latent_attention":
            mixed = plain_latent_mixer(h, w, p + "mix.", mixer, eps)
        elif kind == "rglru":
            mixed = plain_recurrent_mixer(h, w, p + "mix.")
        else:
            raise ValueError(f"unknown layer type {kind}")
        x = x + plain_offset_norm(mixed, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            h = plain_offset_norm(x, w[p + "norm2"], eps)
            x = x + plain_offset_norm(plain_clamped_feed_forward(h, w, p + "mlp.", layer["mlp"]["limit"]), w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return plain_linear(plain_offset_norm(x, w["final.norm"], eps), w["head"])


def plain_generate_greedy(config: dict, w: dict, prompt: list[int], count: int) -> list[int]:
    tokens, out = list(prompt), []
    for _ in range(count):
        token = int(torch.argmax(plain_forward(config, w, tokens)[-1]))
        out.append(token)
        tokens.append(token)
    return out
