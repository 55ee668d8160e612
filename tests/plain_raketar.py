"""A plain implementation of the Raketar decoder, for tests: one function per mechanism, float64, whole
sequences at once (no cache, no state carried between calls, no batching), written from the design's
equations and sharing nothing with the engine.

A model is (config, weights): `config` is the config.json dict, `weights` a dict of float64 tensors by the
checkpoint's names.  `forward(config, weights, tokens)` returns the logits of every position and the residual
stream after every layer run.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


# ---- positions ------------------------------------------------------------------------------------------
def rotate_interleaved(x, positions, dims, base, factor):
    """x: [T, heads, dim].  The first `dims` dims of every head turn, dim 2i with dim 2i + 1, by the angle
    position * base^(-2i / dims) / factor; the rest pass."""
    out = x.clone()
    for i in range(dims // 2):
        frequency = base ** (-2.0 * i / dims) / factor
        angle = positions.to(F64) * frequency
        cos, sin = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * cos - v * sin
        out[..., 2 * i + 1] = v * cos + u * sin
    return out


# ---- differential attention -----------------------------------------------------------------------------
def causal_softmax_attention(q, k, v, scale):
    """q, k: [T, dim], v: [T, vdim]; every position sees itself and all before it."""
    scores = (q @ k.T) * scale
    T = q.shape[0]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, -math.inf)
    return torch.softmax(scores, dim=-1) @ v


def differential_lambda(w, prefix, diff):
    return (math.exp(float((w[prefix + "lq1"] * w[prefix + "lk1"]).sum()))
            - math.exp(float((w[prefix + "lq2"] * w[prefix + "lk2"]).sum())) + diff)


def differential_attention(mixer, w, prefix, h, positions, eps):
    """h: [T, width] -> [T, width]."""
    H, G, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    diff, scale = float(mixer["diff"]), float(mixer["scale"])
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).reshape(T, H, 2, dim)
    k = (h @ w[prefix + "k"].T).reshape(T, G, 2, dim)
    v = (h @ w[prefix + "v"].T).reshape(T, G, vdim)
    rot = mixer.get("rot")
    if rot is not None:
        factor = float(rot["scaling"]["factor"]) if rot.get("scaling") else 1.0
        q = rotate_interleaved(q.reshape(T, 2 * H, dim), positions, int(rot["dims"]), float(rot["base"]), factor).reshape(T, H, 2, dim)
        k = rotate_interleaved(k.reshape(T, 2 * G, dim), positions, int(rot["dims"]), float(rot["base"]), factor).reshape(T, G, 2, dim)
    lam = differential_lambda(w, prefix, diff)
    heads = []
    for head in range(H):
        group = head // (H // G)
        first = causal_softmax_attention(q[:, head, 0], k[:, group, 0], v[:, group], scale)
        second = causal_softmax_attention(q[:, head, 1], k[:, group, 1], v[:, group], scale)
        heads.append(unit_rms(first - lam * second, eps) * (1.0 - diff))
    joined = torch.cat(heads, dim=-1) * torch.sigmoid(h @ w[prefix + "g"].T)
    return joined @ w[prefix + "o"].T


# ---- mLSTM ----------------------------------------------------------------------------------------------
def mlstm_memory(q, k, v, gate_i, gate_f, state=None):
    """The matrix memory alone.  q, k: [T, heads, dim] (q scaled already), v: [T, heads, vdim], gate_i and gate_f: the log
    gates [T, heads].  Returns the heads' results [T, heads, vdim] and the state (S, n, m) after the last token."""
    T, heads, dim = q.shape
    vdim = v.shape[-1]
    if state is None:
        S, n, m = torch.zeros(heads, dim, vdim, dtype=F64), torch.zeros(heads, dim, dtype=F64), torch.zeros(heads, dtype=F64)
    else:
        S, n, m = (part.clone() for part in state)
    out = torch.zeros(T, heads, vdim, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(gate_f[t] + m, gate_i[t])
        keep, take = torch.exp(gate_f[t] + m - m_new), torch.exp(gate_i[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        top = torch.einsum("hdv,hd->hv", S, q[t])
        bottom = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = top / bottom[:, None]
    return out, (S, n, m)


def log_gates(pre_i, pre_f, cap):
    return cap * torch.tanh(pre_i / cap), torch.nn.functional.logsigmoid(cap * torch.tanh(pre_f / cap))


def mlstm(mixer, w, prefix, h, eps, state=None):
    """h: [T, width] -> [T, width].  state: None (zeros) or (S [heads, dim, vdim], n [heads, dim], m [heads]);
    the state after the last token is returned beside the output."""
    heads, dim, vdim, cap = mixer["heads"], mixer["dim"], mixer["vdim"], float(mixer["gate_cap"])
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).reshape(T, heads, dim) * dim ** -0.5
    k = (h @ w[prefix + "k"].T).reshape(T, heads, dim)
    v = (h @ w[prefix + "v"].T).reshape(T, heads, vdim)
    gate_i, gate_f = log_gates(h @ w[prefix + "i"].T + w[prefix + "i.b"], h @ w[prefix + "f"].T + w[prefix + "f.b"], cap)
    out, state = mlstm_memory(q, k, v, gate_i, gate_f, state)
    out = unit_rms(out, eps).reshape(T, heads * vdim) * w[prefix + "norm"] * torch.sigmoid(h @ w[prefix + "g"].T)
    return out @ w[prefix + "o"].T, state


# ---- feed-forwards --------------------------------------------------------------------------------------
def gated_feed_forward(w, prefix, h):
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def routed_feed_forward(mlp, w, prefix, h):
    """Sigmoid scores, the `top` largest chosen, each chosen expert fed with score * h; plus the shared expert."""
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    scores = torch.sigmoid(h @ w[prefix + "router"].T)
    out = torch.zeros(h.shape[0], w[prefix + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        chosen = torch.topk(scores[t], top).indices
        for e in chosen.tolist():
            out[t] += gated_feed_forward(w, f"{prefix}e{e}.", (scores[t, e] * h[t])[None])[0]
    if mlp.get("shared") is not None:
        out = out + gated_feed_forward(w, prefix + "shared.", h)
    return out


def feed_forward(mlp, w, prefix, h):
    if mlp["kind"] == "dense":
        return gated_feed_forward(w, prefix, h)
    return routed_feed_forward(mlp, w, prefix, h)


# ---- the per-layer token input --------------------------------------------------------------------------
def token_side(config, w, layer, tokens, x, mult, eps):
    dim = int(config["token_side"]["dim"])
    e = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ w[f"l{layer}.side.gate"].T) * e
    y = g @ w[f"l{layer}.side.proj"].T
    return x + mult * unit_rms(y, eps) * w[f"l{layer}.side.norm"]


# ---- a layer, the model ---------------------------------------------------------------------------------
def layer_forward(config, w, layer, tokens, positions, x, states=None, key=None):
    spec, eps, mult = config["layers"][layer], float(config["norm"]["eps"]), float(config["residual_mult"])
    prefix = f"l{layer}."
    h = rms_norm(x, w[prefix + "norm1"], eps)
    if spec["type"] == "attention":
        mixed = differential_attention(spec["mixer"], w, prefix + "mix.", h, positions, eps)
    else:
        mixed, state = mlstm(spec["mixer"], w, prefix + "mix.", h, eps, None if states is None else states.get(key))
        if states is not None:
            states[key] = state
    if spec.get("mlp") is not None:
        mixed = mixed + feed_forward(spec["mlp"], w, prefix + "mlp.", h)
    x = x + mult * mixed
    if config.get("token_side") is not None:
        x = token_side(config, w, layer, tokens, x, mult, eps)
    return x


def layer_runs(config):
    """The order in which layers run: (layer, pass of the loop or None, first of its pass)."""
    count, loop = len(config["layers"]), config.get("loop")
    if loop is None:
        return [(layer, None, False) for layer in range(count)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(layer, None, False) for layer in range(start)]
    for t in range(times):
        runs += [(layer, t, layer == start) for layer in range(start, stop)]
    return runs + [(layer, None, False) for layer in range(stop, count)]


def forward(config, w, tokens):
    """tokens: a list of ids.  Returns (logits [T, vocab], residuals [runs, T, width])."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    eps = float(config["norm"]["eps"])
    embedded = w["embed"][tokens]
    x = embedded.clone()
    residuals = []
    for layer, t, first in layer_runs(config):
        if first:
            if t > 0:
                x = x + embedded
            x = x + w["loop.step"][t]
        x = layer_forward(config, w, layer, tokens, positions, x)
        residuals.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return logits, torch.stack(residuals)
