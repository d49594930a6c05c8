"""A plain, slow Rekirax: whole sequences, no cache, one function for each mechanism.

Rekirax is a decoder-only model whose layers are listed in its configuration and of which a group may run
several times in a row. A layer is pre-norm; what its mixer reads is the normed stream plus a short causal
convolution of it. A mixer is windowed attention with a distance bias, or chunked attention beside an HGRN2
recurrence. This file shares no code with the engine: it parses config.json itself and reads the checkpoint
with the ``safetensors`` package. Everything is float64, token by token where the mechanism is a recurrence.

Notation: T tokens, D width, H query heads, G key/value heads; ``h`` is a mixer's input [T, D]; weights are
stored [out, in] and applied as ``h @ W.T``.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch
from safetensors import safe_open


def read_model(model_dir: str, dtype=torch.float64):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(dtype)
    return cfg, w


# -- single mechanisms -------------------------------------------------------------------------------
def unit_rms(x, eps):
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plus_one(x, w, eps):
    """The model's norm: the weight is stored around zero and used as 1 + w."""
    return unit_rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def input_convolution(h, taps_w):
    """h + conv(h): per channel c, conv(h)[t, c] = sum_j taps_w[c, j] * h[t - (n - 1) + j, c] with n taps, rows
    before the sequence's start being zero (the last tap multiplies the token's own row)."""
    T, n = h.shape[0], taps_w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(n):
            s = t - (n - 1) + j
            if s >= 0:
                out[t] += taps_w[:, j] * h[s]
    return out


def turn_half_split(v, positions, base, dims):
    """Rotary turn of the first `dims` entries of the last dimension in the half-split layout: entry i pairs with
    entry i + dims/2 (i < dims/2); at position p the pair (a, b) becomes (a cos - b sin, b cos + a sin) of the
    angle p * base^(-2i/dims). Entries from `dims` on pass unchanged. v: [T, heads, n]."""
    if dims == 0:
        return v
    half = dims // 2
    i = torch.arange(half, dtype=v.dtype)
    angle = positions.to(v.dtype)[:, None] * torch.pow(torch.tensor(float(base), dtype=v.dtype), -2.0 * i / dims)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], dim=-1)


def visible(T, kind, size):
    """[T, T] boolean: may query i see key j. 'window': 0 <= i - j < size; 'chunk': j <= i and both in the same
    block of `size` positions counted from 0."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    if kind == "window":
        return (i - j >= 0) & (i - j < size)
    return (j <= i) & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))


def softmax_over_visible(scores, mask):
    scores = scores.masked_fill(~mask, float("-inf"))
    return torch.softmax(scores, dim=-1)


def windowed_attention(h, w, P, m, eps):
    """The 'attention' mixer: queries and keys normed per head (one weight of size dim for all heads), the values
    are the keys as projected; score = softcap tanh(scale q.k / softcap) - r1_h ln(1 + r2_h (i - j)); sliding window."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[P + "q"].T).reshape(T, H, d)
    k = (h @ w[P + "k"].T).reshape(T, G, d)
    v = k
    q, k = norm_plain(q, w[P + "q.norm"], eps), norm_plain(k, w[P + "k.norm"], eps)
    mask = visible(T, "window", m["mask"]["size"])
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).clamp(min=0).to(h.dtype)
    cap = m.get("softcap")
    heads = []
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s - w[P + "r1"][a] * torch.log1p(w[P + "r2"][a] * dist)
        heads.append(softmax_over_visible(s, mask) @ v[:, g])
    return torch.cat(heads, dim=-1) @ w[P + "o"].T


def chunked_gated_attention(h, w, P, m, eps):
    """The left mixer of a parallel pair: queries and keys normed over their whole projection, the first rot.dims
    entries of every head turned, chunked causal mask, the heads' outputs times sigmoid(W_g h)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = norm_plain(h @ w[P + "q"].T, w[P + "q.norm"], eps).reshape(T, H, d)
    k = norm_plain(h @ w[P + "k"].T, w[P + "k.norm"], eps).reshape(T, G, d)
    v = (h @ w[P + "v"].T).reshape(T, G, dv)
    q = turn_half_split(q, pos, m["rot"]["base"], m["rot"]["dims"])
    k = turn_half_split(k, pos, m["rot"]["base"], m["rot"]["dims"])
    mask = visible(T, "chunk", m["mask"]["size"])
    heads = []
    for a in range(H):
        g = a // (H // G)
        heads.append(softmax_over_visible((q[:, a] @ k[:, g].T) * m["scale"], mask) @ v[:, g])
    return (torch.cat(heads, dim=-1) * torch.sigmoid(h @ w[P + "g"].T)) @ w[P + "o"].T


def hgrn2(h, w, P, m, eps, state=None):
    """The right mixer: per head S <- diag(f) S + (1 - f) v^T, o = S^T q with q = silu(W_q h) and the forget gate
    f = l + (1 - l) sigmoid(W_f h + b); every head's o normed over vdim with one shared weight. Token by token."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = torch.nn.functional.silu(h @ w[P + "q"].T).reshape(T, H, d)
    v = (h @ w[P + "v"].T).reshape(T, H, dv)
    low = w[P + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ w[P + "f"].T + w[P + "f.b"])).reshape(T, H, d)
    S = torch.zeros(H, d, dv, dtype=h.dtype) if state is None else state
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = (S * q[t][:, :, None]).sum(1)
    o = norm_plain(o, w[P + "norm"], eps)
    return o.reshape(T, H * dv) @ w[P + "o"].T


def parallel_pair(h, w, P, m, eps):
    a = chunked_gated_attention(h, w, P + "left.", m["left"], eps)
    b = hgrn2(h, w, P + "right.", m["right"], eps)
    return 0.5 * (norm_plain(a, w[P + "left.out"], eps) + norm_plain(b, w[P + "right.out"], eps))


def gated_feed_forward(h, w, P):
    g = h @ w[P + "gate"].T + w[P + "gate.b"]
    u = h @ w[P + "up"].T + w[P + "up.b"]
    return (gelu_tanh(g) * u) @ w[P + "down"].T + w[P + "down.b"]


# -- the model ---------------------------------------------------------------------------------------
def layer(cfg, w, i, x):
    lc, L, eps = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"]
    h = norm_plus_one(x, w[L + "norm1"], eps)
    if cfg.get("canon"):
        h = input_convolution(h, w[L + "canon1"])
    if lc["type"] == "attention":
        x = x + windowed_attention(h, w, L + "mix.", lc["mixer"], eps)
    else:
        x = x + parallel_pair(h, w, L + "mix.", lc["mixer"], eps)
    if lc.get("mlp") is not None:
        x = x + gated_feed_forward(norm_plus_one(x, w[L + "norm2"], eps), w, L + "mlp.")
    return x


def layer_runs(cfg):
    """The order in which layers run: (layer, pass number if this run opens a pass of the loop, else None)."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg, w, tokens: List[int], streams: Optional[list] = None):
    """Logits [T, vocab] of a whole sequence; `streams` collects the residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x0 = norm_plus_one(w["embed"][torch.tensor(tokens)], w["embed.norm"], eps)
    x = x0
    for i, opens in layer_runs(cfg):
        if opens is not None:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][opens]
        x = layer(cfg, w, i, x)
        if streams is not None:
            streams.append(x.clone())
    return norm_plus_one(x, w["final.norm"], eps) @ w["embed"].T


def greedy_generate(cfg, w, prompt: List[int], n: int) -> List[int]:
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))      # the lowest index on ties
    return ids[len(prompt):]
