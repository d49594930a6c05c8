"""A plain, slow Kugulorn: whole sequences, no cache, one function for each mechanism.

Kugulorn is a decoder-only model whose layers are listed in its configuration: each layer has a mixer
(latent attention or a Mamba-2 state-space mixer) and optionally a gated feed-forward, both between a norm
in front and a norm behind, with a layer scale and a residual multiplier. This file shares no code with
the engine: it parses config.json itself and reads the checkpoint with the ``safetensors`` package.
Everything is computed in float64 by default, token by token where the mechanism is a recurrence.

Notation: T tokens, D width, H heads; ``h`` is a sub-layer's (normalised) input [T, D].
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
def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last dimension (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def grouped_rms_norm(x, weight, eps, groups):
    """The last dimension in `groups` equal parts, each divided by its own root mean square, then * weight."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    parts = parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
    return parts.reshape(x.shape) * weight


def rotate_pairs(v, positions, base, dims):
    """Interleaved rotary turn of the first `dims` entries of the last dimension: the pair (v[2i], v[2i+1])
    at position p is turned by the angle p * base^(-2i/dims); the entries behind `dims` pass unchanged.
    v: [T, ..., n]; positions: [T]."""
    out = v.clone()
    half = dims // 2
    i = torch.arange(half, dtype=v.dtype)
    freq = torch.pow(torch.tensor(float(base), dtype=v.dtype), -2.0 * i / dims)
    angle = positions.to(v.dtype)[:, None] * freq[None, :]                      # [T, half]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    c, s = torch.cos(angle).reshape(shape), torch.sin(angle).reshape(shape)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def silu(v):
    return v * torch.sigmoid(v)


def softplus(v):
    """log(1 + exp(v)), with no clamp; written so that large v does not overflow."""
    return torch.where(v > 0, v + torch.log1p(torch.exp(-v.abs())), torch.log1p(torch.exp(-v.abs())))


def latent_kv(h, positions, w, pre, mixer, eps):
    """What a latent-attention layer leaves for its cache: the normed latent c [T, kv_rank] and the one
    rotated key part [T, rot_dim] that all heads share."""
    r, rd = mixer["kv_rank"], mixer["rot_dim"]
    dkv = h @ w[pre + "dkv"].T
    c = rms_norm(dkv[:, :r], w[pre + "dkv.norm"], eps)
    k_rot = rotate_pairs(dkv[:, r:r + rd], positions, mixer["rot"]["base"], mixer["rot"]["dims"])
    return c, k_rot


def latent_attention(h, positions, w, pre, mixer, eps, shared_kv=None):
    """Queries through a latent; keys and values expanded per head from the cached latent; one rotated key
    part for all heads; a sliding window; softmax. Returns (output [T, D], (c, k_rot))."""
    H, dn, rd, dv = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"]
    T = h.shape[0]
    c_q = rms_norm(h @ w[pre + "dq"].T, w[pre + "dq.norm"], eps)
    q = (c_q @ w[pre + "uq"].T).reshape(T, H, dn + rd)
    q_plain, q_rot = q[..., :dn], rotate_pairs(q[..., dn:], positions, mixer["rot"]["base"], mixer["rot"]["dims"])
    c, k_rot = shared_kv if shared_kv is not None else latent_kv(h, positions, w, pre, mixer, eps)
    k_plain = (c @ w[pre + "uk"].T).reshape(T, H, dn)
    v = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    scores = torch.einsum("thd,shd->hts", q_plain, k_plain) + torch.einsum("thd,sd->hts", q_rot, k_rot)
    scores = scores * mixer["scale"]
    i, j = positions[:, None], positions[None, :]
    visible = (i - j >= 0) & (i - j < mixer["mask"]["size"])
    scores = scores.masked_fill(~visible[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    out = torch.einsum("hts,shd->thd", p, v).reshape(T, H * dv)
    return out @ w[pre + "o"].T, (c, k_rot)


def causal_conv(x, weight, bias, before=None):
    """y[t, ch] = bias[ch] + sum_j weight[ch, j] * x[t - (taps - 1 - j), ch]; the last column is the current
    token's; inputs before the start are zeros (or the rows of `before`, [taps - 1, channels])."""
    taps = weight.shape[1]
    pad = torch.zeros(taps - 1, x.shape[1], dtype=x.dtype) if before is None else before
    xp = torch.cat([pad, x], 0)
    y = bias[None, :].expand(x.shape[0], -1).clone()
    for j in range(taps):
        y = y + xp[j:j + x.shape[0]] * weight[:, j][None, :]
    return y


def ssm_scan(x, B, C, dt, A_log, D, groups, state=None):
    """Per head h (group g = h // (H / groups)), token by token:
         S <- exp(-exp(A_log_h) dt_t) S + dt_t B_t x_t^T   (S is [N, P]);   y_t = S^T C_t + D_h x_t.
    x [T, H, P], B and C [T, G, N], dt [T, H] (already positive). Returns (y [T, H, P], final state)."""
    T, H, P = x.shape
    N = B.shape[-1]
    S = torch.zeros(H, N, P, dtype=x.dtype) if state is None else state.clone()
    per = H // groups
    y = torch.zeros_like(x)
    for t in range(T):
        for hd in range(H):
            g = hd // per
            S[hd] = torch.exp(-torch.exp(A_log[hd]) * dt[t, hd]) * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + D[hd] * x[t, hd]
    return y, S


def mamba2(h, w, pre, mixer, eps):
    """In-projection [z | x | B | C | dt]; causal convolution and silu on x, B, C; dt = softplus(dt + bias);
    the scan; gate with silu(z), then the grouped norm, then the output projection."""
    H, P, N, G = mixer["heads"], mixer["vdim"], mixer["state"], mixer["groups"]
    inner = H * P
    T = h.shape[0]
    proj = h @ w[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"])
    y, _ = ssm_scan(x, B, C, dt, w[pre + "A_log"], w[pre + "D"], G)
    y = y.reshape(T, inner) * silu(z)
    y = grouped_rms_norm(y, w[pre + "norm"], eps, mixer["norm_groups"])
    return y @ w[pre + "o"].T


def gated_feed_forward(h, w, pre, mlp):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    limit = mlp["limit"]
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


# -- the model ---------------------------------------------------------------------------------------
def forward(cfg, w, ids: List[int], return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (positions from 0); with return_layers also the residual
    stream after every layer [L, T, D]."""
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = w["embed"][torch.tensor(ids, dtype=torch.long)]
    positions = torch.arange(len(ids))
    kept: Dict[int, tuple] = {}
    after = []
    for i, layer in enumerate(cfg["layers"]):
        L = f"l{i}."
        h = rms_norm(x, w[L + "norm1"], eps)
        if layer["type"] == "latent_attention":
            src = layer["mixer"].get("kv_from")
            y, kv = latent_attention(h, positions, w, L + "mix.", layer["mixer"], eps, kept[src] if src is not None else None)
            kept[i] = kv
        elif layer["type"] == "mamba2":
            y = mamba2(h, w, L + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + m * w[L + "ls1"] * rms_norm(y, w[L + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = rms_norm(x, w[L + "norm2"], eps)
            y = gated_feed_forward(h, w, L + "mlp.", layer["mlp"])
            x = x + m * w[L + "ls2"] * rms_norm(y, w[L + "norm2b"], eps)
        after.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(after)) if return_layers else logits


def greedy_generate(cfg, w, prompt: List[int], n_new: int) -> List[int]:
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        tok = int(torch.argmax(forward(cfg, w, ids)[-1]))
        out.append(tok)
        ids.append(tok)
    return out
