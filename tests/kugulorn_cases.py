"""Small Kugulorn configurations for the tests (none of them anyone's model), and the comparison of an
engine's logits with the plain implementation's, position by position."""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch

import plain_kugulorn as pk
import replay_util as ru


def latent(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=32, window=9, base=10000.0, dims=None, scale=None, kv_from=None,
           mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "mask": {"size": window}, "rot": {"base": base, "dims": rot_dim if dims is None else dims},
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def mamba(heads=6, vdim=8, state=16, groups=3, conv=4, norm_groups=3, mlp=None):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": mlp}


def dense(ff=96, limit=1.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def model(layers, vocab=300, width=64, eps=1e-5, mult=0.7):
    return {"architecture": "Kugulorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}


# single mechanisms
ONLY_MAMBA = model([mamba()])
ONLY_MAMBA_WIDE_STATE = model([mamba(heads=2, vdim=24, state=80, groups=1, conv=2, norm_groups=1)], width=48, mult=1.0)
ONLY_LATENT = model([latent()])
ONLY_LATENT_MLP = model([latent(heads=3, dim=8, rot_dim=4, vdim=8, kv_rank=24, q_rank=16, window=200, mlp=dense())], width=40)
# several layers: a reader of another layer's pages with a narrower window and one with a wider window than the
# writer's; a feed-forward behind a Mamba layer; a rotation of fewer columns than the rotated part has
MIXED_A = model([
    latent(window=13, mlp=dense(80, 0.8)),
    mamba(),
    latent(window=5, kv_from=0, heads=4, dim=8, vdim=16, q_rank=24),
    mamba(heads=4, vdim=16, state=8, groups=1, conv=3, norm_groups=2, mlp=dense(64, 2.0)),
    latent(window=20, kv_from=0, mlp=dense()),
], vocab=257, width=64, eps=1e-6, mult=0.5)
MIXED_B = model([
    mamba(heads=3, vdim=16, state=24, groups=3, conv=2, norm_groups=1),
    latent(heads=5, dim=24, rot_dim=16, vdim=8, kv_rank=24, q_rank=40, window=33, base=500.0, dims=8),
    latent(heads=1, dim=32, rot_dim=16, vdim=48, kv_rank=24, q_rank=8, window=4, base=500.0, dims=8, kv_from=1, mlp=dense(48, 1.5)),
], vocab=513, width=48, eps=1e-5, mult=1.25)
# scores that one key dominates: a window that is one key off, or a key lost at a page's border, changes a row
PEAKED = model([latent(window=5, scale=6.0), latent(window=16, scale=6.0, heads=1), latent(window=6, scale=6.0, kv_from=1)], width=32)

# the same with windows of hundreds of keys: a single far key often carries a row
PEAKED_FAR = model([latent(window=300, scale=5.0), latent(window=190, scale=5.0, heads=3, kv_from=0)], width=32)

# cached rows of 96 and 160 columns (latents of 64 and 128): sizes that the matrix-core kernel of prompt portions
# takes at pages of 16 tokens in bfloat16; windows shorter and longer than its 64-key tiles; 3 and 5 heads, so
# that a tile of 64 (token, head) rows starts and ends in the middle of a token
TILED = model([
    latent(heads=3, dim=16, rot_dim=32, vdim=16, kv_rank=64, q_rank=32, window=40, mlp=dense(64, 1.2)),
    mamba(heads=4, vdim=8, state=8, groups=2, conv=3, norm_groups=1),
    latent(heads=5, dim=8, rot_dim=32, vdim=24, kv_rank=128, q_rank=40, window=150),
    latent(heads=2, dim=24, rot_dim=32, vdim=8, kv_rank=128, q_rank=16, window=70, kv_from=2),
], vocab=211, width=56, mult=0.6)

# the widest cached rows of the matrix-core kernel: latents of 512 beside 32 and 64 rotated columns
WIDE = model([
    latent(heads=2, dim=16, rot_dim=32, vdim=8, kv_rank=512, q_rank=16, window=90),
    latent(heads=3, dim=8, rot_dim=64, vdim=8, kv_rank=512, q_rank=8, window=200),
], vocab=97, width=32, mult=0.5)

# sizes that are multiples of neither 8 nor 4: the plain bfloat16 product, the scan without staging, rows of the
# pages that are not 16-byte pieces
ODD = model([
    mamba(heads=3, vdim=12, state=10, groups=1, conv=2, norm_groups=3, mlp=dense(52, 1.0)),
    latent(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=18, q_rank=20, window=11),
    mamba(heads=2, vdim=9, state=33, groups=2, conv=5, norm_groups=1),
    latent(heads=2, dim=7, rot_dim=4, vdim=5, kv_rank=19, q_rank=9, window=30),          # a cached row of 23 columns
], vocab=101, width=44, mult=0.9)

# rms(difference, mean taken off) / rms(logits, mean taken off) of a row may be at most this
TOL = {"float32": 5e-6, "bfloat16": 6e-2}
# with the peaked scores of PEAKED, 32-bit rounding shows more (seen: 2e-5)
TOL_PEAKED = 1e-4

_plain: Dict[tuple, np.ndarray] = {}
_weights: Dict[str, tuple] = {}


def plain_logits(model_dir, toks) -> np.ndarray:
    key = (model_dir, tuple(toks))
    if key not in _plain:
        if model_dir not in _weights:
            _weights[model_dir] = pk.read_model(model_dir)
        cfg, w = _weights[model_dir]
        _plain[key] = pk.forward(cfg, w, list(toks)).numpy()
    return _plain[key]


def row_error(got, ref) -> float:
    d = got.astype(np.float64) - ref
    d = d - d.mean()
    r = ref - ref.mean()
    return float(np.sqrt((d * d).mean()) / np.sqrt((r * r).mean()))


def check_against_plain(model_dir, reqs, steps, outputs, dtype, vocab, label="", tol=None):
    got = ru.collect(steps, outputs, vocab)
    tol = tol or TOL[dtype]
    worst, where = 0.0, None
    for rid, toks in reqs.items():
        ref = plain_logits(model_dir, toks)
        assert sorted(got.get(rid, {})) == list(range(len(toks))), f"{rid}: positions missing"
        for pos in range(len(toks)):
            row = got[rid][pos]
            assert np.isfinite(row).all(), f"{label} {rid} position {pos}: non-finite logits"
            e = row_error(row, ref[pos])
            if e > worst:
                worst, where = e, (rid, pos)
    print(f"worst difference from plain [{dtype} {label}]: {worst:.3e} at {where} (allowed {tol:.1e})")
    assert worst <= tol, f"{label}: {where} differs by {worst:.3e} > {tol:.1e}"
    return worst


def requests(vocab, lengths, seed):
    return ru.random_requests(vocab, lengths, seed=seed)
