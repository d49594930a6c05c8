"""Small Rekirax configurations for the tests (none of them anyone's model), and the comparison of an
engine's logits with the plain implementation's, position by position."""
from __future__ import annotations

from typing import Dict

import numpy as np

import plain_rekirax as pr
import replay_util as ru


def attention(heads=4, kv_heads=2, dim=16, window=9, scale=None, softcap=5.0, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window},
         "scale": scale if scale is not None else dim ** -0.5}
    if softcap is not None:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def parallel(heads=4, kv_heads=2, dim=16, vdim=16, chunk=12, base=10000.0, dims=8, scale=None, r_heads=2, r_dim=8, r_vdim=16, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk},
            "rot": {"base": base, "dims": dims}, "scale": scale if scale is not None else dim ** -0.5}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim}}, "mlp": mlp}


def dense(ff=96):
    return {"kind": "dense", "ff": ff}


def model(layers, vocab=300, width=64, eps=1e-5, taps=4, loop=None):
    c = {"architecture": "Rekirax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if taps:
        c["canon"] = {"taps": taps}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


# single mechanisms (no loop): windowed attention with and without the cap; the pair; one-tap and no convolution;
# a feed-forward
ONLY_ATTENTION = model([attention()])
ONLY_ATTENTION_UNCAPPED = model([attention(heads=3, kv_heads=3, dim=24, window=40, softcap=None, mlp=dense(80))], width=48, taps=1)
ONLY_PAIR = model([parallel()])
ONLY_PAIR_WIDE = model([parallel(heads=2, kv_heads=1, dim=32, vdim=8, chunk=70, dims=32, r_heads=3, r_dim=40, r_vdim=72)], width=40, taps=None)
# a loop over the middle; a loop over everything that starts at layer 0; a single pass
LOOPED_A = model([
    parallel(mlp=dense(72)),
    attention(window=13, mlp=dense(64)),
    parallel(heads=6, kv_heads=3, dim=8, vdim=24, chunk=7, dims=4, r_heads=4, r_dim=16, r_vdim=8),
    attention(heads=2, kv_heads=1, dim=32, window=5, softcap=2.0, mlp=dense()),
    parallel(chunk=20, mlp=dense(40)),
], vocab=257, width=64, eps=1e-6, taps=3, loop=(1, 4, 2))
LOOPED_B = model([
    attention(heads=1, kv_heads=1, dim=48, window=33, softcap=30.0),
    parallel(heads=5, kv_heads=5, dim=16, vdim=8, chunk=64, base=500.0, dims=16, r_heads=1, r_dim=64, r_vdim=24, mlp=dense(48)),
], vocab=513, width=48, taps=2, loop=(0, 2, 3))
SINGLE_PASS = model([parallel(mlp=dense(64)), attention()], width=32, taps=5, loop=(1, 2, 1))
# scores that one key dominates: a window or a chunk that is one key off, or a key lost at a page's border, changes
# a row. (Queries and keys are normed, so |q.k| is about dim at most: the scale does the peaking, the cap is far off.)
PEAKED = model([attention(window=5, scale=3.0, softcap=200.0), parallel(chunk=6, scale=3.0), attention(window=16, scale=3.0, softcap=200.0, heads=2, kv_heads=1)],
               width=32, loop=(0, 2, 2))
# the same with windows and chunks of hundreds of keys: a single far key often carries a row
PEAKED_FAR = model([attention(window=300, scale=3.0, softcap=200.0), parallel(chunk=190, scale=3.0, r_dim=8)], width=32)
# sizes that are multiples of neither 8 nor 4; value heads of another width than the keys; more key channels than a
# slice of the recurrence holds and more value columns than a wavefront has lanes
ODD = model([
    parallel(heads=3, kv_heads=1, dim=10, vdim=14, chunk=11, dims=6, r_heads=3, r_dim=33, r_vdim=70, mlp=dense(52)),
    attention(heads=3, kv_heads=1, dim=7, window=30, softcap=3.0),
    parallel(heads=2, kv_heads=2, dim=6, vdim=5, chunk=3, dims=0, r_heads=2, r_dim=5, r_vdim=9),
], vocab=101, width=44, taps=6, loop=(0, 1, 2))

# head sizes and page sizes that the attention kernels shared with the other models take: 64 and 128 (the bfloat16
# matrix-core kernel of prompt portions, the split-key kernel of single tokens), 48 (the 32-bit matrix-core tiles only);
# windows and chunks shorter and longer than a tile of 64 or 128 keys, chunks that end inside a tile of queries
SHARED_KERNELS = model([
    parallel(heads=4, kv_heads=2, dim=64, vdim=64, chunk=100, dims=32, r_heads=2, r_dim=16, r_vdim=16, mlp=dense(64)),
    attention(heads=2, kv_heads=1, dim=128, window=150, softcap=8.0),
    parallel(heads=2, kv_heads=2, dim=128, vdim=128, chunk=37, dims=64, r_heads=1, r_dim=8, r_vdim=8),
    attention(heads=3, kv_heads=3, dim=48, window=70, softcap=None),
    attention(heads=4, kv_heads=1, dim=64, window=20, scale=0.5, softcap=4.0, mlp=dense(64)),
], vocab=211, width=64, loop=(2, 4, 2))

# rms(difference, mean taken off) / rms(logits, mean taken off) of a row may be at most this
# (32-bit: the kernels shared with plain attention work in base 2, one more rounding of every score than the plain
# model has; rows early in a sequence, where a head's recurrent output is still small in front of its unit norm,
# show it most: 1e-5 was seen, 5e-6 through the row kernel)
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
TOL_PEAKED = 1e-4

_plain: Dict[tuple, np.ndarray] = {}
_weights: Dict[str, tuple] = {}


def plain_logits(model_dir, toks) -> np.ndarray:
    key = (model_dir, tuple(toks))
    if key not in _plain:
        if model_dir not in _weights:
            _weights[model_dir] = pr.read_model(model_dir)
        cfg, w = _weights[model_dir]
        _plain[key] = pr.forward(cfg, w, list(toks)).numpy()
    return _plain[key]


def row_error(got, ref) -> float:
    d = got.astype(np.float64) - ref
    d = d - d.mean()
    r = ref - ref.mean()
    return float(np.sqrt((d * d).mean()) / np.sqrt((r * r).mean()))


def check_against_plain(model_dir, reqs, steps, outputs, dtype, vocab, label="", tol=None):
    """32-bit: no row may differ by more than the tolerance. bfloat16: rounding alone moves single rows of these
    small, deep models further than most (the same row by the same amount whatever the schedule), so at most one
    row in fifty may lie above the tolerance and none above twice it."""
    got = ru.collect(steps, outputs, vocab)
    tol = tol or TOL[dtype]
    worst, where, errs = 0.0, None, []
    for rid, toks in reqs.items():
        ref = plain_logits(model_dir, toks)
        assert sorted(got.get(rid, {})) == list(range(len(toks))), f"{rid}: positions missing"
        for pos in range(len(toks)):
            row = got[rid][pos]
            assert np.isfinite(row).all(), f"{label} {rid} position {pos}: non-finite logits"
            e = row_error(row, ref[pos])
            errs.append(e)
            if e > worst:
                worst, where = e, (rid, pos)
    over = sum(e > tol for e in errs)
    print(f"worst difference from plain [{dtype} {label}]: {worst:.3e} at {where} (allowed {tol:.1e}; {over} of {len(errs)} rows above)")
    if dtype == "bfloat16":
        assert worst <= 2 * tol and over <= max(1, len(errs) // 50), f"{label}: {where} differs by {worst:.3e}, {over} of {len(errs)} rows above {tol:.1e}"
    else:
        assert worst <= tol, f"{label}: {where} differs by {worst:.3e} > {tol:.1e}"
    return worst


def requests(vocab, lengths, seed):
    return ru.random_requests(vocab, lengths, seed=seed)
