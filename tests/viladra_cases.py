"""Small Viladra configurations for the tests (none of them anyone's model), and the comparison of an
engine's logits with the plain implementation's, position by position."""
from __future__ import annotations

from typing import Dict

import numpy as np

import plain_viladra as pv
import replay_util as ru


def retention(heads=2, dim=16, vdim=16, decay=None, base=10000.0, dims=8, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay if decay is not None else [1.0 - 2.0 ** -(3 + k) for k in range(heads)]}
    if dims is not None:
        m["rot"] = {"base": base, "dims": dims}
    return {"type": "retention", "mixer": m, "mlp": mlp}


def gla(heads=2, dim=16, vdim=16, tau=8.0, rank=None, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}
    if rank is not None:
        m["rank"] = rank           # (the rank of the decays' map is read off the checkpoint; this key sizes the random one)
    return {"type": "gla", "mixer": m, "mlp": mlp}


def attention(heads=4, kv_heads=2, dim=16, vdim=24, window=9, scale=None, mlp=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
                                           "scale": scale if scale is not None else dim ** -0.5}, "mlp": mlp}


def moe(experts=4, top=2, ff=24, shared=40, scale=1.5):
    return {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff},
            "shared": {"ff": shared} if shared else None}


def model(layers, vocab=300, width=64, eps=1e-5, taps=4, embed_scale=0.7, softcap=20.0):
    c = {"architecture": "Viladra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
         "embedding": {"scale": embed_scale}}
    if taps is not None:
        c["canon"] = {"taps": taps}
    if softcap is not None:
        c["logit_softcap"] = softcap
    return c


# single mechanisms: each mixer alone without a feed-forward, the experts behind the simplest mixer
ONLY_RETENTION = model([retention()])
ONLY_RETENTION_PLAIN = model([retention(heads=3, dim=24, vdim=40, decay=[0.5, 0.96875, 1.0], dims=None)], width=48, taps=1, softcap=None)
ONLY_GLA = model([gla()])
ONLY_GLA_WIDE = model([gla(heads=1, dim=72, vdim=136, tau=3.0, rank=5)], width=40, taps=2)
ONLY_ATTENTION = model([attention()])
ONLY_ATTENTION_SQUARE = model([attention(heads=3, kv_heads=3, dim=24, vdim=24, window=40)], width=48, taps=1, embed_scale=1.0)
ONLY_EXPERTS = model([retention(mlp=moe())])
ONLY_EXPERTS_ALL = model([gla(mlp=moe(experts=3, top=3, ff=16, shared=None, scale=1.0))], width=32)      # every expert chosen, no shared one
NO_CONVOLUTION = model([gla(mlp=moe(experts=3, top=1, ff=16, shared=8)), attention(window=7)], width=32, taps=None)
ONE_EXPERT = model([attention(mlp=moe(experts=1, top=1, ff=32, shared=16, scale=3.0))], width=32)
# several layers in orders of their own: what a layer hands on is a weighted sum over everything before it
MIXED_A = model([
    gla(mlp=moe()),
    attention(window=13, mlp=moe(experts=6, top=1, ff=16, shared=24, scale=2.0)),
    retention(heads=4, dim=8, vdim=24, dims=4),
    attention(heads=2, kv_heads=1, dim=32, vdim=8, window=5, mlp=moe(experts=5, top=4, ff=8, shared=None)),
    gla(heads=4, dim=8, vdim=8, tau=16.0, rank=3, mlp=moe(experts=2, top=1, ff=40)),
], vocab=257, width=64, eps=1e-6, taps=3)
MIXED_B = model([
    attention(heads=1, kv_heads=1, dim=48, vdim=16, window=33),
    retention(heads=1, dim=64, vdim=24, decay=[0.99], base=500.0, dims=64, mlp=moe(experts=7, top=3, ff=16, shared=32, scale=1.75)),
    retention(heads=5, dim=16, vdim=8, dims=16, mlp=moe(experts=3, top=2, ff=24)),
], vocab=513, width=48, taps=2, embed_scale=0.25, softcap=5.0)
# scores that single keys dominate (queries and keys are normed, so |q.k| is about dim at most: the scale does the
# peaking; the score bias lies around -2, so most other keys weigh little): a window that is one key off, or a key lost
# at a page's border, changes a row
PEAKED = model([attention(window=5, scale=3.0), attention(window=16, scale=3.0, heads=2, kv_heads=1, vdim=16)], width=32)
# the same at the head sizes that the matrix-core tiles and the split-key kernel take in bfloat16 (32, 64, 128; keys
# and values of one width), one layer each so that a row shows its own window: one key more or less in a window
# changes a third to two thirds of the rows by more than three times the bfloat16 tolerance
PEAKED_TILES_32 = model([attention(window=9, scale=0.8, heads=4, kv_heads=2, dim=32, vdim=32)], width=64)
PEAKED_TILES_64 = model([attention(window=5, scale=0.6, heads=2, kv_heads=1, dim=64, vdim=64)], width=64)
PEAKED_TILES_128 = model([attention(window=3, scale=0.4, heads=2, kv_heads=2, dim=128, vdim=128)], width=32)
# the same with a window of hundreds of keys, and recurrences that forget slowly: a token far back carries a row
PEAKED_FAR = model([attention(window=300, scale=3.0), retention(heads=2, dim=8, vdim=8, decay=[0.998046875, 1.0]),
                    gla(heads=2, dim=8, vdim=8, tau=64.0)], width=32)
# sizes that are multiples of neither 8 nor 4; more key channels than a slice of the scan holds and more value
# columns than a wavefront has lanes; a width that is odd
ODD = model([
    retention(heads=3, dim=10, vdim=14, dims=6, mlp=moe(experts=5, top=2, ff=13, shared=7)),
    attention(heads=3, kv_heads=1, dim=7, vdim=9, window=30),
    gla(heads=3, dim=33, vdim=70, tau=2.5, rank=7, mlp=moe(experts=3, top=1, ff=9, shared=None)),
    attention(heads=2, kv_heads=2, dim=6, vdim=5, window=3),
], vocab=101, width=43, taps=6)
# the sizes of a larger model's layers: heads of 64 and 128, pages of many sizes
LARGER = model([
    gla(heads=4, dim=64, vdim=128, tau=12.0, rank=16, mlp=moe(experts=6, top=2, ff=96, shared=160)),
    attention(heads=4, kv_heads=2, dim=64, vdim=64, window=100, mlp=moe(experts=6, top=2, ff=96, shared=160)),
    retention(heads=2, dim=128, vdim=128, dims=64, decay=[0.96875, 0.998046875]),
    attention(heads=2, kv_heads=1, dim=128, vdim=128, window=150),
], vocab=211, width=256)

# rms(difference, mean taken off) / rms(logits, mean taken off) of a row may be at most this. Single rows are
# ill-conditioned by the design itself: a head's readout is divided by its own root mean square, so where the
# readout is a sum of one or two terms whose coefficients q.k happen to lie near zero (the first positions of a
# recurrence), the rounding of that dot product is all that is left (seen: a row at position 1 with 50 times the
# error of its neighbours in 32-bit and in bfloat16 alike, the same in every schedule). Hence: few rows above the
# tolerance, none above five times it.
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
TOL_PEAKED = 1e-4

_plain: Dict[tuple, np.ndarray] = {}
_weights: Dict[str, tuple] = {}


def plain_model(model_dir):
    if model_dir not in _weights:
        _weights[model_dir] = pv.read_model(model_dir)
    return _weights[model_dir]


def plain_logits(model_dir, toks) -> np.ndarray:
    key = (model_dir, tuple(toks))
    if key not in _plain:
        cfg, w = plain_model(model_dir)
        _plain[key] = pv.forward(cfg, w, list(toks)).numpy()
    return _plain[key]


_calls: Dict[tuple, np.ndarray] = {}
CLOSE_CALL = 0.02       # a gap between two experts' scores below which bfloat16 rounding may choose the other one
CLOSE_REACH = 4         # positions behind such a token that still carry it: the short convolutions read the last few
                        # inputs, and a recurrence's state the last few tokens most


def closest_call(model_dir, toks) -> np.ndarray:
    key = (model_dir, tuple(toks))
    if key not in _calls:
        cfg, w = plain_model(model_dir)
        _calls[key] = pv.closest_call(cfg, w, list(toks)).numpy()
    return _calls[key]


def row_error(got, ref) -> float:
    d = got.astype(np.float64) - ref
    d = d - d.mean()
    r = ref - ref.mean()
    return float(np.sqrt((d * d).mean()) / np.sqrt((r * r).mean()))


def check_against_plain(model_dir, reqs, steps, outputs, dtype, vocab, label="", tol=None):
    """At most one row in two hundred (32-bit; bfloat16: one in fifty) may lie above the tolerance and none above
    five times it (with an explicit `tol`: none above it). In bfloat16 a token at which the plain model's router makes
    a close call (two experts' scores within CLOSE_CALL of each other at the edge of the choice) is not compared,
    since rounding may rightly choose the other expert there, and neither are the CLOSE_REACH tokens behind it, which
    read that token's streams (the same rows differ in every schedule; 32-bit compares every row)."""
    got = ru.collect(steps, outputs, vocab)
    strict = tol is not None
    tol = tol or TOL[dtype]
    worst, where, errs = 0.0, None, []
    for rid, toks in reqs.items():
        ref = plain_logits(model_dir, toks)
        close = np.zeros(len(toks), dtype=bool)
        if dtype == "bfloat16":
            at = closest_call(model_dir, toks) < CLOSE_CALL
            for pos in range(len(toks)):
                close[pos] = at[max(0, pos - CLOSE_REACH):pos + 1].any()
        assert sorted(got.get(rid, {})) == list(range(len(toks))), f"{rid}: positions missing"
        for pos in range(len(toks)):
            row = got[rid][pos]
            assert np.isfinite(row).all(), f"{label} {rid} position {pos}: non-finite logits"
            if close[pos]:
                continue
            e = row_error(row, ref[pos])
            errs.append(e)
            if e > worst:
                worst, where = e, (rid, pos)
    over = sum(e > tol for e in errs)
    print(f"worst difference from plain [{dtype} {label}]: {worst:.3e} at {where} (allowed {tol:.1e}; {over} of {len(errs)} rows above)")
    if strict:
        assert worst <= tol, f"{label}: {where} differs by {worst:.3e} > {tol:.1e}"
    else:
        few = max(1, len(errs) // (50 if dtype == "bfloat16" else 200))
        assert worst <= 5 * tol and over <= few, f"{label}: {where} differs by {worst:.3e}, {over} of {len(errs)} rows above {tol:.1e}"
    return worst


def requests(vocab, lengths, seed):
    return ru.random_requests(vocab, lengths, seed=seed)
