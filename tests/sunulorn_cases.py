"""Small Sunulorn configurations for the tests (none of them anyone's model), and the comparison of an engine's
logits with the plain implementation's, position by position."""
from __future__ import annotations

from typing import Dict

import numpy as np

import plain_sunulorn as ps
import replay_util as ru


def conv_attention(heads=4, kv_heads=2, dim=16, taps=3, base=10000.0, dims=8, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5}
    if taps is not None:
        m["conv"] = taps
    if dims is not None:
        m["rot"] = {"base": base, "dims": dims}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def window_attention(heads=4, kv_heads=2, dim=16, vdim=24, window=9, keep=3, base=10000.0, dims=16, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if window is not None:
        m["mask"] = {"size": window}
        if keep is not None:
            m["mask"]["keep_first"] = keep
    if dims is not None:
        m["rot"] = {"base": base, "dims": dims}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def sink_attention(heads=4, kv_heads=2, dim=16, vdim=16, scale=None, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention_3", "mixer": m, "mlp": mlp}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(experts=4, top=2, ff=24, limit=1.5, shared=40, shared_limit=2.5):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit},
            "shared": {"ff": shared, "limit": shared_limit} if shared else None}


def model(layers, vocab=300, width=64, eps=1e-5, embed_scale=2.5):
    c = {"architecture": "Sunulorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if embed_scale is not None:
        c["embedding"] = {"scale": embed_scale}
    return c


# single mechanisms: each mixer alone without a feed-forward, each feed-forward behind the simplest mixer
ONLY_CONV = model([conv_attention()])
ONLY_CONV_BARE = model([conv_attention(heads=3, kv_heads=3, dim=24, taps=None, dims=None)], width=48, embed_scale=None)   # no convolution, no turn
ONLY_CONV_ONE_TAP = model([conv_attention(heads=2, kv_heads=1, dim=32, taps=1, dims=32, base=300.0)], width=32)
ONLY_CONV_LONG = model([conv_attention(heads=2, kv_heads=2, dim=8, taps=7, dims=2)], width=40)
ONLY_CONV_MANY_TAPS = model([conv_attention(heads=2, kv_heads=1, dim=8, taps=13, dims=4)], width=24)     # more taps than the four-channel kernel takes
ONLY_WINDOW = model([window_attention()])
ONLY_WINDOW_NO_KEEP = model([window_attention(heads=3, kv_heads=1, dim=24, vdim=8, window=6, keep=None, dims=8)], width=48)
ONLY_WINDOW_OPEN = model([window_attention(heads=2, kv_heads=2, dim=16, vdim=16, window=None, dims=None)], width=32)    # plain causal, no turn
ONLY_WINDOW_KEEP_WIDE = model([window_attention(heads=2, kv_heads=1, dim=16, vdim=32, window=4, keep=11, dims=4)], width=32)   # more kept than the window holds
ONLY_SINK = model([sink_attention()])
ONLY_SINK_ONE_HEAD = model([sink_attention(heads=1, kv_heads=1, dim=40, vdim=24)], width=40)
ONLY_SINK_MANY = model([sink_attention(heads=12, kv_heads=3, dim=8, vdim=8)], width=96)
SHARED_KV = model([sink_attention(), sink_attention(kv_from=0)])
ONLY_DENSE = model([sink_attention(mlp=dense())])
ONLY_EXPERTS = model([sink_attention(mlp=moe())])
ONLY_EXPERTS_ALL = model([conv_attention(mlp=moe(experts=3, top=3, ff=16, shared=None, limit=0.75))], width=32)      # every expert chosen, no shared one
ONE_EXPERT = model([window_attention(mlp=moe(experts=1, top=1, ff=32, shared=16, limit=3.0, shared_limit=0.5))], width=32)
TOP_ONE = model([sink_attention(mlp=moe(experts=6, top=1, ff=16, shared=24))], width=32)
# several layers in orders of their own; layers that read the keys and values of a layer further back, two of them the
# same one; a layer without a feed-forward between layers with one
MIXED_A = model([
    sink_attention(mlp=moe()),
    conv_attention(mlp=dense(40)),
    window_attention(window=13, keep=5, mlp=moe(experts=6, top=1, ff=16, shared=24, limit=1.0, shared_limit=2.0)),
    sink_attention(kv_from=0),
    conv_attention(heads=2, kv_heads=1, dim=32, taps=2, dims=16, mlp=moe(experts=5, top=4, ff=8, shared=None)),
    sink_attention(kv_from=0, mlp=dense(72)),
], vocab=257, width=64, eps=1e-6)
MIXED_B = model([
    window_attention(heads=1, kv_heads=1, dim=48, vdim=16, window=33, keep=2, dims=24, base=500.0),
    window_attention(heads=6, kv_heads=3, dim=8, vdim=8, window=3, keep=0, mlp=dense(96), dims=8),
    conv_attention(heads=6, kv_heads=1, dim=16, taps=4, dims=16, mlp=moe(experts=7, top=3, ff=16, shared=32)),
    sink_attention(heads=2, kv_heads=2, dim=24, vdim=40, mlp=moe(experts=3, top=2, ff=24)),
    sink_attention(heads=2, kv_heads=2, dim=24, vdim=40, kv_from=3),
], vocab=513, width=48, embed_scale=0.25)
# scores that single keys dominate (a large scale): a window that is one key off, a kept token that is lost, a key
# lost at a page's border or a sink that is left out changes a row
PEAKED = model([window_attention(window=5, keep=2, scale=1.5), window_attention(window=16, keep=7, scale=1.5, heads=2, kv_heads=1, vdim=16),
                conv_attention(scale=1.2), sink_attention(scale=1.5)], width=32)
# scores near zero, so that the extra term of the denominator weighs as much as a key: a sink that is left out, not
# scaled or counted twice changes every row
SINK_SOFT = model([conv_attention(scale=0.02), sink_attention(scale=0.02)], width=32)
# the same at the head sizes that the matrix-core tiles and the split-key kernel take in bfloat16 (32, 64, 128; keys and
# values of one width), one layer each so that a row shows its own mask
PEAKED_TILES_32 = model([window_attention(window=9, keep=3, scale=0.8, heads=4, kv_heads=2, dim=32, vdim=32, dims=32)], width=64)
PEAKED_TILES_64 = model([window_attention(window=70, keep=23, scale=0.6, heads=2, kv_heads=1, dim=64, vdim=64, dims=32)], width=64)
PEAKED_TILES_128 = model([window_attention(window=3, keep=130, scale=0.4, heads=2, kv_heads=2, dim=128, vdim=128, dims=64)], width=32)
SINK_TILES_64 = model([sink_attention(heads=4, kv_heads=2, dim=64, vdim=64, scale=0.5)], width=64)
CONV_TILES_128 = model([conv_attention(heads=2, kv_heads=1, dim=128, taps=4, dims=32, scale=0.3)], width=64)
# hundreds of keys: a conv attention that sees everything, a window of 300 that keeps 40, a head whose distance
# penalty is slight: a token far back carries a row
PEAKED_FAR = model([conv_attention(scale=1.2, heads=2, kv_heads=1), window_attention(window=300, keep=40, scale=1.5),
                    sink_attention(heads=16, kv_heads=4, dim=8, vdim=8, scale=2.0)], width=32)
# sizes that are multiples of neither 8 nor 4; a width that is odd
ODD = model([
    conv_attention(heads=3, kv_heads=1, dim=10, taps=5, dims=6, mlp=moe(experts=5, top=2, ff=13, shared=7)),
    window_attention(heads=3, kv_heads=3, dim=6, vdim=9, window=30, keep=1, dims=2),
    sink_attention(heads=2, kv_heads=1, dim=7, vdim=5, mlp=dense(19)),
    sink_attention(heads=2, kv_heads=1, dim=7, vdim=5, kv_from=2, mlp=moe(experts=3, top=1, ff=9, shared=None)),
], vocab=101, width=43)
# head sizes between the kernels' own: keys of 96 with narrower values (the values widened), keys of 80 and of 48 with
# WIDER values (the keys widened, with the unit norm's eps and the score's scale adjusted), the latter read by a second
# layer, six heads over three
UNUSUAL = model([
    window_attention(heads=2, kv_heads=1, dim=96, vdim=32, window=40, keep=9, dims=48, mlp=dense(80)),
    window_attention(heads=2, kv_heads=2, dim=80, vdim=112, window=21, keep=33, dims=80, mlp=moe(experts=9, top=3, ff=40, shared=24)),
    sink_attention(heads=6, kv_heads=3, dim=48, vdim=64, mlp=dense(64)),
    conv_attention(heads=2, kv_heads=1, dim=96, taps=2, dims=64, mlp=moe(experts=2, top=1, ff=56, shared=None)),
    sink_attention(heads=6, kv_heads=3, dim=48, vdim=64, kv_from=2, mlp=dense(64)),
], vocab=333, width=96)
# the sizes of a larger model's layers: heads of 64 and 128, pages of many sizes
LARGER = model([
    conv_attention(heads=4, kv_heads=2, dim=64, taps=4, dims=32, mlp=moe(experts=6, top=2, ff=96, shared=160)),
    window_attention(heads=4, kv_heads=2, dim=64, vdim=64, window=100, keep=26, dims=64, mlp=dense(384)),
    sink_attention(heads=2, kv_heads=1, dim=128, vdim=128, mlp=moe(experts=6, top=2, ff=96, shared=160)),
    sink_attention(heads=2, kv_heads=1, dim=128, vdim=128, kv_from=2),
    window_attention(heads=8, kv_heads=2, dim=32, vdim=48, window=150, keep=17, dims=16, mlp=dense(256)),
], vocab=211, width=256)

# rms(difference, mean taken off) / rms(logits, mean taken off) of a row may be at most this
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
TOL_PEAKED = 1e-4

_plain: Dict[tuple, np.ndarray] = {}
_weights: Dict[str, tuple] = {}


def plain_model(model_dir):
    if model_dir not in _weights:
        _weights[model_dir] = ps.read_model(model_dir)
    return _weights[model_dir]


def plain_logits(model_dir, toks) -> np.ndarray:
    key = (model_dir, tuple(toks))
    if key not in _plain:
        cfg, w = plain_model(model_dir)
        _plain[key] = ps.logits(cfg, w, list(toks)).numpy()
    return _plain[key]


_calls: Dict[tuple, np.ndarray] = {}
CLOSE_CALL = 0.02       # a gap between two experts' scores below which bfloat16 rounding may choose the other one
CLOSE_REACH = 8         # positions behind such a token that still carry it most: the convolutions read the last few
                        # inputs; attention reads every earlier token, but thinly


def closest_call(model_dir, toks) -> np.ndarray:
    key = (model_dir, tuple(toks))
    if key not in _calls:
        cfg, w = plain_model(model_dir)
        _calls[key] = ps.closest_call(cfg, w, list(toks)).numpy()
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
    since rounding may rightly choose the other expert there, and neither are the CLOSE_REACH tokens behind it
    (the same rows differ in every schedule; 32-bit compares every row)."""
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
