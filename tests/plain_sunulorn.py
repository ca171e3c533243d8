"""A plain, slow Sunulorn: whole sequences, no cache, one function for each mechanism.

Sunulorn is a decoder-only model whose layers are listed in its configuration. A layer adds two results to the
residual stream, both computed from the same stream: a mixer behind one RMS norm and a feed-forward behind another.
A mixer is one of three softmax attentions with grouped heads:

* ``attention``: a short causal convolution over time on every channel of the projected queries and keys, the keys
  behind the convolution are also the values, rotary positions on interleaved column pairs, and a softmax whose
  denominator holds one more term, exp(0);
* ``attention_2``: biases, rotary positions on half-split column pairs, queries and keys scaled to unit root mean
  square per head behind the rotation, a sliding window that also keeps the sequence's first tokens, and a sigmoid
  gate per output column;
* ``attention_3``: biases, no rotation but a penalty that grows with the distance between query and key at a rate
  fixed per head, a learned extra term exp(sink_h) in the softmax's denominator, a sigmoid gate per head, and
  optionally the keys and values of an earlier layer instead of projections of its own.

The feed-forward is a gated one (silu) or a mixture of clamped gated experts chosen by sigmoid scores, the score
multiplying the expert's input, beside a shared expert that a sigmoid of the input scales. This file shares no code
with the engine: it parses config.json itself and reads the checkpoint with the ``safetensors`` package. Everything
is float64.

Notation: T tokens, D width, H heads, G key/value heads, d key size, e value size; ``h`` is a sub-layer's input
[T, D]; weights are stored [out, in] and applied as ``h @ W.T``.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List

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


def silu(z):
    return z * torch.sigmoid(z)


def causal_convolution(u, taps_w):
    """Per channel c: y[t, c] = sum_j taps_w[c, j] * u[t - (n - 1) + j, c] with n taps; rows before the sequence's
    start are zero, and the last tap multiplies the token's own row."""
    T, n = u.shape[0], taps_w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(n):
            s = t - (n - 1) + j
            if s >= 0:
                y[t] += taps_w[:, j] * u[s]
    return y


def angles(positions, base, dims):
    """[T, dims / 2]: position times base^(-2i / dims)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.tensor(positions, dtype=torch.float64)[:, None] * base ** (-2.0 * i / dims)[None, :]


def turn_interleaved(v, positions, base, dims):
    """v [T, heads, d]: columns 2i and 2i + 1 (i < dims / 2) form a pair that is turned by the position's angle;
    columns from dims on pass."""
    a = angles(positions, base, dims)
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = v.clone()
    x, y = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = x * c - y * s
    out[..., 1:dims:2] = y * c + x * s
    return out


def turn_half_split(v, positions, base, dims):
    """v [T, heads, d]: column i pairs with column i + dims / 2 (i < dims / 2); columns from dims on pass."""
    a = angles(positions, base, dims)
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    half = dims // 2
    out = v.clone()
    x, y = v[..., :half], v[..., half:dims]
    out[..., :half] = x * c - y * s
    out[..., half:dims] = y * c + x * s
    return out


def visible(T, mask):
    """[T, T] booleans: whether query position i (row) sees key position j (column): causal, and with a mask
    {size, keep_first} only the last `size` positions and the sequence's first `keep_first` ones."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    see = j <= i
    if mask is not None:
        see = see & ((i - j < mask["size"]) | (j < mask.get("keep_first", 0)))
    return see


def softmax_attention(q, k, v, scale, mask=None, slopes=None, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H, e]. Query head h reads key/value head h // (H / G).
    score = scale q.k - slopes[h] (i - j) over the visible keys; weights exp(score) / (sum exp(score) + exp(sink[h])),
    the last term only with a sink (it has no value)."""
    T, H, _ = q.shape
    G, e = k.shape[1], v.shape[2]
    see = visible(T, mask)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(q.dtype)
    out = torch.zeros(T, H, e, dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if slopes is not None:
            s = s - slopes[h] * dist
        s = s.masked_fill(~see, -math.inf)
        m = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h])
        p = torch.exp(s - m)
        denom = p.sum(-1, keepdim=True)
        if sink is not None:
            denom = denom + torch.exp(sink[h] - m)
        out[:, h] = (p / denom) @ v[:, g]
    return out


def project(h, w, name, bias):
    y = h @ w[name].T
    return y + w[name + ".b"] if bias else y


# -- the three mixers --------------------------------------------------------------------------------
def conv_attention_mixer(h, w, pre, m, eps):
    """'attention': queries and keys through a short convolution, values are the keys behind it, interleaved turn,
    one more term exp(0) in the denominator."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q, k = project(h, w, pre + "q", False), project(h, w, pre + "k", False)
    if m.get("conv"):
        q, k = causal_convolution(q, w[pre + "q.conv"]), causal_convolution(k, w[pre + "k.conv"])
    v = k.view(T, G, d)
    q, k = q.view(T, H, d), k.view(T, G, d)
    pos = list(range(T))
    rot = m.get("rot")
    if rot:
        q = turn_interleaved(q, pos, rot["base"], rot["dims"])
        k = turn_interleaved(k, pos, rot["base"], rot["dims"])
    o = softmax_attention(q, k, v, m["scale"], sink=torch.zeros(H, dtype=h.dtype))
    return o.reshape(T, H * d) @ w[pre + "o"].T


def window_attention_mixer(h, w, pre, m, eps):
    """'attention_2': biases, half-split turn, unit root mean square per head behind it, window with kept first
    tokens, a gate per output column."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = project(h, w, pre + "q", True).view(T, H, d)
    k = project(h, w, pre + "k", True).view(T, G, d)
    v = project(h, w, pre + "v", True).view(T, G, e)
    pos = list(range(T))
    rot = m.get("rot")
    if rot:
        q = turn_half_split(q, pos, rot["base"], rot["dims"])
        k = turn_half_split(k, pos, rot["base"], rot["dims"])
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    o = softmax_attention(q, k, v, m["scale"], mask=m.get("mask")).reshape(T, H * e)
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T + w[pre + "o.b"]


def head_slopes(H):
    return [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]


def keys_values_3(h, w, pre, m):
    T = h.shape[0]
    G, d, e = m["kv_heads"], m["dim"], m["vdim"]
    return project(h, w, pre + "k", True).view(T, G, d), project(h, w, pre + "v", True).view(T, G, e)


def sink_attention_mixer(h, w, pre, m, eps, kv=None):
    """'attention_3': biases, a distance penalty per head, a learned sink, a gate per head. `kv`: keys and values
    of the layer that `kv_from` names (this layer then has no projections for them)."""
    T = h.shape[0]
    H, e = m["heads"], m["vdim"]
    q = project(h, w, pre + "q", True).view(T, H, m["dim"])
    k, v = kv if kv is not None else keys_values_3(h, w, pre, m)
    o = softmax_attention(q, k, v, m["scale"], slopes=head_slopes(H), sink=w[pre + "sink"])
    o = o * torch.sigmoid(h @ w[pre + "g"].T)[:, :, None]
    return o.reshape(T, H * e) @ w[pre + "o"].T


# -- feed-forwards -----------------------------------------------------------------------------------
def dense_ff(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def clamped_expert(h, w, pre, limit):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def router_scores(h, w, pre):
    return torch.sigmoid(h @ w[pre + "router"].T)


def chosen_experts(scores, top):
    """Per token the indices of the `top` largest scores (the lower index wins a tie)."""
    out = []
    for row in scores:
        order = sorted(range(len(row)), key=lambda e: (-float(row[e]), e))
        out.append(order[:top])
    return out


def routed_experts(h, w, pre, mlp):
    scores = router_scores(h, w, pre)
    chosen = chosen_experts(scores, mlp["router"]["top"])
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t]:
            y[t] += clamped_expert(scores[t, e] * h[t:t + 1], w, pre + "e%d." % e, mlp["expert"]["limit"])[0]
    shared = mlp.get("shared")
    if shared:
        y = y + torch.sigmoid(h @ w[pre + "shared.sg"].T) * clamped_expert(h, w, pre + "shared.", shared["limit"])
    return y


def feed_forward(h, w, pre, mlp):
    if mlp is None:
        return torch.zeros_like(h)
    return dense_ff(h, w, pre) if mlp.get("kind", "dense") == "dense" else routed_experts(h, w, pre, mlp)


# -- the model ---------------------------------------------------------------------------------------
def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


def layer(x, w, i, lc, cfg, kept):
    """x + mixer(norm1(x)) + ff(norm2(x)). `kept`: the keys and values that 'attention_3' layers made, by layer."""
    eps = cfg["norm"]["eps"]
    L = "l%d." % i
    m = lc["mixer"]
    h = rms_norm(x, w[L + "norm1"], eps)
    if lc["type"] == "attention":
        y = conv_attention_mixer(h, w, L + "mix.", m, eps)
    elif lc["type"] == "attention_2":
        y = window_attention_mixer(h, w, L + "mix.", m, eps)
    elif lc["type"] == "attention_3":
        if m.get("kv_from") is None:
            kept[i] = keys_values_3(h, w, L + "mix.", m)
            y = sink_attention_mixer(h, w, L + "mix.", m, eps)
        else:
            y = sink_attention_mixer(h, w, L + "mix.", m, eps, kv=kept[m["kv_from"]])
    else:
        raise ValueError(lc["type"])
    if lc.get("mlp") is not None:
        y = y + feed_forward(rms_norm(x, w[L + "norm2"], eps), w, L + "mlp.", lc["mlp"])
    return x + y


def streams(cfg, w, tokens: List[int]):
    """The residual stream behind every layer, [layers, T, D]."""
    x = w["embed"][torch.tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    kept, out = {}, []
    for i, lc in enumerate(cfg["layers"]):
        x = layer(x, w, i, lc, cfg, kept)
        out.append(x)
    return torch.stack(out)


def logits(cfg, w, tokens: List[int]):
    x = streams(cfg, w, tokens)[-1]
    return rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T


def closest_call(cfg, w, tokens: List[int]):
    """Per token the smallest gap between the last chosen and the first rejected router score over all routed
    layers (a tiny gap means rounding may choose another expert there)."""
    x = w["embed"][torch.tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    kept = {}
    gap = torch.full((len(tokens),), math.inf, dtype=torch.float64)
    for i, lc in enumerate(cfg["layers"]):
        mlp = lc.get("mlp")
        if mlp is not None and mlp.get("kind") == "moe" and mlp["router"]["top"] < mlp["router"]["experts"]:
            s = router_scores(rms_norm(x, w["l%d.norm2" % i], cfg["norm"]["eps"]), w, "l%d.mlp." % i)
            srt = torch.sort(s, dim=-1, descending=True).values
            top = mlp["router"]["top"]
            gap = torch.minimum(gap, srt[:, top - 1] - srt[:, top])
        x = layer(x, w, i, lc, cfg, kept)
    return gap


def greedy_generate(cfg, w, prompt: List[int], n_new: int) -> List[int]:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(logits(cfg, w, toks)[-1])))
    return toks[len(prompt):]
