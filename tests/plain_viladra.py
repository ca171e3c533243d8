"""A plain, slow Viladra: whole sequences, no cache, one function for each mechanism.

Viladra is a decoder-only model whose layers are listed in its configuration. A sub-layer reads the residual
stream itself (plus a short causal convolution of it over time) and its result is RMS-normed before it is added
back. A mixer is linear attention with one fixed decay per head and rotated queries and keys ("retention"),
linear attention with a decay per key channel that a low-rank map of the input decides ("gla"), or windowed
attention whose weights are sigmoids of the scores instead of a softmax ("attention"). The feed-forward is a
mixture of small experts beside a shared one. What a layer hands on is a learned weighted sum of the embedding's
output and the results of all layers so far. This file shares no code with the engine: it parses config.json
itself and reads the checkpoint with the ``safetensors`` package. Everything is float64, token by token where
the mechanism is a recurrence.

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
    """Rotary turn of the first `dims` entries of the last dimension: entry i pairs with entry i + dims/2; at
    position p the pair (a, b) becomes (a cos - b sin, b cos + a sin) of the angle p * base^(-2i/dims). Entries
    from `dims` on pass unchanged. v: [T, heads, n]."""
    if dims == 0:
        return v
    half = dims // 2
    i = torch.arange(half, dtype=v.dtype)
    angle = positions.to(v.dtype)[:, None] * torch.pow(torch.tensor(float(base), dtype=v.dtype), -2.0 * i / dims)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], dim=-1)


def decayed_outer_sums(q, k, v, decay):
    """The linear-attention recurrence, token by token and head by head:
    S_t = diag(decay_t) S_(t-1) + k_t v_t^T (the decay scales the rows, which belong to key channels), o_t = S_t^T q_t.
    q, k: [T, H, d]; v: [T, H, e]; decay: [T, H, d]. Returns [T, H, e]."""
    T, H, d = q.shape
    e = v.shape[-1]
    out = torch.zeros(T, H, e, dtype=q.dtype)
    for hd in range(H):
        S = torch.zeros(d, e, dtype=q.dtype)
        for t in range(T):
            S = decay[t, hd][:, None] * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    return out


def retention_mixer(h, w, pre, m, eps):
    """Fixed decay per head, rotated queries and keys, keys scaled by d^(-1/2) after the turn; every head's result
    divided by its root mean square (no weight), times silu of a gate projection, then the output projection."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ w[pre + "q"].T).view(T, H, d)
    k = (h @ w[pre + "k"].T).view(T, H, d)
    v = (h @ w[pre + "v"].T).view(T, H, e)
    rot = m.get("rot") or {"base": 1.0, "dims": 0}
    q = turn_half_split(q, pos, rot["base"], rot["dims"])
    k = turn_half_split(k, pos, rot["base"], rot["dims"]) * d ** -0.5
    decay = torch.tensor(m["decay"], dtype=h.dtype)[None, :, None].expand(T, H, d)
    o = unit_rms(decayed_outer_sums(q, k, v, decay), eps).reshape(T, H * e)
    return (o * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def gla_mixer(h, w, pre, m, eps):
    """A decay per key channel, sigmoid(z)^(1/tau) with z from a low-rank map of the input; queries scaled by
    d^(-1/2); every head's result RMS-normed with one weight shared by the heads, times silu of a gate
    projection, then the output projection."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[pre + "k"].T).view(T, H, d)
    v = (h @ w[pre + "v"].T).view(T, H, e)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    decay = torch.exp(torch.nn.functional.logsigmoid(z) / m["tau"]).view(T, H, d)
    o = unit_rms(decayed_outer_sums(q, k, v, decay), eps) * w[pre + "norm"]
    return (o.reshape(T, H * e) * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def sigmoid_attention_mixer(h, w, pre, m, eps):
    """Windowed attention without a softmax: key j's weight for query i is sigmoid(scale q_i.k_j + pb_head) if
    0 <= i - j < window, else 0, and the weights are not normalised. Queries and keys are RMS-normed over their whole
    projections; biases on the projections; one sigmoid output gate per head."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms(h @ w[pre + "q"].T + w[pre + "q.b"], eps) * w[pre + "q.norm"]
    k = unit_rms(h @ w[pre + "k"].T + w[pre + "k.b"], eps) * w[pre + "k.norm"]
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).view(T, G, e)
    q, k = q.view(T, H, d), k.view(T, G, d)
    gate = torch.sigmoid(h @ w[pre + "g"].T)                    # [T, H]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (i - j >= 0) & (i - j < m["mask"]["size"])
    out = torch.zeros(T, H, e, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] + w[pre + "pb"][hd]
        p = torch.where(seen, torch.sigmoid(s), torch.zeros_like(s))
        out[:, hd] = (p @ v[:, g]) * gate[:, hd:hd + 1]
    return out.reshape(T, H * e) @ w[pre + "o"].T + w[pre + "o.b"]


def small_ff(h, w, pre):
    """W_down relu(W_up h)^2."""
    return torch.relu(h @ w[pre + "up"].T) ** 2 @ w[pre + "down"].T


def routed_experts(h, w, pre, mlp):
    """Every token goes to the `top` experts with the largest softmax scores (the lowest index wins a tie); their
    results are weighted by those scores times router.scale, not renormalised; a shared expert is added."""
    r = mlp["router"]
    scores = torch.softmax(h @ w[pre + "router"].T, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(r["experts"]), key=lambda x: (-float(scores[t, x]), x))[:r["top"]]
        for x in order:
            out[t] += scores[t, x] * r["scale"] * small_ff(h[t:t + 1], w, "%se%d." % (pre, x))[0]
    if mlp.get("shared") is not None:
        out = out + small_ff(h, w, pre + "shared.")
    return out


def chosen_experts(h, w, pre, mlp):
    """[T, top] expert indices per token and the gap between the last chosen score and the first one left out."""
    r = mlp["router"]
    scores = torch.softmax(h @ w[pre + "router"].T, dim=-1)
    srt = torch.sort(scores, dim=-1, descending=True).values
    gap = (srt[:, r["top"] - 1] - srt[:, r["top"]]) if r["top"] < r["experts"] else torch.ones(h.shape[0], dtype=h.dtype)
    return torch.topk(scores, r["top"], dim=-1).indices, gap


# -- the model ---------------------------------------------------------------------------------------
MIXERS = {"retention": retention_mixer, "gla": gla_mixer, "attention": sigmoid_attention_mixer}


def layer(x, w, i, lc, cfg, gaps=None):
    """x + norm1(mixer(x + conv1(x))), then the same with the feed-forward, if the layer has one. `gaps` (a list)
    collects, per layer with experts, how far each token's last chosen score lies above the first one left out."""
    eps = cfg["norm"]["eps"]
    L = "l%d." % i
    canon = cfg.get("canon") is not None
    h = input_convolution(x, w[L + "canon1"]) if canon else x
    x = x + unit_rms(MIXERS[lc["type"]](h, w, L + "mix.", lc["mixer"], eps), eps) * w[L + "norm1"]
    if lc.get("mlp") is not None:
        h = input_convolution(x, w[L + "canon2"]) if canon else x
        if gaps is not None:
            gaps.append(chosen_experts(h, w, L + "mlp.", lc["mlp"])[1])
        x = x + unit_rms(routed_experts(h, w, L + "mlp.", lc["mlp"]), eps) * w[L + "norm2"]
    return x


def streams(cfg, w, tokens: List[int], gaps=None):
    """The residual stream as every layer hands it on ([layers, T, D]) and the last one. What layer i hands on is
    sum_j dwa_i[j] X_j over X_0 (the embedding's output) and the results X_1 .. X_(i+1) of the layers so far."""
    x = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    kept = [x]
    handed = []
    for i, lc in enumerate(cfg["layers"]):
        kept.append(layer(x, w, i, lc, cfg, gaps))
        a = w["l%d.dwa" % i]
        x = sum(a[j] * kept[j] for j in range(i + 2))
        handed.append(x)
    return torch.stack(handed), x


def logits(cfg, w, tokens: List[int]):
    """[T, vocab]: final norm, the embedding table as the head, then cap * tanh(. / cap)."""
    _, x = streams(cfg, w, tokens)
    z = (unit_rms(x, cfg["norm"]["eps"]) * w["final.norm"]) @ w["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


def forward(cfg, w, tokens: List[int]):
    return logits(cfg, w, tokens)


def closest_call(cfg, w, tokens: List[int]):
    """[T]: per token, the smallest gap over the layers between the last chosen expert's score and the first one
    left out (1 where no layer has a choice to make). A token with a small gap is one whose experts a rounding can change."""
    gaps: List[torch.Tensor] = []
    streams(cfg, w, tokens, gaps)
    out = torch.ones(len(tokens), dtype=torch.float64)
    for g in gaps:
        out = torch.minimum(out, g)
    return out


def greedy_generate(cfg, w, prompt: List[int], n_new: int) -> List[int]:
    """n_new tokens, each the largest logit's (the lowest index on a tie) given everything before it."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(logits(cfg, w, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
