"""A plain, slow Kegorax decoder in numpy float64: whole sequences, no cache, no state.

One function per mechanism, each written from its equation; nothing here knows of pages,
slots, batches or kernels, and nothing is shared with the engine.  The tests compare what the
engine does, however its work is cut, with these functions run over the whole sequence.

Notation: ``T`` tokens, ``E`` width; a mixer has ``H`` heads with keys of ``D`` and values of ``Dv``
channels (``G`` key heads where they are fewer).  Weights are ``[out, in]`` and applied as ``W x``.
``cfg`` is config.json as a dict, ``w`` a dict name -> float64 array.
"""
from __future__ import annotations

import math

import numpy as np


# ----------------------------------------------------------------------------- small pieces
def rms_div(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ----------------------------------------------------------------------------- attention
def rotate_half(x, base, dims):
    """``x [T, heads, D]`` at positions 0..T-1: channel i < dims/2 turns with channel i + dims/2 by the angle
    ``p * base^(-2i/dims)``; channels from ``dims`` on pass."""
    T = x.shape[0]
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = np.arange(T)[:, None] * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def visible(T, mask):
    """``[T, T]`` bool: may query i read key j.  ``mask``: {} (causal), {"size"} with ``chunked`` (same chunk of
    ``size`` positions counted from 0) or a sliding window of ``size`` that also keeps the first ``keep_first``."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    ok = j <= i
    if not mask:
        return ok
    size = mask["size"]
    if mask.get("chunked"):
        return ok & (i // size == j // size)
    return ok & ((i - j < size) | (j < mask.get("keep_first", 0)))


def attention_heads(q, k, v, scale, see, sink=None, slopes=None):
    """``q [T, H, D]``, ``k [T, G, D]``, ``v [T, G, Dv]`` -> ``[T, H, Dv]``.  Head h reads key head ``h // (H / G)``.
    Score ``(q . k) scale - slope_h (i - j)``; softmax over the visible keys whose denominator also holds
    ``exp(sink_h)``, an entry without a value (``sink`` None: no such entry)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    dist = np.arange(T)[:, None] - np.arange(T)[None, :]
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if slopes is not None:
            s = s - slopes[h] * dist
        s = np.where(see, s, -np.inf)
        m = s.max(axis=1, keepdims=True)
        if sink is not None:
            m = np.maximum(m, sink[h])
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def chunked_sink_attention(h, w, p, m):
    """The left side of a "parallel" mixer: rotated queries and keys, chunked mask, a learned sink a head,
    a sigmoid gate a head on the heads' outputs."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, G, D)
    v = (h @ w[p + "v"].T).reshape(T, G, Dv)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q, k = rotate_half(q, rot["base"], rot["dims"]), rotate_half(k, rot["base"], rot["dims"])
    see = visible(T, {"size": m["mask"]["size"], "chunked": True})
    o = attention_heads(q, k, v, m["scale"], see, sink=w[p + "sink"])
    o = o * sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * Dv) @ w[p + "o"].T


def distance_slopes(H):
    return np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])


def windowed_bias_attention(h, w, p, m, eps):
    """The left side of a "parallel_2" mixer: biased projections, queries and keys normed head by head, no
    rotation, a bias that grows with the distance, a sliding window that keeps the first tokens, one added to
    the softmax's denominator."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, Dv)
    q = rms_div(q, eps) * w[p + "q.norm"]
    k = rms_div(k, eps) * w[p + "k.norm"]
    see = visible(T, {"size": m["mask"]["size"], "keep_first": m["mask"].get("keep_first", 0)})
    o = attention_heads(q, k, v, m["scale"], see, sink=np.zeros(H), slopes=distance_slopes(H))
    return o.reshape(T, H * Dv) @ w[p + "o"].T


# ----------------------------------------------------------------------------- recurrences
def decay_recurrence(q, k, v, decay):
    """One head: ``S <- diag(decay_t) S + k_t v_t^T``, ``o_t = S^T q_t`` after the update.  ``decay [T, D]``
    (or ``[T, 1]`` for one number a token); S starts at zero."""
    T, D = q.shape
    S = np.zeros((D, v.shape[1]))
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = decay[t][:, None] * S + np.outer(k[t], v[t])
        o[t] = S.T @ q[t]
    return o


def delta_recurrence(q, k, v, beta, g):
    """One head of the gated delta rule: ``S <- diag(g_t) S; u = beta_t (v_t - S^T k_t); S <- S + k_t u^T;
    o_t = S^T q_t``."""
    T, D = q.shape
    S = np.zeros((D, v.shape[1]))
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o


def gated_linear_attention(h, w, p, m, eps):
    """The right side of a "parallel" mixer: a decay a token and key channel, ``sigmoid(z)^(1/tau)``."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, Dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, D)
    o = np.stack([decay_recurrence(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], axis=1)
    o = rms_div(o, eps) * w[p + "norm"]
    return (o.reshape(T, H * Dv) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def retention(h, w, p, m, eps):
    """The right side of a "parallel_2" mixer: one fixed decay a head, keys times D^-1/2."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, H, D) * D ** -0.5
    v = (h @ w[p + "v"].T).reshape(T, H, Dv)
    o = np.stack([decay_recurrence(q[:, i], k[:, i], v[:, i], np.full((T, 1), m["decay"][i])) for i in range(H)], axis=1)
    o = rms_div(o, eps)
    return (o.reshape(T, H * Dv) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def causal_conv_silu(x, taps_w):
    """``x [T, C]`` through a convolution over time a channel, ``taps_w [C, taps]`` with the last column the
    token's own, zeros before the start; then SiLU."""
    T, C = x.shape
    taps = taps_w.shape[1]
    y = np.zeros_like(x)
    for j in range(taps):
        back = taps - 1 - j
        y[back:] += x[:T - back] * taps_w[:, j]
    return silu(y)


def channel_delta(h, w, p, m, eps):
    """The "channel_delta" mixer."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ w[p + "q"].T, w[p + "q.conv"]).reshape(T, G, D)
    k = causal_conv_silu(h @ w[p + "k"].T, w[p + "k.conv"]).reshape(T, G, D)
    v = causal_conv_silu(h @ w[p + "v"].T, w[p + "v.conv"]).reshape(T, H, Dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w[p + "b"].T)
    x = ((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, D)
    g = np.exp(-np.exp(w[p + "A_log"])[None, :, None] * softplus(x))
    o = np.stack([delta_recurrence(q[:, i // (H // G)], k[:, i // (H // G)], v[:, i], beta[:, i], g[:, i])
                  for i in range(H)], axis=1)
    o = rms_div(o, eps) * w[p + "norm"]
    gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T)
    return (o.reshape(T, H * Dv) * gate) @ w[p + "o"].T


# ----------------------------------------------------------------------------- mixers of two
def parallel_mixer(h, w, p, m, eps):
    left = chunked_sink_attention(h, w, p + "left.", m["left"])
    right = gated_linear_attention(h, w, p + "right.", m["right"], eps)
    return 0.5 * (rms_div(left, eps) * w[p + "left.out"] + rms_div(right, eps) * w[p + "right.out"])


def parallel_2_mixer(h, w, p, m, eps):
    left = windowed_bias_attention(h, w, p + "left.", m["left"], eps)
    right = retention(h, w, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ----------------------------------------------------------------------------- feed-forwards
def dense_ff(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(z, correction, top, groups, keep, scale):
    """From router logits ``z [n]``: (chosen experts, their weights).  Scores ``sigmoid(z)``; the choice is by
    score + correction among the experts of the ``keep`` groups (of ``groups`` equal groups of neighbours) whose
    two best choice scores add up highest; weights are the scores times ``scale``."""
    s = sigmoid(z)
    c = s + correction
    n = len(z)
    per = n // groups
    gs = np.array([np.sort(c[g * per:(g + 1) * per])[::-1][:2].sum() for g in range(groups)])
    kept = np.argsort(-gs, kind="stable")[:keep]
    masked = np.full(n, -np.inf)
    for g in kept:
        masked[g * per:(g + 1) * per] = c[g * per:(g + 1) * per]
    chosen = np.argsort(-masked, kind="stable")[:top]
    return chosen, s[chosen] * scale


def route_margin(z, correction, top, groups, keep):
    """By how much the choice of ``route`` is decided: the smaller of the gap between the last kept group's score
    and the next group's, and the gap between the last chosen expert's choice score and the next one's among the
    kept groups' experts (infinite where there is no next).  A computation in fewer bits may choose otherwise
    where this is within its rounding."""
    c = sigmoid(z) + correction
    n = len(z)
    per = n // groups
    gs = np.array([np.sort(c[g * per:(g + 1) * per])[::-1][:2].sum() for g in range(groups)])
    order = np.argsort(-gs, kind="stable")
    gap = gs[order[keep - 1]] - gs[order[keep]] if keep < groups else np.inf
    allowed = np.sort(np.concatenate([c[g * per:(g + 1) * per] for g in order[:keep]]))[::-1]
    if top < len(allowed):
        gap = min(gap, allowed[top - 1] - allowed[top])
    return gap


def moe_ff(h, w, p, mlp, choices=None):
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    logits = h @ w[p + "router"].T
    for t in range(h.shape[0]):
        chosen, wts = route(logits[t], w[p + "correction"], r["top"], groups["count"], groups["keep"], r["scale"])
        if choices is not None:
            choices.append((logits[t], chosen, route_margin(logits[t], w[p + "correction"], r["top"], groups["count"], groups["keep"])))
        for e, a in zip(chosen, wts):
            q = f"{p}e{e}."
            out[t] += a * ((silu(h[t] @ w[q + "gate"].T) * (h[t] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out


# ----------------------------------------------------------------------------- the model
def run_order(cfg):
    """(layer, pass number if the layer is the first of a pass over the looped span else None)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["stop"] <= loop["start"]:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def forward(cfg, w, tokens, taps=None, choices=None):
    """Logits ``[T, vocab]`` of the whole sequence.  ``taps``: a list that receives the residual stream after
    every layer run; ``choices``: one that receives (router logits, chosen experts, ``route_margin``) of every routed token."""
    eps = cfg["norm"]["eps"]
    scale = (cfg.get("embedding") or {}).get("scale", 1.0)
    x0 = w["embed"][np.asarray(tokens)] * scale
    x = x0.copy()
    for i, enters in run_order(cfg):
        layer = cfg["layers"][i]
        p = f"l{i}."
        if enters is not None:
            if enters > 0:
                x = x + x0
            x = x + w["loop.step"][enters]
        h = rms_div(x, eps) * w[p + "norm1"]
        kind = layer["type"]
        if kind == "parallel":
            x = x + parallel_mixer(h, w, p + "mix.", layer["mixer"], eps)
        elif kind == "parallel_2":
            x = x + parallel_2_mixer(h, w, p + "mix.", layer["mixer"], eps)
        elif kind == "channel_delta":
            x = x + channel_delta(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(kind)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_div(x, eps) * w[p + "norm2"]
            x = x + (dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(h, w, p + "mlp.", mlp, choices))
        if taps is not None:
            taps.append(x.copy())
    return (rms_div(x, eps) * w["final.norm"]) @ w["embed"].T
