"""A plain, slow Dinasun decoder in numpy float64: whole sequences, no cache, no state.

One function per mechanism, each written from its equation; nothing here knows of pages,
slots, batches or kernels, and nothing is shared with the engine.  The tests compare what the
engine does, however its work is cut, with these functions run over the whole sequence.

Notation: ``T`` tokens, ``E`` width; a mixer has ``H`` heads of ``D`` channels (attention: ``G`` key
heads).  Weights are ``[out, in]`` and applied as ``W x``.
"""
from __future__ import annotations

import math

import numpy as np


# ----------------------------------------------------------------------------- small pieces
def rms_div(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def softmax(z):
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    return e / e.sum(axis=-1, keepdims=True)


def dyt(x, w, prefix):
    """Dynamic tanh: ``tanh(alpha x) * weight + bias``; no statistic of the row enters."""
    return np.tanh(float(w[prefix + ".alpha"]) * x) * w[prefix] + w[prefix + ".b"]


# ----------------------------------------------------------------------------- mixers
def shifted(h):
    """Row t is row t - 1 of ``h``; the first row is zero."""
    out = np.zeros_like(h)
    out[1:] = h[:-1]
    return out


def wkv_decay(xw, w, p):
    """The decay of every token, head and key channel from the decay's own mix ``xw [T, E]``:
    ``exp(-exp(W2 tanh(W1 xw) + w0))``."""
    return np.exp(-np.exp(np.tanh(xw @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"]))


def wkv_recurrence(r, k, v, decay, u):
    """Per head over ``[T, D]`` rows: ``o_t = (S + diag(u) k_t v_t^T)^T r_t`` from the state before the
    token, then ``S <- diag(decay_t) S + k_t v_t^T``; S starts at zero."""
    T, D = r.shape
    S = np.zeros((D, D))
    o = np.zeros((T, D))
    for t in range(T):
        kv = np.outer(k[t], v[t])
        o[t] = (S + u[:, None] * kv).T @ r[t]
        S = decay[t][:, None] * S + kv
    return o


def wkv(h, w, m, eps, p):
    """Time mixing: each of r, k, v, g and the decay reads ``h + (h_before - h) mu``; per head the
    recurrence above; every head's read-out over its root mean square, times a weight a channel,
    times ``silu(Wg ..)``, then ``Wo``."""
    H, D = m["heads"], m["dim"]
    T = h.shape[0]
    d = shifted(h) - h
    mix = {s: h + d * w[p + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ w[p + "r"].T).reshape(T, H, D)
    k = (mix["k"] @ w[p + "k"].T).reshape(T, H, D)
    v = (mix["v"] @ w[p + "v"].T).reshape(T, H, D)
    gate = silu(mix["g"] @ w[p + "g"].T)
    decay = wkv_decay(mix["w"], w, p).reshape(T, H, D)
    u = w[p + "u"].reshape(H, D)
    o = np.stack([wkv_recurrence(r[:, i], k[:, i], v[:, i], decay[:, i], u[i]) for i in range(H)], axis=1)
    o = rms_div(o, eps).reshape(T, H * D) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


def query_temperature(positions, coef, every):
    """``1 + coef ln(floor((p + 1) / every) + 1)`` for every position."""
    pos = np.asarray(positions, dtype=np.int64)
    return 1.0 + coef * np.log((pos + 1) // every + 1.0)


def distance_slopes(H):
    """``2^(-8 (h + 1) / H)`` for head h."""
    return np.asarray([2.0 ** (-8.0 * (i + 1) / H) for i in range(H)])


def attention(h, w, m, eps, p):
    """Causal softmax attention in which the values are the keys as projected; queries and keys are
    normed head by head (RMS, one weight for all heads), the queries warmed with their position, and
    ``slope_h (i - j)`` is taken off every score."""
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = k
    q = rms_div(q, eps) * w[p + "q.norm"]
    k = rms_div(k, eps) * w[p + "k.norm"]
    temp = m.get("q_temp")
    if temp is not None:
        q = q * query_temperature(np.arange(T), temp["coef"], temp["every"])[:, None, None]
    slopes = distance_slopes(H)
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    out = np.zeros((T, H, v.shape[-1]))
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"] - slopes[a] * (i - j)
        s = np.where(j <= i, s, -np.inf)
        out[:, a] = softmax(s) @ v[:, g]
    return out.reshape(T, -1) @ w[p + "o"].T


# ----------------------------------------------------------------------------- feed-forward
def expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def table_experts(h, tokens, w, mlp, p):
    """Every token's experts come from a table by its id, each with weight 1 / top; a shared expert
    runs for every token and is added."""
    top = mlp["router"]["top"]
    table = np.asarray(w[p + "table"]).astype(np.int64)
    out = np.zeros_like(h)
    for t, tok in enumerate(tokens):
        for e in table[int(tok)]:
            out[t] += expert(h[t], w, f"{p}e{int(e)}.") / top
    if mlp.get("shared") is not None:
        out = out + expert(h, w, p + "shared.")
    return out


# ----------------------------------------------------------------------------- the model
def run_order(cfg):
    """(layer, first of its pass?) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if loop is None:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    out = [(i, False) for i in range(a)]
    for _ in range(times):
        out += [(i, i == a) for i in range(a, b)]
    return out + [(i, False) for i in range(b, n)]


def forward(cfg, w, tokens, layers_out=None):
    """Logits ``[T, vocab]`` of the whole sequence.  ``layers_out``: a list that receives the residual
    stream after every layer run."""
    eps = cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    x = w["embed"][np.asarray(tokens, dtype=np.int64)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x0 = x
    for i, enters in run_order(cfg):
        layer, p = cfg["layers"][i], f"l{i}."
        if enters:
            x = np.concatenate([x, x0], axis=-1) @ w["loop.in"].T
        h = dyt(x, w, p + "norm1")
        mixer = wkv if layer["type"] == "wkv" else attention
        x = x + mult * dyt(mixer(h, w, layer["mixer"], eps, p + "mix."), w, p + "norm1b")
        if layer.get("mlp") is not None:
            h = dyt(x, w, p + "norm2")
            x = x + mult * dyt(table_experts(h, tokens, w, layer["mlp"], p + "mlp."), w, p + "norm2b")
        if layers_out is not None:
            layers_out.append(x.copy())
    return dyt(x, w, "final.norm") @ w["embed"].T
