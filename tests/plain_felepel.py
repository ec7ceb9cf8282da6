"""A plain, slow implementation of the Felepel design: whole sequences, no cache, float64, one function per
mechanism.  It is what the tests hold the engine against and shares nothing with the library's code.

Notation: ``x`` [T, W] is the residual stream of one sequence, ``cfg`` the dict of config.json, ``w`` a dict of
float64 arrays by checkpoint tensor name.
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x: np.ndarray, weight: np.ndarray | None, eps: float) -> np.ndarray:
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if weight is None else y * weight


def silu(z: np.ndarray) -> np.ndarray:
    return z / (1.0 + np.exp(-z))


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z: np.ndarray) -> np.ndarray:
    return np.logaddexp(0.0, z)


def embed(tokens, w, first_position: int = 0) -> np.ndarray:
    tokens = np.asarray(tokens)
    pos = np.arange(first_position, first_position + len(tokens))
    return w["embed"][tokens] + w["pos"][pos]


# ---------------------------------------------------------------- attention with capped scores, a distance term, chunks
def attention_scores_mask(T: int, chunk: int | None) -> np.ndarray:
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    ok = j <= i
    if chunk:
        ok &= (i // chunk) == (j // chunk)
    return ok


def chunked_attention(h: np.ndarray, m: dict, w: dict, p: str) -> np.ndarray:
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    ok = attention_scores_mask(T, (m.get("mask") or {}).get("size"))
    dist = np.maximum(np.arange(T)[:, None] - np.arange(T)[None, :], 0).astype(np.float64)
    out = np.zeros((T, H, V))
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        cap = m.get("softcap")
        if cap:
            s = cap * np.tanh(s / cap)
        if p + "r1" in w:
            s = s - w[p + "r1"][hh] * np.log1p(w[p + "r2"][hh] * dist)
        s = np.where(ok, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        e = np.exp(s)
        out[:, hh] = (e / e.sum(axis=1, keepdims=True)) @ v[:, g]
    return out.reshape(T, H * V) @ w[p + "o"].T + w[p + "o.b"]


# ---------------------------------------------------------------- the gated delta rule with a decay per key channel
def short_conv(x: np.ndarray, taps: np.ndarray) -> np.ndarray:
    """y[t, c] = sum_j taps[c, j] * x[t - (K - 1) + j, c], zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C)), x])
    y = np.zeros((T, C))
    for j in range(K):
        y += padded[j:j + T] * taps[:, j]
    return y


def unit(x: np.ndarray) -> np.ndarray:
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def channel_delta(h: np.ndarray, m: dict, w: dict, p: str, eps: float, state=None, return_state: bool = False):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, D)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, D)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, V)
    q = unit(q) * D ** -0.5
    k = unit(k)
    beta = sigmoid(h @ w[p + "b"].T)                                           # [T, H]
    a = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]                 # [T, H * D]
    decay = np.exp(-np.exp(w[p + "A_log"])[None, :, None] * softplus(a).reshape(T, H, D))
    gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, V)
    S = np.zeros((H, D, V)) if state is None else state.copy()
    o = np.zeros((T, H, V))
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            S[hh] *= decay[t, hh][:, None]
            u = beta[t, hh] * (v[t, hh] - S[hh].T @ k[t, g])
            S[hh] += np.outer(k[t, g], u)
            o[t, hh] = S[hh].T @ q[t, g]
    o = rms_norm(o, w[p + "norm"], eps) * gate
    out = o.reshape(T, H * V) @ w[p + "o"].T
    return (out, S) if return_state else out


# ---------------------------------------------------------------- experts chosen within the best groups
def route(h: np.ndarray, r: dict, router: np.ndarray):
    """ids [T, top] by descending score, weights [T, top], and the margin between the last chosen and the best
    left-out score among the experts that may be chosen."""
    z = h @ router.T
    z = z - z.max(axis=1, keepdims=True)
    s = np.exp(z)
    s /= s.sum(axis=1, keepdims=True)
    T, E = s.shape
    allowed = np.ones((T, E), dtype=bool)
    groups = r.get("groups")
    if groups and groups["count"] > 1:
        per = E // groups["count"]
        gs = s.reshape(T, groups["count"], per).max(axis=2)
        best = np.argsort(-gs, axis=1, kind="stable")[:, :groups["keep"]]
        keep = np.zeros((T, groups["count"]), dtype=bool)
        np.put_along_axis(keep, best, True, axis=1)
        allowed = np.repeat(keep, per, axis=1)
    masked = np.where(allowed, s, -1.0)
    order = np.argsort(-masked, axis=1, kind="stable")
    ids = order[:, :r["top"]]
    weights = np.take_along_axis(s, ids, axis=1)
    n_allowed = allowed.sum(axis=1)
    nxt = np.take_along_axis(masked, order[:, min(r["top"], E - 1):min(r["top"], E - 1) + 1], axis=1)[:, 0]
    margin = np.where(n_allowed > r["top"], weights[:, -1] - nxt, np.inf)
    return ids, weights, margin


def moe(h: np.ndarray, f: dict, w: dict, p: str) -> np.ndarray:
    ids, weights, _ = route(h, f["router"], w[p + "router"])
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t], weights[t]):
            pe = f"{p}e{e}."
            out[t] += wt * ((silu(h[t] @ w[pe + "gate"].T) * (h[t] @ w[pe + "up"].T)) @ w[pe + "down"].T)
    return out


# ---------------------------------------------------------------- the model
def layer_prefix(cfg: dict, i: int) -> str:
    j = cfg["layers"][i].get("weights_of")
    return f"l{i if j is None else j}."


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one sequence from its first token (and the stream behind every layer run)."""
    eps = cfg["norm"]["eps"]
    x = embed(tokens, w)
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = layer_prefix(cfg, i)
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            y = chunked_attention(h, layer["mixer"], w, p + "mix.")
        elif layer["type"] == "channel_delta":
            y = channel_delta(h, layer["mixer"], w, p + "mix.", eps)
        else:
            raise ValueError(f"unknown mixer {layer['type']!r}")
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = rms_norm(x, w[p + "norm2"], eps)
            x = x + rms_norm(moe(h, layer["mlp"], w, p + "mlp."), w[p + "norm2b"], eps)
        streams.append(x.copy())
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, np.stack(streams)) if return_layers else logits
