"""A plain, slow implementation of the Taminex design: float64, whole sequences, no cache, one function per mechanism.

It is written from the design's formulas and shares nothing with the library; the library's logits are held against it.
``w`` maps tensor names to float64 arrays; a linear weight is [out, in] and applied as ``W x``.

A layer:      x <- x + norm1(mixer(x));  x <- x + norm2(ff(x))        (the parts read x itself; a norm on outputs only)
norm:         y / sqrt(mean(y^2) + eps) * weight
attention:    q, k, v = W x + b;  every head of q and of k normed over its dim with a shared weight;  the first rot.dims
              dimensions of a head rotated in neighbouring pairs (2i, 2i+1) by the angle p * base^(-2i / dims);
              score = q . k * scale, j <= i;  softmax whose denominator also holds exp(sink_h);  W_o on the heads
delta:        q, k, v through a causal convolution per channel and silu;  q, k to unit length (q also * dim^-1/2);
              beta = sigmoid(W_b x);  g = exp(-exp(A_log_h) * softplus(W_a x + dt_bias_h));
              S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
              o / rms(o) * weight * silu(W_g x);  W_o
latent:       c = norm(W_dkv x) (or another layer's c);  k_h = W_uk,h c, v_h = W_uv,h c;  score = q_h . k_h * scale, j <= i;
              softmax;  heads * sigmoid(W_g x);  W_o
feed-forward: W_down relu(W_up x)^2
logits:       cap * tanh(embed . norm(x) * logit_scale / cap)
"""
from __future__ import annotations

import numpy as np


def rms_norm(y: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps) * weight


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def rotate_pairs(x: np.ndarray, positions: np.ndarray, dims: int, base: float) -> np.ndarray:
    """x [T, heads, dim]: dimensions 2i and 2i+1 (i < dims / 2) turned by positions * base^(-2i / dims)."""
    out = x.copy()
    for i in range(dims // 2):
        a = positions * base ** (-2.0 * i / dims)
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        u, v = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = u * c - v * s
        out[:, :, 2 * i + 1] = v * c + u * s
    return out


def causal_softmax(scores: np.ndarray, first: int, sink: float | None = None) -> np.ndarray:
    """scores [T, N]: row t (position first + t) sees columns 0 .. first + t.  ``sink``: exp(sink) joins every row's
    denominator.  Returns the weights, zeros where nothing is seen."""
    T, N = scores.shape
    out = np.zeros_like(scores)
    for t in range(T):
        row = scores[t, :first + t + 1]
        m = row.max() if sink is None else max(row.max(), sink)
        e = np.exp(row - m)
        out[t, :first + t + 1] = e / (e.sum() + (0.0 if sink is None else np.exp(sink - m)))
    return out


def attention(h: np.ndarray, m: dict, w: dict, p: str, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    q, k = rms_norm(q, w[p + "q.norm"], eps), rms_norm(k, w[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot is not None and rot["dims"] > 0:
        pos = np.arange(T, dtype=np.float64)
        q, k = rotate_pairs(q, pos, rot["dims"], rot["base"]), rotate_pairs(k, pos, rot["dims"], rot["base"])
    out = np.zeros((T, H, V))
    for head in range(H):
        g = head // (H // G)
        probs = causal_softmax(q[:, head] @ k[:, g].T * m["scale"], 0, float(w[p + "sink"][head]))
        out[:, head] = probs @ v[:, g]
    return out.reshape(T, H * V) @ w[p + "o"].T


def short_convolution(x: np.ndarray, taps: np.ndarray) -> np.ndarray:
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, j] x[t - (K - 1 - j), c], zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    y = np.zeros_like(x)
    for t in range(T):
        for j in range(K):
            back = K - 1 - j
            if t - back >= 0:
                y[t] += taps[:, j] * x[t - back]
    return y


def head_delta(h: np.ndarray, m: dict, w: dict, p: str, eps: float, return_state: bool = False, state=None):
    """``state`` [heads, dim, vdim]: what an earlier piece of the sequence left (the convolution starts anew all the same)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, D)
    k = silu(short_convolution(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, D)
    v = silu(short_convolution(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, V)
    q = q / np.sqrt(np.sum(q * q, axis=-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt(np.sum(k * k, axis=-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w[p + "b"].T)                                                    # [T, H]
    decay = np.exp(-np.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))      # [T, H]
    o = np.zeros((T, H, V))
    states = np.zeros((H, D, V))
    for head in range(H):
        g = head // (H // G)
        S = np.zeros((D, V)) if state is None else state[head].copy()
        for t in range(T):
            S = decay[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + np.outer(k[t, g], u)
            o[t, head] = S.T @ q[t, g]
        states[head] = S
    o = o / np.sqrt(np.mean(o * o, axis=-1, keepdims=True) + eps) * w[p + "norm"]
    out = (o.reshape(T, H * V) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T
    return (out, states) if return_state else out


def latent_of(h: np.ndarray, w: dict, p: str, eps: float) -> np.ndarray:
    return rms_norm(h @ w[p + "dkv"].T, w[p + "dkv.norm"], eps)


def latent_attention(h: np.ndarray, c: np.ndarray, m: dict, w: dict, p: str) -> np.ndarray:
    """``c`` [T, kv_rank]: the latents this layer attends over (its own, or another layer's)."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (c @ w[p + "uk"].T).reshape(T, H, D)
    v = (c @ w[p + "uv"].T).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for head in range(H):
        out[:, head] = causal_softmax(q[:, head] @ k[:, head].T * m["scale"], 0) @ v[:, head]
    return (out.reshape(T, H * V) * sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def feed_forward(h: np.ndarray, w: dict, p: str) -> np.ndarray:
    return np.maximum(h @ w[p + "up"].T, 0.0) ** 2 @ w[p + "down"].T


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of a whole sequence (and the residual stream behind every layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    latents, streams = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        if layer["type"] == "attention":
            y = attention(x, m, w, p, eps)
        elif layer["type"] == "delta":
            y = head_delta(x, m, w, p, eps)
        else:
            if m.get("kv_from") is None:
                latents[i] = latent_of(x, w, p, eps)
            y = latent_attention(x, latents[i if m.get("kv_from") is None else m["kv_from"]], m, w, p)
        x = x + rms_norm(y, w[f"l{i}.norm1"], eps)
        if layer["mlp"] is not None:
            x = x + rms_norm(feed_forward(x, w, f"l{i}.mlp."), w[f"l{i}.norm2"], eps)
        streams.append(x.copy())
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap")
    if cap is not None:
        logits = cap * np.tanh(logits / cap)
    return (logits, streams) if return_layers else logits
