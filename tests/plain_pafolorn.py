"""A plain, slow Pafolorn in NumPy float64: one function per mechanism, whole sequences only, nothing kept between
calls.  It is what the engine is compared with; it shares no code with it (the model folder is read with the
safetensors package, the formulas are written out here)."""
from __future__ import annotations

import json
import os

import numpy as np


def read_model_folder(folder):
    """config.json as a dict, tensors as float64 NumPy arrays by name."""
    import torch
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(torch.float64).numpy()
    return cfg, tensors


# --------------------------------------------------------------------------- small functions
def unit_rms(x, eps):
    """Rows scaled to a root mean square of one (eps under the root)."""
    return x / np.sqrt(np.mean(np.square(x), axis=-1, keepdims=True) + eps)


def unit_length(x, eps=1e-6):
    return x / np.sqrt(np.sum(np.square(x), axis=-1, keepdims=True) + eps)


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def swish(z):
    return z * logistic(z)


def soft_plus(z):
    return np.logaddexp(0.0, z)


def squared_ramp(z):
    return np.square(np.maximum(z, 0.0))


# --------------------------------------------------------------------------- mechanisms
def short_filter(x, taps):
    """x [T, C], taps [C, K]: y[t, c] = sum_k taps[c, k] x[t - (K - 1 - k), c], zeros before the sequence."""
    T, C = x.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C)), x], axis=0)
    y = np.zeros((T, C))
    for k in range(K):
        y += padded[k:k + T] * taps[:, k][None, :]
    return y


def turn_halves(v, places, n_turned, base):
    """v [T, heads, d]: entry i of the first ``n_turned`` is paired with entry i + n_turned / 2 and the pair is turned
    by the angle place * base^(-2i / n_turned); what lies behind passes."""
    out = v.copy()
    half = n_turned // 2
    if half == 0:
        return out
    speed = base ** (-2.0 * np.arange(half) / n_turned)
    ang = np.asarray(places, dtype=np.float64)[:, None] * speed[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = v[..., :half], v[..., half:n_turned]
    out[..., :half] = a * c - b * s
    out[..., half:n_turned] = b * c + a * s
    return out


def visible(T, window, keep_first, start=0):
    """[T, T] booleans: the query at row i (position start + i) sees the key at column j."""
    i = start + np.arange(T)[:, None]
    j = start + np.arange(T)[None, :]
    return (j <= i) & ((i - j < window) | (j < keep_first))


def delta_recurrence(q, k, v, beta, decay, S0=None):
    """One head.  q, k [T, D] (already of unit length, q scaled), v [T, Dv], beta [T], decay [T, D] (a row of S
    each).  Returns the read-outs [T, Dv] and the last S [D, Dv]."""
    T, D = q.shape
    S = np.zeros((D, v.shape[1])) if S0 is None else S0.copy()
    o = np.zeros_like(v)
    for t in range(T):
        S = decay[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def delta_mixer(W, p, m, h, eps, per_channel):
    """The gated delta rule of a layer; tensors under ``p``; m: heads, kv_heads, dim, vdim, conv."""
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = swish(short_filter(h @ W[p + "q"].T, W[p + "q.conv"])).reshape(T, G, D)
    k = swish(short_filter(h @ W[p + "k"].T, W[p + "k.conv"])).reshape(T, G, D)
    v = swish(short_filter(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(T, H, Dv)
    q = unit_length(q) * D ** -0.5
    k = unit_length(k)
    beta = logistic(h @ W[p + "b"].T)
    rate = np.exp(W[p + "A_log"])
    if per_channel:
        step = soft_plus((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).reshape(T, H, D)
        decay = np.exp(-rate[None, :, None] * step)
        gate = logistic((h @ W[p + "g1"].T) @ W[p + "g2"].T)
    else:
        step = soft_plus(h @ W[p + "a"].T + W[p + "dt_bias"])
        decay = np.repeat(np.exp(-rate[None, :] * step)[:, :, None], D, axis=2)
        gate = swish(h @ W[p + "g"].T)
    o = np.zeros((T, H, Dv))
    for i in range(H):
        o[:, i], _ = delta_recurrence(q[:, i // (H // G)], k[:, i // (H // G)], v[:, i], beta[:, i], decay[:, i])
    y = unit_rms(o, eps) * W[p + "norm"][None, None, :] * gate.reshape(T, H, Dv)
    return y.reshape(T, H * Dv) @ W[p + "o"].T


def attend(q, k, v, m, with_weights=False):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] of one whole sequence (already normalised and turned): capped scores,
    the window with its kept first tokens, softmax, weighted values [T, H, Dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    seen = visible(T, m["mask"]["size"], m["mask"]["keep_first"])
    cap = m.get("softcap") or 0.0
    o = np.zeros((T, H, v.shape[2]))
    weights = np.zeros((H, T, T))
    for i in range(H):
        g = i // (H // G)
        s = (q[:, i] @ k[:, g].T) * m["scale"]
        if cap > 0.0:
            s = cap * np.tanh(s / cap)
        s = np.where(seen, s, -np.inf)
        w = np.exp(s - s.max(axis=1, keepdims=True))
        weights[i] = w / w.sum(axis=1, keepdims=True)
        o[:, i] = weights[i] @ v[:, g]
    return (o, weights) if with_weights else o


def window_attention(W, p, m, h, eps, with_weights=False):
    """Softmax attention with grouped key heads, a norm over the whole query and key projections, a turn of the
    first rot.dims entries, a capped score, and a window that also keeps the first tokens."""
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    places = np.arange(T)
    q = (unit_rms(h @ W[p + "q"].T, eps) * W[p + "q.norm"]).reshape(T, H, D)
    k = (unit_rms(h @ W[p + "k"].T, eps) * W[p + "k.norm"]).reshape(T, G, D)
    v = (h @ W[p + "v"].T).reshape(T, G, Dv)
    q = turn_halves(q, places, m["rot"]["dims"], m["rot"]["base"])
    k = turn_halves(k, places, m["rot"]["dims"], m["rot"]["base"])
    o, w = attend(q, k, v, m, with_weights=True)
    y = o.reshape(T, H * Dv) @ W[p + "o"].T
    return (y, w) if with_weights else y


def dense_ff(W, p, h):
    return squared_ramp(h @ W[p + "up"].T) @ W[p + "down"].T


# --------------------------------------------------------------------------- the model
def forward(cfg, W, ids, with_layers=False):
    """Logits [T, V] of a whole sequence; with ``with_layers`` also the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = unit_rms(W["embed"][np.asarray(ids)], eps) * W["embed.norm"]
    after = []
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        if L["type"] == "channel_delta":
            y = delta_mixer(W, p + "mix.", m, x, eps, True)
        else:
            y = m["left_scale"] * window_attention(W, p + "mix.left.", m["left"], x, eps) \
                + m["right_scale"] * delta_mixer(W, p + "mix.right.", m["right"], x, eps, False)
        x = x + unit_rms(y, eps) * W[p + "norm1"] * W[p + "ls1"]
        if L.get("mlp") is not None:
            x = x + unit_rms(dense_ff(W, p + "mlp.", x), eps) * W[p + "norm2"] * W[p + "ls2"]
        after.append(x.copy())
    logits = (unit_rms(x, eps) * W["final.norm"]) @ W["embed"].T * cfg["logit_scale"]
    return (logits, after) if with_layers else logits


def forward_logits(cfg, W, ids):
    return forward(cfg, W, ids)


def greedy_generate(cfg, W, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(np.argmax(forward(cfg, W, ids)[-1])))
    return ids[len(prompt):]
