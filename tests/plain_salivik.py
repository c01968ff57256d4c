"""A plain, slow Salivik in NumPy float64: one function per mechanism, whole sequences only, no cache and no
state kept between calls.  It is what the engine is compared with; it shares no code with it (the model folder
is read with the safetensors package, the formulas are written out here)."""
from __future__ import annotations

import json
import math
import os

import numpy as np


def read_model_folder(folder):
    """config.json as a dict, tensors as float64 (integer tables as int64) NumPy arrays by name."""
    import torch
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = t.to(torch.float64).numpy() if t.dtype.is_floating_point else t.to(torch.int64).numpy()
    return cfg, tensors


# --------------------------------------------------------------------------- small functions
def unit_rms(x, eps):
    """Rows scaled to a root mean square of one (eps under the root)."""
    return x / np.sqrt(np.mean(np.square(x), axis=-1, keepdims=True) + eps)


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def swish(z):
    return z * logistic(z)


# --------------------------------------------------------------------------- rotation
def turn_speeds(rot):
    """(speeds [dims / 2], length factor): base^(-2i / dims); with ``scaling`` the slow entries are slowed by
    ``factor`` along a ramp between two places found from the turns that fit into ``original`` positions, and
    sine and cosine grow by 0.1 ln(factor) + 1."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    speed = np.array([base ** (-2.0 * i / dims) for i in range(half)], dtype=np.float64)
    sc = rot.get("scaling")
    if not sc:
        return speed, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def place(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(place(sc["fast"])), 0)
    hi = min(math.ceil(place(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(half) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return speed / factor * ramp + speed * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn_halves(v, places, rot, single=False):
    """v [T, ..., d]: entry i of the first ``dims`` entries is paired with entry i + dims / 2 and the pair is turned
    by the angle place * speed_i; what lies behind passes.  ``single``: place, speed and angle are rounded to
    32-bit floats as a 32-bit program forms them."""
    dims = rot["dims"]
    half = dims // 2
    out = v.copy()
    if half == 0:
        return out
    speed, length = turn_speeds(rot)
    if single:
        ang = (np.asarray(places, dtype=np.float32)[:, None] * speed.astype(np.float32)[None, :]).astype(np.float64)
    else:
        ang = np.asarray(places, dtype=np.float64)[:, None] * speed[None, :]
    shape = (len(places),) + (1,) * (v.ndim - 2) + (half,)
    c, s = (np.cos(ang) * length).reshape(shape), (np.sin(ang) * length).reshape(shape)
    a, b = v[..., :half], v[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def window_mask(T, size):
    """[T, T] True where row i sees column j: 0 <= i - j < size."""
    d = np.arange(T)[:, None] - np.arange(T)[None, :]
    return (d >= 0) & (d < size)


def softmax_with_sink(scores, mask, sink):
    """Rows of weights exp(s_j) / (exp(sink) + sum over seen j of exp(s_j)); ``sink`` [..., 1] broadcasts."""
    s = np.where(mask, scores, -np.inf)
    m = np.maximum(s.max(axis=-1, keepdims=True), sink)
    e = np.where(mask, np.exp(s - m), 0.0)
    return e / (np.exp(sink - m) + e.sum(axis=-1, keepdims=True))


# --------------------------------------------------------------------------- mixers
def attention(W, p, m, h, single=False):
    """Softmax attention over a window with grouped key heads; a key, before it is turned, is also the value; the
    denominator holds one more term exp(0); the heads' results pass a logistic gate of the input."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    assert m["vdim"] == D
    places = np.arange(T)
    q = (h @ W[p + "mix.q"].T).reshape(T, H, D)
    k = (h @ W[p + "mix.k"].T).reshape(T, G, D)
    v = k
    q, k = turn_halves(q, places, m["rot"], single), turn_halves(k, places, m["rot"], single)
    mask = window_mask(T, m["mask"]["size"])
    out = np.zeros((T, H, D))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        w = softmax_with_sink(s, mask, np.zeros((T, 1)))
        out[:, hd] = w @ v[:, g]
    gate = logistic(h @ W[p + "mix.g"].T)
    return (out.reshape(T, H * D) * gate) @ W[p + "mix.o"].T


def retention(W, p, m, h, eps, single=False):
    """Per head S <- decay S + k v^T, o = S^T q, token by token from S = 0; o scaled to a root mean square of one,
    times swish(W_g h), projected."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    places = np.arange(T)
    q = turn_halves((h @ W[p + "mix.q"].T).reshape(T, H, D), places, m["rot"], single)
    k = turn_halves((h @ W[p + "mix.k"].T).reshape(T, H, D), places, m["rot"], single) * D ** -0.5
    v = (h @ W[p + "mix.v"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        S = np.zeros((D, Dv))
        for t in range(T):
            S = m["decay"][hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps).reshape(T, H * Dv)
    return (o * swish(h @ W[p + "mix.g"].T)) @ W[p + "mix.o"].T


def latent_attention(W, p, m, h, eps, single=False):
    """Queries through a narrow normalised vector; keys and values unfolded per head from one narrow normalised
    vector a token, beside one turned key piece that all heads share; a window; a learned term per head in the
    softmax's denominator."""
    T = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    places = np.arange(T)
    cq = unit_rms(h @ W[p + "mix.dq"].T, eps) * W[p + "mix.dq.norm"]
    q = (cq @ W[p + "mix.uq"].T).reshape(T, H, dn + dr)
    q_flat, q_turn = q[..., :dn], turn_halves(q[..., dn:], places, m["rot"], single)
    down = h @ W[p + "mix.dkv"].T
    c = unit_rms(down[:, :r], eps) * W[p + "mix.dkv.norm"]
    k_turn = turn_halves(down[:, r:], places, m["rot"], single)
    k_flat = (c @ W[p + "mix.uk"].T).reshape(T, H, dn)
    v = (c @ W[p + "mix.uv"].T).reshape(T, H, dv)
    mask = window_mask(T, m["mask"]["size"])
    out = np.zeros((T, H, dv))
    for hd in range(H):
        s = (q_flat[:, hd] @ k_flat[:, hd].T + q_turn[:, hd] @ k_turn.T) * m["scale"]
        w = softmax_with_sink(s, mask, np.full((T, 1), W[p + "mix.sink"][hd]))
        out[:, hd] = w @ v[:, hd]
    return out.reshape(T, H * dv) @ W[p + "mix.o"].T


# --------------------------------------------------------------------------- feed-forwards
def capped_gated(W, p, h, limit):
    g = np.minimum(h @ W[p + "gate"].T, limit)
    u = np.clip(h @ W[p + "up"].T, -limit, limit)
    return (g * logistic(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def router_choice(z, top):
    """The ``top`` largest entries of each row (the lower index wins a tie) and the softmax over just those."""
    order = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zz = np.take_along_axis(z, order, axis=-1)
    e = np.exp(zz - zz.max(axis=-1, keepdims=True))
    return order, e / e.sum(axis=-1, keepdims=True)


def routed_ff(W, p, f, h, routes=None, slack=0.0):
    """sum over a token's chosen experts of weight * expert(h), plus the shared expert.  ``routes`` (position ->
    experts): choices made elsewhere are followed where every one of them lies within ``slack`` of the own last
    choice's logit; the weights are then the softmax over the followed experts' own logits."""
    n, top = f["router"]["experts"], f["router"]["top"]
    z = h @ W[p + "router"].T + W[p + "router.b"]
    order, weight = router_choice(z, top)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        ids, wt = list(order[t]), weight[t]
        if routes is not None and t in routes and sorted(routes[t]) != sorted(ids):
            theirs = list(routes[t])
            floor = z[t, ids[-1]]
            if len(set(theirs)) == top and all(z[t, e] >= floor - slack for e in theirs):
                ids = theirs
                zz = z[t, ids]
                e = np.exp(zz - zz.max())
                wt = e / e.sum()
        for e_, w_ in zip(ids, wt):
            out[t] += w_ * capped_gated(W, f"{p}e{e_}.", h[t:t + 1], f["expert"]["limit"])[0]
    if f.get("shared"):
        out += capped_gated(W, p + "shared.", h, f["shared"]["limit"])
    return out


def feed_forward(W, p, f, h, routes=None, slack=0.0):
    if f["kind"] == "dense":
        return capped_gated(W, p, h, f["limit"])
    return routed_ff(W, p, f, h, routes, slack)


# --------------------------------------------------------------------------- the model
def run_order(cfg):
    """The layers in the order they run: those before ``loop.start`` once, ``start .. stop - 1`` ``times`` times,
    the rest once; each entry is (layer, True where a pass of the loop starts)."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b, times = lp["start"], lp["stop"], lp["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg, W, ids, routes=None, slack=0.0, single=False, layers_out=None):
    """Logits [T, V] of one whole sequence.  ``routes``: run -> position -> experts (see ``routed_ff``).
    ``layers_out``: a list that receives the stream after every run of a layer."""
    eps = cfg["norm"]["eps"]
    x = unit_rms(W["embed"][np.asarray(ids)], eps) * W["embed.norm"]
    x0 = x
    for run, (i, pass_start) in enumerate(run_order(cfg)):
        L, p = cfg["layers"][i], f"l{i}."
        if pass_start:
            x = np.concatenate([x, x0], axis=-1) @ W["loop.in"].T
        h = unit_rms(x, eps) * W[p + "norm1"]
        if L["type"] == "attention":
            x = x + attention(W, p, L["mixer"], h, single)
        elif L["type"] == "retention":
            x = x + retention(W, p, L["mixer"], h, eps, single)
        elif L["type"] == "latent_attention":
            x = x + latent_attention(W, p, L["mixer"], h, eps, single)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            h = unit_rms(x, eps) * W[p + "norm2"]
            x = x + feed_forward(W, p + "mlp.", L["mlp"], h, None if routes is None else routes.get(run), slack)
        if layers_out is not None:
            layers_out.append(x.copy())
    return (unit_rms(x, eps) * W["final.norm"]) @ W["head"].T


def forward_logits(cfg, W, ids):
    return forward(cfg, W, ids)
