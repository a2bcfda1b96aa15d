"""A plain, slow Dafotar forward pass over whole sequences (NumPy, no cache, no state carried
between calls).

Test-only oracle: one function per mechanism, written from the design's equations, sharing
nothing with the engine's product path.  It reads config.json keys itself and looks weights
up by their checkpoint names.  Every function takes ``dt`` (``np.float32`` or ``np.float64``)
and carries out all arithmetic in that type.

Notation: T tokens, W the model width, S residual streams, H query heads, G key/value heads,
D the query/key size of a head, E its value size.
"""
from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- norms
def layer_norm(x, w, b, eps, dt):
    """(x - mean) / sqrt(var + eps) * w + b over the last axis, var the mean squared deviation."""
    x = x.astype(dt)
    mu = x.mean(axis=-1, keepdims=True)
    d = x - mu
    var = (d * d).mean(axis=-1, keepdims=True)
    return d / np.sqrt(var + dt(eps)) * w.astype(dt) + b.astype(dt)


def unit_rms(x, eps, dt):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = x.astype(dt)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + dt(eps))


# ---------------------------------------------------------------- short causal convolution
def short_conv(h, w, dt):
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j); rows before the sequence are zero.
    h: [T, W]; w: [W, taps]."""
    h = h.astype(dt)
    T, taps = h.shape[0], w.shape[1]
    out = h.copy()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j].astype(dt) * h[s]
    return out


# ---------------------------------------------------------------- residual streams
def streams_read(xs, w_in, dt):
    """u = sum_s w_in[s] x_s.   xs: [T, S, W]."""
    return np.einsum("s,tsw->tw", w_in.astype(dt), xs.astype(dt))


def streams_write(xs, w_mix, w_out, y, dt):
    """x'_t = sum_s w_mix[s, t] x_s + w_out[t] y, every new stream from the old ones."""
    new = np.einsum("sr,tsw->trw", w_mix.astype(dt), xs.astype(dt))
    return new + w_out.astype(dt)[None, :, None] * y.astype(dt)[:, None, :]


# ---------------------------------------------------------------- rotations
def rotate(x, positions, base, dims, dt, interleaved=False, sign=1.0):
    """Turn pairs of the first ``dims`` channels of each head by sign * pos * base^(-2m/dims).
    Pair m is (m, m + dims/2), or (2m, 2m + 1) when ``interleaved``.  x: [T, heads, size]."""
    x = x.astype(dt).copy()
    half = dims // 2
    m = np.arange(half, dtype=dt)
    freq = np.power(dt(base), -(dt(2.0) * m) / dt(dims))
    ang = dt(sign) * positions.astype(dt)[:, None] * freq[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    if interleaved:
        a, b = x[..., 0:dims:2].copy(), x[..., 1:dims:2].copy()
        x[..., 0:dims:2] = a * c - b * s
        x[..., 1:dims:2] = b * c + a * s
    else:
        a, b = x[..., :half].copy(), x[..., half:dims].copy()
        x[..., :half] = a * c - b * s
        x[..., half:dims] = b * c + a * s
    return x


# ---------------------------------------------------------------- attention
def attention_keys_values(h, wts, pre, mx, eps, positions, dt):
    """Keys after head norm and rotation, values after their rotation: what a layer keeps."""
    T = h.shape[0]
    G, D, E = mx["kv_heads"], mx["dim"], mx["vdim"]
    k = (h @ wts[pre + "k"].astype(dt).T).reshape(T, G, D)
    v = (h @ wts[pre + "v"].astype(dt).T).reshape(T, G, E)
    k = unit_rms(k, eps, dt) * wts[pre + "k.norm"].astype(dt)
    rot = mx.get("rot")
    if rot is not None:
        k = rotate(k, positions, rot["base"], rot["dims"], dt)
        v = rotate(v, positions, rot["base"], E, dt)
    return k, v


def attention(h, wts, pre, mx, eps, positions, dt, kv=None):
    """Softmax attention of every token over itself and the keys before it inside the window.
    ``kv``: keys and values of another layer, used instead of this layer's own.
    Returns (output [T, W], (keys, values))."""
    h = h.astype(dt)
    T = h.shape[0]
    H, G, D, E = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (h @ wts[pre + "q"].astype(dt).T).reshape(T, H, D)
    q = unit_rms(q, eps, dt) * wts[pre + "q.norm"].astype(dt)
    rot = mx.get("rot")
    if rot is not None:
        q = rotate(q, positions, rot["base"], rot["dims"], dt)
    if kv is None:
        kv = attention_keys_values(h, wts, pre, mx, eps, positions, dt)
    k, v = kv
    window = (mx.get("mask") or {}).get("size")
    temp = wts[pre + "temp"].astype(dt)
    out = np.zeros((T, H, E), dt)
    for hq in range(H):
        g = hq // (H // G)
        s = (q[:, hq, :] @ k[:, g, :].T) * dt(mx["scale"]) * temp[hq]
        i, j = np.arange(T)[:, None], np.arange(T)[None, :]
        seen = (j <= i) if window is None else ((j <= i) & (i - j < window))
        s = np.where(seen, s, -np.inf)
        p = np.exp(s - s.max(axis=-1, keepdims=True))
        p = p / p.sum(axis=-1, keepdims=True)
        out[:, hq, :] = p @ v[:, g, :]
    if rot is not None:
        out = rotate(out, positions, rot["base"], E, dt, sign=-1.0)
    return out.reshape(T, H * E) @ wts[pre + "o"].astype(dt).T, kv


# ---------------------------------------------------------------- matrix-memory recurrence
def log_sigmoid(x):
    return np.where(x >= 0, -np.log1p(np.exp(-np.abs(x))), x - np.log1p(np.exp(-np.abs(x))))


def mlstm(h, wts, pre, mx, eps, dt):
    """Token by token from a zero state, the running maximum starting at 0."""
    h = h.astype(dt)
    T = h.shape[0]
    H, D, E, cap = mx["heads"], mx["dim"], mx["vdim"], dt(mx["gate_cap"])
    q = (h @ wts[pre + "q"].astype(dt).T).reshape(T, H, D) * dt(D) ** dt(-0.5)
    k = (h @ wts[pre + "k"].astype(dt).T).reshape(T, H, D)
    v = (h @ wts[pre + "v"].astype(dt).T).reshape(T, H, E)
    gi = cap * np.tanh((h @ wts[pre + "i"].astype(dt).T + wts[pre + "i.b"].astype(dt)) / cap)
    gf = log_sigmoid(cap * np.tanh((h @ wts[pre + "f"].astype(dt).T + wts[pre + "f.b"].astype(dt)) / cap))
    S = np.zeros((H, D, E), dt)
    n = np.zeros((H, D), dt)
    m = np.zeros((H,), dt)
    o = np.zeros((T, H, E), dt)
    for t in range(T):
        m_new = np.maximum(gf[t] + m, gi[t])
        a = np.exp(gf[t] + m - m_new)
        b = np.exp(gi[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        m = m_new
        num = np.einsum("hde,hd->he", S, q[t])
        den = np.maximum(np.abs((n * q[t]).sum(axis=-1)), np.exp(-m)) + dt(1e-6)
        o[t] = num / den[:, None]
    o = unit_rms(o, eps, dt).reshape(T, H * E) * wts[pre + "norm"].astype(dt)
    gate = h @ wts[pre + "g"].astype(dt).T
    o = o * (dt(1.0) / (dt(1.0) + np.exp(-gate)))
    return o @ wts[pre + "o"].astype(dt).T


# ---------------------------------------------------------------- feed-forward
def feed_forward(h, wts, pre, dt):
    h = h.astype(dt)
    g = np.maximum(h @ wts[pre + "gate"].astype(dt).T, 0)
    return (g * (h @ wts[pre + "up"].astype(dt).T)) @ wts[pre + "down"].astype(dt).T


# ---------------------------------------------------------------- the model
def forward(cfg: dict, wts: dict, tokens, dt=np.float64, per_layer=None):
    """Logits [T, vocab] of one sequence from position 0.  ``per_layer``: a list that receives
    the residual stream (the sum of the streams) after every layer."""
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams")
    taps = (cfg.get("canon") or {}).get("taps")
    tokens = np.asarray(tokens)
    T = len(tokens)
    positions = np.arange(T)
    x = wts["embed"].astype(dt)[tokens]
    xs = np.repeat(x[:, None, :], S, axis=1) if S else None
    kept = {}
    for l, layer in enumerate(cfg["layers"]):
        pre, mx = f"l{l}.", layer["mixer"]
        for q, has in ((1, True), (2, layer.get("mlp") is not None)):
            if not has:
                continue
            u = streams_read(xs, wts[f"{pre}hc{q}.in"], dt) if S else x
            h = layer_norm(u, wts[f"{pre}norm{q}"], wts[f"{pre}norm{q}.b"], eps, dt)
            if q == 1:
                if taps:
                    h = short_conv(h, wts[pre + "canon1"], dt)
                if layer["type"] == "attention":
                    src = mx.get("kv_from")
                    y, kept[l] = attention(h, wts, pre + "mix.", mx, eps, positions, dt,
                                           kv=kept[src] if src is not None else None)
                elif layer["type"] == "mlstm":
                    y = mlstm(h, wts, pre + "mix.", mx, eps, dt)
                else:
                    raise ValueError(f"unknown layer type {layer['type']!r}")
            else:
                y = feed_forward(h, wts, pre + "mlp.", dt)
            if S:
                xs = streams_write(xs, wts[f"{pre}hc{q}.mix"], wts[f"{pre}hc{q}.out"], y, dt)
            else:
                x = x + y
        if per_layer is not None:
            per_layer.append(xs.sum(axis=1) if S else x.copy())
    if S:
        x = xs.sum(axis=1)
    x = layer_norm(x, wts["final.norm"], wts["final.norm.b"], eps, dt)
    return x @ wts["embed"].astype(dt).T
