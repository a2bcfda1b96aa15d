"""A plain, slow Pubunex forward pass over whole sequences (NumPy, no cache, no state carried
between calls).

Test-only oracle: one function per mechanism, written from the design's equations, sharing
nothing with the engine's product path.  It reads config.json keys itself and looks weights up
by their checkpoint names.  Every function takes ``dt`` (``np.float32`` or ``np.float64``) and
carries out all arithmetic in that type.

Notation: T tokens, W the model width, H query heads, G key/value heads, D the query/key size
of a head, E its value size, C the size of the latent, R the rotated part of a latent head.
"""
from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def unit_rms(x, eps, dt):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = x.astype(dt)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + dt(eps))


def rms_norm_offset(x, w, eps, dt):
    """unit_rms(x) * (1 + w): the gain is stored around zero."""
    return unit_rms(x, eps, dt) * (dt(1.0) + w.astype(dt))


def rms_norm_plain(x, w, eps, dt):
    """unit_rms(x) * w."""
    return unit_rms(x, eps, dt) * w.astype(dt)


# ---------------------------------------------------------------- rotations
def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2, and the factor on sines and cosines.  With ``scaling``
    (factor, original, fast, slow) the frequencies below a ramp are divided by the factor:
    f_i <- f_i / factor * r_i + f_i (1 - r_i), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    lo and hi the (floored, ceiled, clipped) dimensions at which ``fast`` and ``slow`` turns fit
    into ``original`` positions; the factor on sin and cos is 0.1 ln(factor) + 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = np.power(float(base), -2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, freqs, magnitude, interleaved, dt):
    """Rotate the first 2 * len(freqs) channels of the last axis; x: [T, heads, size].
    Pairs are (i, i + n) ('half') or (2i, 2i + 1) (interleaved), n = len(freqs)."""
    x = x.astype(dt).copy()
    n = len(freqs)
    ang = positions.astype(np.float64)[:, None] * freqs[None, :]
    cs = (np.cos(ang) * magnitude).astype(dt)[:, None, :]
    sn = (np.sin(ang) * magnitude).astype(dt)[:, None, :]
    if interleaved:
        a, b = x[..., 0:2 * n:2].copy(), x[..., 1:2 * n:2].copy()
        x[..., 0:2 * n:2] = a * cs - b * sn
        x[..., 1:2 * n:2] = b * cs + a * sn
    else:
        a, b = x[..., :n].copy(), x[..., n:2 * n].copy()
        x[..., :n] = a * cs - b * sn
        x[..., n:2 * n] = b * cs + a * sn
    return x


# ---------------------------------------------------------------- softmax attention
def causal_attention(q, k, v, scale, sinks, dt):
    """q: [T, H, D], k: [T, G, D], v: [T, G, E] -> [T, H, E].  Token i sees j <= i.  ``sinks``
    ([H] or None): exp(sink_h) joins the denominator, with no key and no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]), dt)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h, :] @ k[:, g, :].T) * dt(scale)
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
        m = s.max(axis=1, keepdims=True)
        if sinks is not None:
            m = np.maximum(m, dt(sinks[h]))
        p = np.exp(s - m)
        den = p.sum(axis=1, keepdims=True)
        if sinks is not None:
            den = den + np.exp(dt(sinks[h]) - m)
        out[:, h, :] = (p / den) @ v[:, g, :]
    return out


def attention_mixer(x, positions, w, pre, m, dt):
    """Grouped-query attention with biases on all four projections, partial rotary positions
    (pairs (i, i + dims/2)) with optional frequency scaling, scale from the config."""
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = x.shape[0]
    lin = lambda n: x @ w[pre + n].astype(dt).T + w[pre + n + ".b"].astype(dt)
    q, k, v = lin("q").reshape(T, H, D), lin("k").reshape(T, G, D), lin("v").reshape(T, G, E)
    rot = m.get("rot")
    if rot:
        f, mag = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, positions, f, mag, False, dt), rotate(k, positions, f, mag, False, dt)
    o = causal_attention(q, k, v, m["scale"], None, dt).reshape(T, H * E)
    return o @ w[pre + "o"].astype(dt).T + w[pre + "o.b"].astype(dt)


def latent_attention_mixer(x, positions, w, pre, m, eps, dt):
    """Attention whose keys and values are made from one latent row per token: c =
    rms_norm(first C rows of W_dkv x); one rotated key part (the last R rows, pairs (2i, 2i + 1))
    shared by all heads; head h's key is [W_uk,h c, rotated part], its value W_uv,h c; the
    softmax's denominator holds a sink per head."""
    H, D, R, E, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = x.shape[0]
    q = (x @ w[pre + "q"].astype(dt).T).reshape(T, H, D + R)
    dkv = x @ w[pre + "dkv"].astype(dt).T
    c = rms_norm_plain(dkv[:, :C], w[pre + "dkv.norm"], eps, dt)
    f, mag = rotary_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    k_rot = rotate(dkv[:, None, C:], positions, f, mag, True, dt)                    # [T, 1, R]
    q_rot = rotate(q[:, :, D:], positions, f, mag, True, dt)
    k_plain = (c @ w[pre + "uk"].astype(dt).T).reshape(T, H, D)
    v = (c @ w[pre + "uv"].astype(dt).T).reshape(T, H, E)
    qq = np.concatenate([q[:, :, :D], q_rot], axis=2)
    kk = np.concatenate([k_plain, np.broadcast_to(k_rot, (T, H, R))], axis=2)
    o = causal_attention(qq, kk, v, m["scale"], w[pre + "sink"].astype(dt), dt).reshape(T, H * E)
    return o @ w[pre + "o"].astype(dt).T


# ---------------------------------------------------------------- gated delta rule
def causal_conv_silu(x, taps_w, dt):
    """silu(sum_j taps_w[:, j] x_(t - taps + 1 + j)); zeros before the start.  x: [T, channels]."""
    T, n = x.shape[0], taps_w.shape[1]
    padded = np.concatenate([np.zeros((n - 1, x.shape[1]), dt), x.astype(dt)], axis=0)
    y = np.zeros_like(x, dtype=dt)
    for j in range(n):
        y += padded[j:j + T] * taps_w[:, j].astype(dt)[None, :]
    return silu(y)


def unit_vector(x, dt):
    return x / np.sqrt((x * x).sum(axis=-1, keepdims=True) + dt(1e-6))


def delta_recurrence(q, k, v, beta, decay, dt, S0=None):
    """Per head: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    q, k: [T, H, D]; v: [T, H, E]; beta, decay: [T, H].  Returns o [T, H, E] and the last S."""
    T, H, D = q.shape
    E = v.shape[2]
    S = np.zeros((H, D, E), dt) if S0 is None else S0.astype(dt).copy()
    o = np.zeros((T, H, E), dt)
    for t in range(T):
        for h in range(H):
            S[h] *= decay[t, h]
            u = beta[t, h] * (v[t, h] - S[h].T @ k[t, h])
            S[h] += np.outer(k[t, h], u)
            o[t, h] = S[h].T @ q[t, h]
    return o, S


def delta_mixer(x, w, pre, m, eps, dt):
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = x.shape[0]
    lin = lambda n: x @ w[pre + n].astype(dt).T
    q = causal_conv_silu(lin("q"), w[pre + "q.conv"], dt).reshape(T, G, D)
    k = causal_conv_silu(lin("k"), w[pre + "k.conv"], dt).reshape(T, G, D)
    v = causal_conv_silu(lin("v"), w[pre + "v.conv"], dt).reshape(T, H, E)
    q = unit_vector(q, dt) * dt(D ** -0.5)
    k = unit_vector(k, dt)
    rep = H // G
    q, k = np.repeat(q, rep, axis=1), np.repeat(k, rep, axis=1)       # head h reads q/k head h // rep
    beta = sigmoid(lin("b"))
    decay = np.exp(-np.exp(w[pre + "A_log"].astype(dt))[None, :] * softplus(lin("a") + w[pre + "dt_bias"].astype(dt)[None, :]))
    o, _ = delta_recurrence(q, k, v, beta, decay, dt)
    o = unit_rms(o, eps, dt) * w[pre + "norm"].astype(dt)[None, None, :]
    o = o.reshape(T, H * E) * silu(lin("g"))
    return o @ w[pre + "o"].astype(dt).T


# ---------------------------------------------------------------- feed-forward
def clamped_expert(x, w, pre, limit, dt):
    """g = min(W_gate x, limit), u = clamp(W_up x, +-limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = np.minimum(x @ w[pre + "gate"].astype(dt).T, dt(limit))
    u = np.clip(x @ w[pre + "up"].astype(dt).T, -dt(limit), dt(limit))
    return (g * sigmoid(dt(1.702) * g) * (u + dt(1.0))) @ w[pre + "down"].astype(dt).T


def route(x, router_w, top, dt):
    """Sigmoid scores; the ``top`` largest are chosen (the lower index among equals); the weights
    are the scores themselves.  Returns ids [T, top] and weights [T, top]."""
    s = sigmoid(x.astype(dt) @ router_w.astype(dt).T)
    ids = np.argsort(-s, axis=1, kind="stable")[:, :top]
    return ids, np.take_along_axis(s, ids, axis=1)


def route_margins(x, router_w, top, dt):
    """Per token, the gap between the last chosen router logit and the first one left out
    (infinite when every expert is chosen): how close the choice was."""
    z = np.sort(x.astype(dt) @ router_w.astype(dt).T, axis=1)[:, ::-1]
    return z[:, top - 1] - z[:, top] if z.shape[1] > top else np.full(len(x), np.inf)


def moe(x, w, pre, mlp, dt, margins=None):
    """sum over a token's chosen experts of expert(weight * x), plus the shared expert of x."""
    ids, wts = route(x, w[pre + "router"], mlp["router"]["top"], dt)
    if margins is not None:
        margins.append(route_margins(x, w[pre + "router"], mlp["router"]["top"], dt))
    out = np.zeros_like(x, dtype=dt)
    for t in range(x.shape[0]):
        for e, s in zip(ids[t], wts[t]):
            out[t] += clamped_expert((s * x[t])[None, :], w, f"{pre}e{e}.", mlp["expert"]["limit"], dt)[0]
    if mlp.get("shared"):
        out += clamped_expert(x, w, pre + "shared.", mlp["shared"]["limit"], dt)
    return out


# ---------------------------------------------------------------- the model
def layer_calls(cfg):
    """[(layer, adds the embedding first)]: layers start..stop-1 run ``times`` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["times"] <= 1:
        return [(i, False) for i in range(n)]
    calls = [(i, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        calls += [(i, p > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return calls + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg, w, tokens, dt=np.float64, trace=None, margins=None):
    """Logits [T, vocab] of one sequence from position 0.  ``trace``: a list that receives the
    residual stream after every layer run; ``margins``: one that receives, per routed layer run,
    how close each token's choice of experts was."""
    tokens = np.asarray(tokens)
    pos = np.arange(len(tokens))
    eps = cfg["norm"]["eps"]
    x0 = w["embed"].astype(dt)[tokens]
    x = x0.copy()
    for i, again in layer_calls(cfg):
        L, pre = cfg["layers"][i], f"l{i}."
        if again:
            x = x + x0
        h = rms_norm_offset(x, w[pre + "norm1"], eps, dt)
        if L["type"] == "delta":
            y = delta_mixer(h, w, pre + "mix.", L["mixer"], eps, dt)
        elif L["type"] == "attention":
            y = attention_mixer(h, pos, w, pre + "mix.", L["mixer"], dt)
        elif L["type"] == "latent_attention":
            y = latent_attention_mixer(h, pos, w, pre + "mix.", L["mixer"], eps, dt)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            y = y + moe(h, w, pre + "mlp.", L["mlp"], dt, margins)
        x = x + y
        if trace is not None:
            trace.append(x.copy())
    x = rms_norm_offset(x, w["final.norm"], eps, dt)
    return x @ w["head"].astype(dt).T
