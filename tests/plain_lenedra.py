"""A plain, slow implementation of the Lenedra design in float64 numpy, one function per mechanism.

Everything is written from the design's equations and shares no code with the package: whole
sequences at once, no cache, no batching.  ``forward`` takes a config.json dictionary and the
tensors by their file names.

Notation: ``h`` [T, W] a sublayer's (normed) input for one sequence, ``eps`` the norms' constant, ``t``
the tensors by file name, ``p`` the prefix of a mixer's or feed-forward's tensors, ``m`` the mixer's
(or feed-forward's) object of config.json.  Linear weights are ``[out, in]`` and applied as ``h @ W.T``.
"""
from __future__ import annotations

import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, times ``w``."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


# ---------------------------------------------------------------- embedding and output
def embed(tokens, t, scale):
    return t["embed"][np.asarray(tokens)] * scale


def output(x, t, eps, softcap):
    """The model's norm (gain stored around zero), the head, and the soft cap on the logits."""
    z = rms_norm(x, 1.0 + t["final.norm"], eps) @ t["head"].T
    return softcap * np.tanh(z / softcap) if softcap else z


# ---------------------------------------------------------------- masks
def window_mask(T, size, keep_first=0):
    """[i, j] true where query i sees key j: j <= i and (i - j < size or j < keep_first)."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def chunk_mask(T, size):
    """[i, j] true where j <= i and both lie in the same chunk of ``size`` positions counted from 0."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def mask_of(m, T):
    mask = m.get("mask")
    if mask is None:
        return window_mask(T, T + 1)
    if m.get("_chunked"):
        return chunk_mask(T, mask["size"])
    return window_mask(T, mask["size"], mask.get("keep_first", 0))


def distance_slopes(H):
    return np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])


def softmax_attention(q, k, v, mask, scale, slopes=None, sink=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; query head h reads key/value head h // (H / G).
    score = scale q.k - slope_h (i - j); softmax over the visible keys, whose denominator also holds
    exp(sink_h) where a sink is given.  Returns [T, H, Dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    dist = (np.arange(T)[:, None] - np.arange(T)[None, :]).astype(np.float64)
    for h in range(H):
        g = h // (H // G)
        s = q[:, h] @ k[:, g].T * scale
        if slopes is not None:
            s = s - slopes[h] * dist
        s = np.where(mask, s, -np.inf)
        top = s.max(axis=1, keepdims=True)
        if sink is not None:
            top = np.maximum(top, sink[h])
        e = np.exp(s - top)
        den = e.sum(axis=1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[h] - top)
        out[:, h] = (e / den) @ v[:, g]
    return out


# ---------------------------------------------------------------- mixers
def attention(h, m, t, p, eps):
    """What the key projection returns is used twice: raw as the value, normed as the key; q and k normed per head with a gain shared by
    the heads; a distance bias; a sliding window that also keeps the first tokens."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ t[p + "q"].T + t[p + "q.b"]).reshape(T, H, D)
    k = (h @ t[p + "k"].T + t[p + "k.b"]).reshape(T, G, D)
    v = k
    q = rms_norm(q, t[p + "q.norm"], eps)
    k = rms_norm(k, t[p + "k.norm"], eps)
    o = softmax_attention(q, k, v, mask_of(m, T), m["scale"], slopes=distance_slopes(H))
    return o.reshape(T, -1) @ t[p + "o"].T + t[p + "o.b"]


def chunked_sink_attention(h, m, t, p):
    """The left member of a pair: biased projections, no norm, no position, a chunked mask, a sink."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T + t[p + "q.b"]).reshape(T, H, D)
    k = (h @ t[p + "k"].T + t[p + "k.b"]).reshape(T, G, D)
    v = (h @ t[p + "v"].T + t[p + "v.b"]).reshape(T, G, Dv)
    o = softmax_attention(q, k, v, mask_of(dict(m, _chunked=True), T), m["scale"], sink=t[p + "sink"])
    return o.reshape(T, -1) @ t[p + "o"].T


def short_convolution(x, w):
    """Causal convolution over time per channel: x [T, C], w [C, taps], the last column is the current token's."""
    T, C = x.shape
    taps = w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x], axis=0)
    y = np.zeros((T, C))
    for j in range(taps):
        y += padded[j:j + T] * w[:, j]
    return y


def gated_delta_rule(h, m, t, p, eps):
    """The right member of a pair.  Per head S [dim, vdim]: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q, with a decay per head and key channel."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ t[p + "q"].T, t[p + "q.conv"])).reshape(T, G, D)
    k = silu(short_convolution(h @ t[p + "k"].T, t[p + "k.conv"])).reshape(T, G, D)
    v = silu(short_convolution(h @ t[p + "v"].T, t[p + "v.conv"])).reshape(T, H, Dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ t[p + "b"].T)                                                   # [T, H]
    a = (h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "dt_bias"]
    g = np.exp(-np.exp(t[p + "A_log"])[None, :, None] * softplus(a).reshape(T, H, D))  # [T, H, D]
    gate = sigmoid((h @ t[p + "g1"].T) @ t[p + "g2"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        c = hd // (H // G)
        S = np.zeros((D, Dv))
        for i in range(T):
            S = g[i, hd][:, None] * S
            u = beta[i, hd] * (v[i, hd] - S.T @ k[i, c])
            S = S + np.outer(k[i, c], u)
            o[i, hd] = S.T @ q[i, c]
    o = rms_norm(o, t[p + "norm"], eps) * gate
    return o.reshape(T, -1) @ t[p + "o"].T


def parallel(h, m, t, p, eps):
    left = chunked_sink_attention(h, m["left"], t, p + "left.")
    right = gated_delta_rule(h, m["right"], t, p + "right.", eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ---------------------------------------------------------------- feed-forwards
def gated_ff(h, t, p):
    return (silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def route(z, correction, top, groups, keep, scale):
    """z [T, E] router logits over experts and identity experts.  Returns (chosen [T, top], weights [T, top])."""
    T, E = z.shape
    e = np.exp(z - z.max(axis=1, keepdims=True))
    s = e / e.sum(axis=1, keepdims=True)
    choice = s + correction
    if groups > 1:
        per = E // groups
        best = choice.reshape(T, groups, per).max(axis=2)
        order = np.argsort(-best, axis=1, kind="stable")[:, :keep]
        allowed = np.zeros((T, groups), dtype=bool)
        np.put_along_axis(allowed, order, True, axis=1)
        choice = np.where(np.repeat(allowed, per, axis=1), choice, -np.inf)
    chosen = np.argsort(-choice, axis=1, kind="stable")[:, :top]
    w = np.take_along_axis(s, chosen, axis=1)
    w = w / (w.sum(axis=1, keepdims=True) + 1e-20) * scale
    return chosen, w


def experts_ff(h, f, t, p):
    r = f["router"]
    E, ident = r["experts"], r.get("identity", 0)
    g = r.get("groups") or {"count": 1, "keep": 1}
    z = h @ t[p + "router"].T
    chosen, w = route(z, t[p + "correction"], r["top"], g["count"], g["keep"], r.get("scale", 1.0))
    y = np.zeros_like(h)
    for i in range(h.shape[0]):
        for e, wt in zip(chosen[i], w[i]):
            y[i] += wt * (h[i] if e >= E else gated_ff(h[i:i + 1], t, f"{p}e{e}.")[0])
    if f.get("shared") is not None:
        y = y + gated_ff(h, t, p + "shared.")
    assert ident == z.shape[1] - E
    return y


def feed_forward(h, f, t, p):
    if f["kind"] == "dense":
        return gated_ff(h, t, p)
    if f["kind"] == "moe":
        return experts_ff(h, f, t, p)
    raise ValueError(f["kind"])


# ---------------------------------------------------------------- the model
def hyper_sublayer(xs, t, p, norm_w, eps, fn):
    """xs [S, T, W].  u = sum_s in[s] x_s; y = fn(norm(u)); x_t <- sum_s mix[s, t] x_s + out[t] y."""
    u = np.tensordot(t[p + "in"], xs, axes=(0, 0))
    y = fn(rms_norm(u, 1.0 + norm_w, eps))
    return np.tensordot(t[p + "mix"].T, xs, axes=(1, 0)) + t[p + "out"][:, None, None] * y[None]


def forward(config, t, tokens, layer_outputs=None):
    """Logits [T, vocab] of one sequence.  ``layer_outputs``: a list that receives the residual stream (the sum
    of the streams) after every layer."""
    t = {k: np.asarray(v, dtype=np.float64) for k, v in t.items()}
    eps = config["norm"]["eps"]
    S = config.get("streams")                       # absent: one stream and the plain residual sum
    x = embed(tokens, t, (config.get("embedding") or {}).get("scale", 1.0))
    xs = np.repeat(x[None], S, axis=0) if S is not None else None
    for l, layer in enumerate(config["layers"]):
        p, m = f"l{l}.", layer["mixer"]
        if layer["type"] == "attention":
            mixer = lambda h: attention(h, m, t, p + "mix.", eps)
        elif layer["type"] == "parallel":
            mixer = lambda h: parallel(h, m, t, p + "mix.", eps)
        else:
            raise ValueError(layer["type"])
        ff = (lambda h: feed_forward(h, layer["mlp"], t, p + "mlp.")) if layer.get("mlp") is not None else None
        if S is not None:
            xs = hyper_sublayer(xs, t, p + "hc1.", t[p + "norm1"], eps, mixer)
            if ff is not None:
                xs = hyper_sublayer(xs, t, p + "hc2.", t[p + "norm2"], eps, ff)
            x = xs.sum(axis=0)
        else:
            x = x + mixer(rms_norm(x, 1.0 + t[p + "norm1"], eps))
            if ff is not None:
                x = x + ff(rms_norm(x, 1.0 + t[p + "norm2"], eps))
        if layer_outputs is not None:
            layer_outputs.append(x.copy())
    return output(x, t, eps, config.get("logit_softcap"))
