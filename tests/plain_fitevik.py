"""A plain, slow implementation of the Fitevik design in float64 numpy, one function per mechanism.

Everything is written from the design's equations and shares no code with the package: whole
sequences at once, no cache, no batching.  ``forward`` takes a config.json dictionary and the
tensors by their file names.

Notation: ``x`` [T, W] residual stream of one sequence (sublayers read it as it is; the norm stands
behind the sublayer), ``eps`` the norms' constant, ``t`` the tensors by file name, ``p`` the prefix of
a mixer's or feed-forward's tensors.  Linear weights are ``[out, in]`` and applied as ``h @ W.T``.
"""
from __future__ import annotations

import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def relu_squared(z):
    return np.square(np.maximum(z, 0.0))


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, times ``w``."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def layer_norm(x, t, name, eps):
    """(x - mean) / sqrt(var + eps) * w + b; the variance is the mean of the squared deviations."""
    mu = np.mean(x, axis=-1, keepdims=True)
    dev = x - mu
    var = np.mean(dev * dev, axis=-1, keepdims=True)
    return dev / np.sqrt(var + eps) * t[name] + t[name + ".b"]


# ---------------------------------------------------------------- embedding and output
def embed(tokens, positions, t, eps):
    """Token row plus the learned row of the position, then the model's norm."""
    x = t["embed"][np.asarray(tokens)] + t["pos"][np.asarray(positions)]
    return layer_norm(x, t, "embed.norm", eps)


def output(x, t, eps, logit_scale):
    return layer_norm(x, t, "final.norm", eps) @ t["head"].T * logit_scale


# ---------------------------------------------------------------- mixers
def hgrn2(h, m, t, p, eps, state=None):
    """Linear attention whose forget gate is also (one minus) the key.  Per head S [dim, vdim]:
    S <- diag(f) S + (1 - f) v^T, o = S^T q, f = l + (1 - l) sigmoid(W_f h + b_f), q = silu(W_q h).
    Returns (mixer output [T, W], the states after the last token [heads, dim, vdim])."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ t[p + "q"].T).reshape(T, H, D)
    v = (h @ t[p + "v"].T).reshape(T, H, Dv)
    low = t[p + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ t[p + "f"].T + t[p + "f.b"])).reshape(T, H, D)
    S = np.zeros((H, D, Dv)) if state is None else state.copy()
    o = np.zeros((T, H, Dv))
    for i in range(T):
        S = f[i][:, :, None] * S + (1.0 - f[i])[:, :, None] * v[i][:, None, :]
        o[i] = np.einsum("hdv,hd->hv", S, q[i])
    o = rms_norm(o, t[p + "norm"], eps)                       # per head over vdim, one gain for all heads
    return o.reshape(T, H * Dv) @ t[p + "o"].T, S


def head_slopes(H):
    return np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])


def keys_and_values(h, m, t, p, eps):
    """What an attention layer with projections of its own keeps per token: the normed keys and the values."""
    T = h.shape[0]
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    k = rms_norm(h @ t[p + "k"].T, t[p + "k.norm"], eps).reshape(T, G, D)      # one norm over all heads at once
    v = (h @ t[p + "v"].T).reshape(T, G, Dv)
    return k, v


def mixed_softmax_attention(q, k, v, window, scale, slopes, talk, sink, first=0):
    """``q`` [T, H, dim] at positions first .. first + T - 1; ``k`` [first + T, G, dim] and ``v`` [first + T, G, vdim]
    from position 0.  raw_g = scale q_g . k_j - slope_g (i - j); score_h = sum_g talk[h, g] raw_g; inside the
    window softmax with exp(sink_h) added to the denominator.  ``slopes``, ``talk``, ``sink`` may be None."""
    T, H, _ = q.shape
    G = k.shape[1]
    kv_of = [g // (H // G) for g in range(H)]
    out = np.zeros((T, H, v.shape[2]))
    for r in range(T):
        i = first + r
        lo = max(0, i - window + 1) if window else 0
        raw = np.zeros((H, i + 1 - lo))
        for g in range(H):
            raw[g] = k[lo:i + 1, kv_of[g]] @ q[r, g] * scale
            if slopes is not None:
                raw[g] -= slopes[g] * (i - np.arange(lo, i + 1))
        mixed = talk @ raw if talk is not None else raw                      # [H, keys]
        for g in range(H):
            top = mixed[g].max() if sink is None else max(mixed[g].max(), sink[g])
            e = np.exp(mixed[g] - top)
            w = e / (e.sum() + (math.exp(sink[g] - top) if sink is not None else 0.0))   # the sink counts once and has no value
            out[r, g] = w @ v[lo:i + 1, kv_of[g]]
    return out


def window_of(m):
    """Keys a query sees, its own included; 0 (every earlier key) where the mixer has no mask."""
    return m["mask"]["size"] if m.get("mask") else 0


def attention(h, m, t, p, eps, k, v):
    """Softmax attention inside a sliding window with a distance bias, scores mixed over the heads, and a
    sink in the denominator.  ``k`` [T, G, dim], ``v`` [T, G, vdim]: this layer's or another's."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    q = rms_norm(h @ t[p + "q"].T, t[p + "q.norm"], eps).reshape(T, H, D)
    out = mixed_softmax_attention(q, k, v, window_of(m), m["scale"], head_slopes(H), t[p + "talk"], t[p + "sink"])
    return out.reshape(T, -1) @ t[p + "o"].T


# ---------------------------------------------------------------- feed-forwards
def dense_mlp(h, t, p):
    return relu_squared(h @ t[p + "up"].T + t[p + "up.b"]) @ t[p + "down"].T + t[p + "down.b"]


def routed_experts(h, f, t, p):
    """Every token's ``top`` experts by router logit, weighted by the softmax over the chosen logits."""
    E, top = f["router"]["experts"], f["router"]["top"]
    z = h @ t[p + "router"].T + t[p + "router.b"]
    out = np.zeros((h.shape[0], t[p + "e0.down"].shape[0]))
    for i in range(h.shape[0]):
        chosen = np.argsort(-z[i], kind="stable")[:top]
        w = np.exp(z[i, chosen] - z[i, chosen].max())
        w /= w.sum()
        for e, we in zip(chosen, w):
            out[i] += we * (relu_squared(h[i] @ t[p + f"e{e}.up"].T) @ t[p + f"e{e}.down"].T)
    return out


def feed_forward(h, f, t, p):
    return dense_mlp(h, t, p) if f["kind"] == "dense" else routed_experts(h, f, t, p)


# ---------------------------------------------------------------- the model
def forward(cfg, t, tokens, keep_layers=False):
    """Logits [T, vocab] of one sequence from position 0; with ``keep_layers`` also the stream after every layer."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    x = embed(tokens, np.arange(T), t, eps)
    kept, streams = {}, []
    for l, layer in enumerate(cfg["layers"]):
        p, m = f"l{l}.", layer["mixer"]
        if layer["type"] == "hgrn2":
            y, _ = hgrn2(x, m, t, p + "mix.", eps)
        elif layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[l] = keys_and_values(x, m, t, p + "mix.", eps)
                src = l
            y = attention(x, m, t, p + "mix.", eps, *kept[src])
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + layer_norm(y, t, p + "norm1", eps)
        if layer.get("mlp") is not None:
            x = x + layer_norm(feed_forward(x, layer["mlp"], t, p + "mlp."), t, p + "norm2", eps)
        streams.append(x.copy())
    logits = output(x, t, eps, cfg.get("logit_scale", 1.0))
    return (logits, np.stack(streams)) if keep_layers else logits
