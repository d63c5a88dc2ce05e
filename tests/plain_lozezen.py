"""A plain, slow implementation of the Lozezen decoder: float64, whole sequences, no cache, one function per
mechanism.  It imports nothing from the package; the tests compare the engine with it.

``cfg`` is the dict of a config.json, ``w`` maps tensor names to float64 arrays, ``tokens`` is one sequence.
"""
from __future__ import annotations

import math

import numpy as np

RGLRU_C = 8.0          # the exponent's factor in the recurrent unit's decay


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """Every row of the last axis divided by sqrt(mean of squares + eps)."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def norm_one_plus(x, weight, eps):
    return unit_rms(x, eps) * (1.0 + weight)


def linear(x, w, name, bias=False):
    y = x @ w[name].T
    return y + w[name + ".b"] if bias else y


def rotate(x, positions, dims, base, factor=1.0, interleaved=False):
    """x [T, heads, dim]: the first ``dims`` dims of every head turned by angle p * base^(-2i/dims) / factor;
    pair i is (2i, 2i+1) if ``interleaved`` else (i, i + dims/2)."""
    half = dims // 2
    freq = base ** (-2.0 * np.arange(half) / dims) / factor
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = x.copy()
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    else:
        a, b = x[..., :half], x[..., half:dims]
        out[..., :half] = a * c - b * s
        out[..., half:dims] = b * c + a * s
    return out


def masked_softmax_attention(q, k, v, scale, visible):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; ``visible [T, T]`` (bool) says whether query i sees key j (the caller
    masks the future too).  Query head h uses key/value head h // (H / G).  -> [T, H, dv]"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = np.where(visible, s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


def window_attention(h, w, pre, m):
    """The mixer ``attention``: grouped queries, biases, a rotation of the first dims of neighbouring pairs with
    scaled-down frequencies, a sliding window."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w, pre + "q", True).reshape(T, H, d)
    k = linear(h, w, pre + "k", True).reshape(T, G, d)
    v = linear(h, w, pre + "v", True).reshape(T, G, dv)
    rot = m["rot"]
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    pos = np.arange(T)
    q = rotate(q, pos, rot["dims"], rot["base"], factor, interleaved=True)
    k = rotate(k, pos, rot["dims"], rot["base"], factor, interleaved=True)
    size = m["mask"]["size"]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    o = masked_softmax_attention(q, k, v, m["scale"], (j <= i) & (i - j < size))
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def chunk_attention(h, w, pre, m, eps):
    """The left half of ``parallel``: biases, a norm per head on queries and keys, no positions in the scores,
    keys of the query's own chunk only, a gate per head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w, pre + "q", True).reshape(T, H, d)
    k = linear(h, w, pre + "k", True).reshape(T, G, d)
    v = linear(h, w, pre + "v", True).reshape(T, G, dv)
    q = unit_rms(q, eps) * w[pre + "q.norm"]
    k = unit_rms(k, eps) * w[pre + "k.norm"]
    size = m["mask"]["size"]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    o = masked_softmax_attention(q, k, v, m["scale"], (j <= i) & (i // size == j // size))
    gate = sigmoid(h @ w[pre + "g"].T)                       # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def retention(h, w, pre, m, eps):
    """The right half of ``parallel``: per head S <- decay S + k v^T, o = S^T q; no softmax, no denominator."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = linear(h, w, pre + "q").reshape(T, H, d)
    k = linear(h, w, pre + "k").reshape(T, H, d)
    v = linear(h, w, pre + "v").reshape(T, H, dv)
    rot = m.get("rot")
    if rot is not None:
        pos = np.arange(T)
        q, k = rotate(q, pos, rot["dims"], rot["base"]), rotate(k, pos, rot["dims"], rot["base"])
    k = k * d ** -0.5
    o = np.zeros((T, H, dv))
    for hd in range(H):
        S = np.zeros((d, dv))
        for t in range(T):
            S = m["decay"][hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps).reshape(T, H * dv)
    return (o * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def parallel_mixer(h, w, pre, m, eps):
    return m["left_scale"] * chunk_attention(h, w, pre + "left.", m["left"], eps) \
        + m["right_scale"] * retention(h, w, pre + "right.", m["right"], eps)


def causal_conv(x, weight, bias):
    """x [T, C]; weight [C, taps], the last column the current token's; zeros before the start."""
    T, C = x.shape
    taps = weight.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x])
    out = np.zeros((T, C)) + bias
    for j in range(taps):
        out += padded[j:j + T] * weight[:, j]
    return out


def rglru(h, w, pre, m):
    """The mixer ``rglru``: a gated branch times a linear recurrence over a short convolution's output."""
    T = h.shape[0]
    width, blocks = m["width"], m["blocks"]
    y = gelu_tanh(linear(h, w, pre + "y", True))
    u = causal_conv(linear(h, w, pre + "x", True), w[pre + "conv"], w[pre + "conv.b"])
    bs = width // blocks
    ub = u.reshape(T, blocks, bs)
    r = sigmoid(np.einsum("tbi,boi->tbo", ub, w[pre + "ra"]) + w[pre + "ra.b"]).reshape(T, width)
    i = sigmoid(np.einsum("tbi,boi->tbo", ub, w[pre + "ri"]) + w[pre + "ri.b"]).reshape(T, width)
    log_a = -RGLRU_C * r * softplus(w[pre + "lam"])
    a = np.exp(log_a)
    mult = np.sqrt(1.0 - a * a)
    S = np.zeros(width)
    out = np.zeros((T, width))
    for t in range(T):
        S = a[t] * S + mult[t] * i[t] * u[t]
        out[t] = S
    return (out * y) @ w[pre + "o"].T


def dense_ffn(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def mixer(kind, h, w, pre, m, eps):
    if kind == "attention":
        return window_attention(h, w, pre, m)
    if kind == "parallel":
        return parallel_mixer(h, w, pre, m, eps)
    if kind == "rglru":
        return rglru(h, w, pre, m)
    raise ValueError(kind)


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out``: a list that receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        a = mixer(layer["type"], norm_one_plus(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
        x = x + norm_one_plus(a, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            f = dense_ffn(norm_one_plus(x, w[p + "norm2"], eps), w, p + "mlp.")
            x = x + norm_one_plus(f, w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm_one_plus(x, w["final.norm"], eps) @ w["head"].T
