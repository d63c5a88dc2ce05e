"""A plain, slow implementation of the Divasun decoder, written from its equations: one function per
mechanism, whole sequences at a time, on the CPU in 64-bit floats.  It shares no code with the engine;
the tests compare the engine's parts and whole models with it.

Notation: ``T`` tokens of one sequence, ``d`` the width; a linear weight ``W`` is stored ``[out, in]``
and applied as ``x @ W.T``.  ``P`` is a dictionary of one sublayer's tensors by their last name
(``P["q"]``, ``P["q.norm"]``, ...).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def short_conv(h, w):
    """``h + conv(h)``: ``conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j]``, rows before the first count as zeros."""
    T, d = h.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, d, dtype=h.dtype), h], 0)
    out = h.clone()
    for j in range(taps):
        out = out + w[:, j] * padded[j:j + T]
    return out


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def general_delta(h, P, heads: int, dim: int, eps: float, state: Optional[torch.Tensor] = None):
    """The generalised delta rule, token by token.  ``state``: ``[heads, dim, dim]`` (key channel, value
    channel) or None for zeros; returns (output ``[T, d]``, last state)."""
    T = h.shape[0]
    r = (h @ P["r"].T).view(T, heads, dim)
    k = (h @ P["k"].T).view(T, heads, dim)
    v = (h @ P["v"].T).view(T, heads, dim)
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ P["w1"].T) @ P["w2"].T + P["w0"])).view(T, heads, dim)
    rate = torch.sigmoid(h @ P["a"].T + P["a.b"]).view(T, heads, dim)
    gate = torch.sigmoid(h @ P["g"].T)
    unit = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(heads, dim, dim, dtype=h.dtype) if state is None else state.clone()
    outs = []
    for t in range(T):
        seen = torch.einsum("hi,hij->hj", unit[t], S)                      # u^T S, per head
        S = decay[t][:, :, None] * S - (rate[t] * unit[t])[:, :, None] * seen[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        outs.append(torch.einsum("hij,hi->hj", S, r[t]))
    o = torch.stack(outs, 0)                                               # [T, heads, dim]
    o = rms_unit(o, eps).reshape(T, heads * dim) * P["norm"] * gate
    return o @ P["o"].T, S


def bias_slopes(heads: int):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=F)


def attention_keys_values(h, P, kv_heads: int, dim: int, vdim: int, eps: float):
    T = h.shape[0]
    k = rms_unit(h @ P["k"].T, eps) * P["k.norm"]
    v = h @ P["v"].T
    return k.view(T, kv_heads, dim), v.view(T, kv_heads, vdim)


def attention(h, P, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float,
              q_temp=None, kv=None, first_position: int = 0):
    """Causal attention with a bias on the distance.  ``kv``: (keys, values) of ALL positions from 0 (another
    layer's, or this layer's earlier ones joined with the new); None: made from ``h``, which then starts at 0."""
    T = h.shape[0]
    q = rms_unit(h @ P["q"].T, eps) * P["q.norm"]
    pos = torch.arange(first_position, first_position + T)
    if q_temp is not None:
        coef, every = q_temp
        q = q * (1.0 + coef * torch.log(torch.floor((pos + 1).to(F) / every) + 1.0))[:, None]
    q = q.view(T, heads, dim)
    keys, values = kv if kv is not None else attention_keys_values(h, P, kv_heads, dim, vdim, eps)
    n = keys.shape[0]
    slopes = bias_slopes(heads)
    out = torch.zeros(T, heads, vdim, dtype=h.dtype)
    j = torch.arange(n)
    for hd in range(heads):
        g = hd // (heads // kv_heads)
        s = (q[:, hd] @ keys[:, g].T) * scale - slopes[hd] * (pos[:, None] - j[None, :]).to(F)
        s = s.masked_fill(j[None, :] > pos[:, None], float("-inf"))
        out[:, hd] = torch.softmax(s, -1) @ values[:, g]
    return out.reshape(T, heads * vdim) @ P["o"].T


def moe(h, P, experts: int, top: int, margins: Optional[list] = None):
    """Every token's ``top`` experts by sigmoid score; the score scales what goes into the expert.  ``margins`` takes
    every token's distance between the last chosen logit and the first that was not (how close the call was)."""
    z = h @ P["router"].T
    s = torch.sigmoid(z)
    if margins is not None and top < experts:
        ranked = torch.sort(z, dim=-1, descending=True).values
        margins.extend((ranked[:, top - 1] - ranked[:, top]).tolist())
    out = torch.zeros(h.shape[0], P["e0.down"].shape[0], dtype=h.dtype)
    order = torch.argsort(-s, dim=-1, stable=True)[:, :top]
    for t in range(h.shape[0]):
        for e in order[t].tolist():
            x = s[t, e] * h[t]
            out[t] += gelu_erf(x @ P[f"e{e}.up"].T) @ P[f"e{e}.down"].T
    return out


def sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None,
            margins: Optional[list] = None):
    """Logits ``[T, vocab]`` of one whole sequence from position 0."""
    W = {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        h1 = short_conv(layer_norm(x, W[pre + "norm1"], W[pre + "norm1.b"], eps), W[pre + "canon1"])
        P = sub(W, pre + "mix.")
        if layer["type"] == "general_delta":
            a, _ = general_delta(h1, P, m["heads"], m["dim"], eps)
        elif layer["type"] == "attention":
            G = m.get("kv_heads", m["heads"])
            vdim = m.get("vdim", m["dim"])
            if m.get("kv_from") is not None:
                kv = kept[m["kv_from"]]
            else:
                kv = kept[i] = attention_keys_values(h1, P, G, m["dim"], vdim, eps)
            qt = (m["q_temp"]["coef"], m["q_temp"]["every"]) if m.get("q_temp") else None
            a = attention(h1, P, m["heads"], G, m["dim"], vdim, m["scale"], eps, q_temp=qt, kv=kv)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            h2 = short_conv(layer_norm(x, W[pre + "norm2"], W[pre + "norm2.b"], eps), W[pre + "canon2"])
            f = layer["mlp"]
            a = a + moe(h2, sub(W, pre + "mlp."), f["router"]["experts"], f["router"]["top"], margins)
        x = x + a
        if layers_out is not None:
            layers_out.append(x.clone())
    y = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return y @ W["head"].T
