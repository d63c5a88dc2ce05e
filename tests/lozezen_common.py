"""Shared by the Lozezen tests: small configurations that differ in every size and option, random weights from the
tests' own generator, model folders in temporary places, and the plain implementation's logits."""
from __future__ import annotations

import json
import math
import os
import tempfile
from typing import Dict, List, Optional

import numpy as np
import torch

import plain_lozezen as P


def window_attention(heads, kv_heads, dim, vdim, scale, window, rot_dims, base=10000.0, factor=None):
    rot = {"dims": rot_dims, "base": base}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window}, "rot": rot}


def parallel(left, right, left_scale, right_scale):
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def chunk_attention(heads, kv_heads, dim, vdim, scale, chunk):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": chunk}}


def retention(heads, dim, vdim, decay, rot_dims, base=10000.0):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": {"dims": rot_dims, "base": base}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(vocab, width, layers, eps, scale):
    return {"architecture": "Lozezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": layers}


# no size a power of two where it need not be: groups of three heads on two key/value heads, values wider than keys, a
# window of 19 and a chunk of 11 (neither a multiple of a page), a rotation of 10 of 24 dims, retention with values
# narrower than keys and a rotation of a part of the head, 3 blocks of 24 channels, a convolution of 3 taps, a recurrent
# unit wider than the model, an attention layer without feed-forward
CFG_A = config(131, 72, [
    {"type": "rglru", "mixer": {"width": 72, "blocks": 3, "conv": 3}, "mlp": dense(40)},
    {"type": "attention", "mixer": window_attention(6, 2, 24, 40, 0.31, 19, 10, base=500.0, factor=2.5), "mlp": None},
    {"type": "parallel", "mixer": parallel(chunk_attention(4, 2, 16, 24, 0.4, 11), retention(3, 24, 16, [0.9, 0.97, 0.995], 12, base=300.0), 0.7, 1.3),
     "mlp": dense(56)},
    {"type": "rglru", "mixer": {"width": 96, "blocks": 2, "conv": 2}, "mlp": None},
], eps=1e-4, scale=3.0)

# sizes that the bfloat16 kernels like (multiples of 16, head sizes of the matrix-core kernels); one key/value head per
# head in the window attention, one for all in the chunked one; one block; a convolution of 5 taps; a window and a chunk
# that are whole pages; no scaling of the rotation's frequencies
CFG_B = config(200, 128, [
    {"type": "parallel", "mixer": parallel(chunk_attention(4, 1, 32, 32, 0.2, 32), retention(2, 64, 64, [0.96, 0.99], 64), 1.0, 0.5), "mlp": None},
    {"type": "attention", "mixer": window_attention(4, 4, 64, 64, 0.125, 48, 64), "mlp": dense(256)},
    {"type": "rglru", "mixer": {"width": 128, "blocks": 1, "conv": 5}, "mlp": dense(128)},
    {"type": "attention", "mixer": window_attention(2, 1, 64, 32, 0.15, 80, 32, factor=4.0), "mlp": dense(64)},
], eps=1e-6, scale=0.5)

# head sizes that are no multiples of 8 (20 with a rotation of 6 dims; 12 in the chunked attention; 20 in retention, with
# values of 12), a convolution of one tap (no inputs to carry), a window of 1 (a token sees itself alone) and a chunk of 1
CFG_C = config(97, 40, [
    {"type": "attention", "mixer": window_attention(2, 1, 20, 12, 0.3, 1, 6, base=50.0, factor=1.5), "mlp": dense(24)},
    {"type": "rglru", "mixer": {"width": 40, "blocks": 5, "conv": 1}, "mlp": None},
    {"type": "parallel", "mixer": parallel(chunk_attention(3, 3, 12, 20, 0.35, 1), retention(2, 20, 12, [0.5, 0.999], 20), 1.0, 1.0), "mlp": dense(16)},
    {"type": "attention", "mixer": window_attention(3, 3, 20, 20, 0.25, 7, 20, base=1000.0), "mlp": None},
], eps=1e-5, scale=1.0)

# one kind of mixer only: a model without any pages, and one without any recurrent state
CFG_D = config(64, 48, [
    {"type": "rglru", "mixer": {"width": 48, "blocks": 4, "conv": 4}, "mlp": dense(32)},
    {"type": "rglru", "mixer": {"width": 32, "blocks": 2, "conv": 2}, "mlp": None},
], eps=1e-5, scale=2.0)
CFG_E = config(64, 48, [
    {"type": "attention", "mixer": window_attention(3, 3, 16, 16, 0.3, 25, 8), "mlp": None},
    {"type": "attention", "mixer": window_attention(6, 2, 8, 8, 0.4, 300, 8, factor=3.0), "mlp": dense(24)},
], eps=1e-5, scale=0.7)

CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D, "E": CFG_E}


def random_weights(cfg: dict, seed: int, sharp_keys: float = 1.0) -> Dict[str, torch.Tensor]:
    """Every tensor of the design for ``cfg``, float32 values that bfloat16 holds exactly.  ``sharp_keys``: the key
    projections (the keys' norm weights in the chunked attention) are multiplied by it, which makes the softmax peaked, so
    that single keys (often far back, or at a window's edge) carry an output and a lost or a wrongly seen key shows."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def mat(out, inp, gain=1.0):
        return torch.randn(out, inp, generator=g) * (gain / math.sqrt(inp))

    def vec(n, mean=0.0, std=0.1):
        return mean + std * torch.randn(n, generator=g)

    def softmax_half(pre, m, head_norm):
        w[pre + "q"], w[pre + "q.b"] = mat(m["heads"] * m["dim"], d), vec(m["heads"] * m["dim"], std=0.3)
        w[pre + "k"], w[pre + "k.b"] = mat(m["kv_heads"] * m["dim"], d), vec(m["kv_heads"] * m["dim"], std=0.3)
        w[pre + "v"], w[pre + "v.b"] = mat(m["kv_heads"] * m["vdim"], d), vec(m["kv_heads"] * m["vdim"], std=0.3)
        w[pre + "o"] = mat(d, m["heads"] * m["vdim"])
        if head_norm:
            w[pre + "q.norm"], w[pre + "k.norm"] = vec(m["dim"], 1.0, 0.2), vec(m["dim"], 1.0, 0.2) * sharp_keys
            w[pre + "g"] = mat(m["heads"], d, 2.0)
        else:
            w[pre + "k"] = w[pre + "k"] * sharp_keys

    w = {"embed": torch.randn(cfg["vocab"], d, generator=g) / cfg["embedding"]["scale"], "final.norm": vec(d), "head": mat(cfg["vocab"], d)}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        w[pre + "norm1"], w[pre + "norm1b"] = vec(d), vec(d)
        if layer["type"] == "attention":
            softmax_half(pre + "mix.", m, False)
        elif layer["type"] == "rglru":
            wd, bs = m["width"], m["width"] // m["blocks"]
            w[pre + "mix.y"], w[pre + "mix.y.b"] = mat(wd, d), vec(wd, std=0.3)
            w[pre + "mix.x"], w[pre + "mix.x.b"] = mat(wd, d), vec(wd, std=0.3)
            w[pre + "mix.conv"], w[pre + "mix.conv.b"] = 0.5 * torch.randn(wd, m["conv"], generator=g), vec(wd, std=0.3)
            for gate in ("ra", "ri"):
                w[pre + "mix." + gate] = torch.randn(m["blocks"], bs, bs, generator=g) * (2.0 / math.sqrt(bs))
                w[pre + "mix." + gate + ".b"] = torch.randn(m["blocks"], bs, generator=g)
            w[pre + "mix.lam"] = vec(wd, -2.0, 1.5)          # decays from close to 1 down to small ones
            w[pre + "mix.o"] = mat(d, wd)
        else:
            softmax_half(pre + "mix.left.", m["left"], True)
            r = m["right"]
            for k, rows in (("q", r["heads"] * r["dim"]), ("k", r["heads"] * r["dim"]), ("v", r["heads"] * r["vdim"]), ("g", r["heads"] * r["vdim"])):
                w[pre + "mix.right." + k] = mat(rows, d)
            w[pre + "mix.right.o"] = mat(d, r["heads"] * r["vdim"])
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            w[pre + "norm2"], w[pre + "norm2b"] = vec(d), vec(d)
            w[pre + "mlp.gate"], w[pre + "mlp.up"], w[pre + "mlp.down"] = mat(ff, d), mat(ff, d), mat(d, ff)
    return {k: v.to(torch.bfloat16).float().contiguous() for k, v in w.items()}


def make_folder(cfg: dict, weights: Dict[str, torch.Tensor], dtype: torch.dtype = torch.bfloat16, folder: Optional[str] = None) -> str:
    from llama_cu_amd.weights import write_safetensors
    folder = folder or tempfile.mkdtemp(prefix="lcu_lozezen_")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), {k: v.to(dtype) for k, v in weights.items()})
    return folder


def as_numpy(weights: Dict[str, torch.Tensor]) -> Dict[str, np.ndarray]:
    return {k: v.double().numpy() for k, v in weights.items()}


def plain_logits(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    return torch.from_numpy(P.forward(cfg, as_numpy(weights), tokens))


def tokens_of(vocab: int, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def assert_close(got, want, rel: float, what: str = "") -> None:
    """The largest difference, relative to the largest expected magnitude."""
    got, want = torch.as_tensor(got).detach().double().cpu(), torch.as_tensor(want).detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} against {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30)
    assert err <= rel, f"{what}: relative error {err:.3e} exceeds {rel:.1e}"
