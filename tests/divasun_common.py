"""Shared by the Divasun tests: small configurations that differ in every size and option, random weights from
the tests' own generator, model folders in temporary places, and the plain implementation's logits."""
from __future__ import annotations

import json
import math
import os
import tempfile
from typing import Dict, List, Optional

import torch

import plain_divasun as P


def attention(heads, kv_heads, dim, vdim, scale, q_temp=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def config(vocab, width, layers, taps, eps, scale):
    return {"architecture": "Divasun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "embedding": {"scale": scale}, "layers": layers}


# no size a power of two where it need not be; groups of three heads; values narrower than keys; a layer that reads
# another's keys and values; a layer without feed-forward; several experts a token; a delta rule whose head size
# no kernel keeps in registers; a temperature that changes every 7 positions
CFG_A = config(131, 72, [
    {"type": "attention", "mixer": attention(6, 2, 24, 16, 0.31, q_temp=(0.5, 7)), "mlp": moe(5, 2, 40)},
    {"type": "general_delta", "mixer": {"heads": 3, "dim": 32}, "mlp": None},
    {"type": "attention", "mixer": attention(6, 2, 24, 16, 0.2, kv_from=0), "mlp": moe(7, 3, 24)},
    {"type": "general_delta", "mixer": {"heads": 2, "dim": 20}, "mlp": moe(4, 4, 16)},
], taps=3, eps=1e-4, scale=3.0)
RANKS_A = {1: 5, 3: 3}

# sizes that the bfloat16 kernels take (multiples of 8, but for one expert size); as many key/value heads as heads; one expert a token
CFG_B = config(200, 128, [
    {"type": "general_delta", "mixer": {"heads": 2, "dim": 64}, "mlp": moe(6, 1, 64)},
    {"type": "attention", "mixer": attention(4, 4, 32, 32, 0.18, q_temp=(0.25, 16)), "mlp": moe(6, 2, 32)},
    {"type": "general_delta", "mixer": {"heads": 4, "dim": 16}, "mlp": moe(3, 1, 44)},
    {"type": "attention", "mixer": attention(4, 4, 32, 32, 0.25, kv_from=1), "mlp": None},
], taps=4, eps=1e-5, scale=8.0)
RANKS_B = {0: 8, 2: 4}

# a convolution of one tap (no state), of two taps; attention first and alone
CFG_C1 = config(97, 64, [
    {"type": "attention", "mixer": attention(2, 1, 16, 40, 0.4), "mlp": moe(3, 1, 32)},
    {"type": "general_delta", "mixer": {"heads": 1, "dim": 48}, "mlp": moe(2, 2, 24)},
], taps=1, eps=1e-6, scale=1.0)
CFG_C2 = dict(CFG_C1, canon={"taps": 2})
RANKS_C = {1: 2}


# one kind of mixer only: a model without any pages, and one without any recurrent state
CFG_D = config(64, 48, [
    {"type": "general_delta", "mixer": {"heads": 2, "dim": 16}, "mlp": moe(3, 1, 16)},
    {"type": "general_delta", "mixer": {"heads": 1, "dim": 24}, "mlp": None},
], taps=3, eps=1e-5, scale=2.0)
RANKS_D = {0: 3, 1: 6}
CFG_E = config(64, 48, [
    {"type": "attention", "mixer": attention(3, 3, 8, 8, 0.5, q_temp=(1.0, 1)), "mlp": None},
    {"type": "attention", "mixer": attention(3, 3, 8, 8, 0.3, kv_from=0), "mlp": moe(2, 1, 8)},
], taps=5, eps=1e-5, scale=0.5)


# head sizes of the attention that are no multiples of 8 (the engine fills its heads up with dims of zeros): 20 with
# values of 12; 60, which filled up is a size of the matrix-core kernels, with values of 64
CFG_F = config(80, 64, [
    {"type": "attention", "mixer": attention(3, 1, 20, 12, 0.3, q_temp=(0.4, 5)), "mlp": moe(3, 1, 16)},
    {"type": "attention", "mixer": attention(2, 2, 60, 64, 0.15), "mlp": None},
    {"type": "attention", "mixer": attention(3, 1, 20, 12, 0.4, kv_from=0), "mlp": moe(2, 2, 24)},
], taps=2, eps=1e-5, scale=1.5)


def random_weights(cfg: dict, ranks: Dict[int, int], seed: int, sharp_keys: float = 1.0) -> Dict[str, torch.Tensor]:
    """Every tensor of the design for ``cfg`` (``ranks``: the decay's low rank per delta layer), bfloat16-exact
    float32 values.  ``sharp_keys``: the keys' norm weights are multiplied by it, which makes the softmax peaked, so
    that single keys (often far back) carry an output and a lost key shows."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def mat(out, inp, gain=1.0):
        return torch.randn(out, inp, generator=g) * (gain / math.sqrt(inp))

    def vec(n, mean=0.0, std=0.1):
        return mean + std * torch.randn(n, generator=g)

    w = {"embed": torch.randn(cfg["vocab"], d, generator=g) / cfg["embedding"]["scale"],
         "final.norm": vec(d, 1.0), "final.norm.b": vec(d), "head": mat(cfg["vocab"], d)}
    taps = cfg["canon"]["taps"]
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        w[pre + "norm1"], w[pre + "norm1.b"] = vec(d, 1.0), vec(d)
        w[pre + "canon1"] = 0.3 * torch.randn(d, taps, generator=g)
        hd = m["heads"] * m["dim"]
        if layer["type"] == "general_delta":
            for k in ("r", "k", "v", "g", "a"):
                w[pre + "mix." + k] = mat(hd, d)
            w[pre + "mix.a.b"] = vec(hd, 0.0, 1.0)
            w[pre + "mix.w1"] = mat(ranks[i], d)
            w[pre + "mix.w2"] = mat(hd, ranks[i], 2.0)
            w[pre + "mix.w0"] = vec(hd, 0.0, 1.0)
            w[pre + "mix.norm"] = vec(hd, 1.0)
            w[pre + "mix.o"] = mat(d, hd)
        else:
            w[pre + "mix.q"] = mat(hd, d)
            w[pre + "mix.q.norm"] = vec(hd, 1.0)
            w[pre + "mix.o"] = mat(d, m["heads"] * m["vdim"])
            if m.get("kv_from") is None:
                w[pre + "mix.k"] = mat(m["kv_heads"] * m["dim"], d)
                w[pre + "mix.v"] = mat(m["kv_heads"] * m["vdim"], d)
                w[pre + "mix.k.norm"] = vec(m["kv_heads"] * m["dim"], 1.0) * sharp_keys
        f = layer.get("mlp")
        if f is not None:
            w[pre + "norm2"], w[pre + "norm2.b"] = vec(d, 1.0), vec(d)
            w[pre + "canon2"] = 0.3 * torch.randn(d, taps, generator=g)
            w[pre + "mlp.router"] = mat(f["router"]["experts"], d, 8.0)
            for e in range(f["router"]["experts"]):
                w[pre + f"mlp.e{e}.up"] = mat(f["expert"]["ff"], d)
                w[pre + f"mlp.e{e}.down"] = mat(d, f["expert"]["ff"])
    return {k: v.to(torch.bfloat16).float().contiguous() for k, v in w.items()}


def make_folder(cfg: dict, weights: Dict[str, torch.Tensor], dtype: torch.dtype = torch.bfloat16, folder: Optional[str] = None) -> str:
    from llama_cu_amd.weights import write_safetensors
    folder = folder or tempfile.mkdtemp(prefix="lcu_divasun_")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), {k: v.to(dtype) for k, v in weights.items()})
    return folder


def plain_logits(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    return P.forward(cfg, weights, tokens)


def tokens_of(vocab: int, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def safe_tokens(cfg: dict, weights: Dict[str, torch.Tensor], n: int, seed: int, margin: float = 0.12) -> List[int]:
    """``n`` random tokens for which the plain model's routers make no close call (every chosen logit at least
    ``margin`` above the first that is not chosen): a choice of experts is discrete, and bfloat16 rounding (of a
    layer's input, a hundredth of its size after a few layers) may make a close one fall the other way, which is no
    fault and would hide those that are.  Such sequences are rare among long ones: comparisons of long bfloat16 runs
    are made between two runs of the engine instead."""
    for k in range(400):
        toks = tokens_of(cfg["vocab"], n, seed + 1000 * k)
        margins: List[float] = []
        P.forward(cfg, weights, toks, margins=margins)
        if not margins or min(margins) >= margin:
            return toks
    raise AssertionError("no sequence without a close call of a router was found")


def assert_close(got: torch.Tensor, want: torch.Tensor, rel: float, what: str = "") -> None:
    """The largest difference, relative to the largest expected magnitude."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} against {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30)
    assert err <= rel, f"{what}: relative error {err:.3e} exceeds {rel:.1e}"
