"""The generalised delta rule: a recurrent mixer whose state per head is a matrix in 32-bit.

With the mixer's input ``h`` and, per head, key channels ``i`` and value channels ``j``:

    r = W_r h,  k = W_k h,  v = W_v h                       (heads x dim each)
    w = exp(-exp(-1/2) * sigmoid(W_w2 tanh(W_w1 h) + w0))    decay per head and key channel
    a = sigmoid(W_a h + a_b)                                 removal rate per head and key channel
    u = k / sqrt(sum_i k_i^2 + 1e-6)                          the head's unit key
    S <- diag(w) S - (a * u) (u^T S) + k v^T                  decay and removal both act on S as the token found it
    o = S^T r

Each head's ``o`` is divided by its root mean square, the heads side by side are multiplied by a weight per
column and by ``sigmoid(W_g h)``, and ``W_o`` maps them back to the width.  The six projections that read ``h``
are one matrix product; everything between it and ``W_o`` is 32-bit and runs in the kernels of
``csrc/kernels/delta_rule.hip``.  The state ``[heads, dim, dim]`` lives in the engine's state slots: it starts at
zero at a request's position 0 and is carried from step to step, so a prompt may be cut anywhere.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import fused_rows
from .base import BuildContext, Part, SlotState, TensorSpec, register_part
from .linear import Weight, linear


class GeneralDelta(Part):
    graph_safe = True

    # the tensors' names under the part's own; ``names`` replaces any
    NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "a": "a", "a_bias": "a.b", "w1": "w1", "w2": "w2", "w0": "w0",
             "norm": "norm", "o": "o"}
    FUSED = ("r", "k", "v", "g", "a", "w1")          # the projections of the input, in the order of the fused matrix's rows

    def __init__(self, hidden_size: int, heads: int, head_dim: int, decay_rank: int, norm_eps: float,
                 names: Optional[Dict[str, str]] = None):
        self.hidden_size, self.heads, self.head_dim = int(hidden_size), int(heads), int(head_dim)
        self.decay_rank, self.norm_eps = int(decay_rank), float(norm_eps)
        if self.decay_rank < 1 or self.decay_rank > 512:
            raise ValueError(f"general_delta: the decay's low rank {decay_rank} is not supported (1 to 512)")
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, hd, rank, nm = self.hidden_size, self.heads * self.head_dim, self.decay_rank, self.names
        t = {nm[k]: TensorSpec((hd, d)) for k in ("r", "k", "v", "g", "a")}
        t[nm["w1"]] = TensorSpec((rank, d))
        t[nm["w2"]] = TensorSpec((hd, rank))
        t[nm["a_bias"]] = TensorSpec((hd,))
        t[nm["w0"]] = TensorSpec((hd,))
        t[nm["norm"]] = TensorSpec((hd,), init="one_plus_normal")
        t[nm["o"]] = TensorSpec((d, hd))
        return t

    def fused_groups(self, dtype, device):
        return [(tuple(self.names[k] for k in self.FUSED), 0)]

    def cache_need(self):
        return SlotState((self.heads, self.head_dim, self.head_dim), torch.float32)

    def load(self, tensors, build: BuildContext) -> None:
        nm, hd = self.names, self.heads * self.head_dim
        self.w_in = Weight(fused_rows([tensors[nm[k]] for k in self.FUSED]), build)
        self.offsets = {"r": 0, "k": hd, "v": 2 * hd, "g": 3 * hd, "a": 4 * hd, "l": 5 * hd}
        self.w_o = Weight(tensors[nm["o"]], build)
        # what enters the recurrence is 32-bit: the kernels take these in 32-bit whatever the file holds
        self.w2 = tensors[nm["w2"]].float().t().contiguous()        # [rank, heads * dim]: the kernel's lanes read neighbours
        self.w0 = tensors[nm["w0"]].float().contiguous()
        self.a_bias = tensors[nm["a_bias"]].float().contiguous()
        self.norm = tensors[nm["norm"]].float().contiguous()
        self.dtype = build.dtype

    def forward(self, h, step, cache, out_dtype=None):
        if cache.state is None:
            raise ops.KernelError("general_delta: the layer was given no state slots")
        proj = linear(h, self.w_in, out_dtype=self.dtype)
        y = ops.delta_rule(proj, self.offsets, self.w2, self.w0, self.a_bias, self.norm, cache.state, step, self.heads,
                           self.head_dim, self.head_dim, self.norm_eps)
        return linear(y, self.w_o, out_dtype=out_dtype or self.dtype)


register_part("mixer", "general_delta", GeneralDelta)
