"""Retention: linear attention with a fixed decay per head, without softmax and without a denominator.

With the mixer's input ``h`` and, per head, key channels ``i`` and value channels ``j``:

    q = W_q h,  k = W_k h   (heads x dim),   v = W_v h,  g = W_g h   (heads x vdim)
    q, k <- rotated by the token's position (the position part: a rotation of the first dims of each head)
    k <- k * dim^(-1/2)
    S <- decay[head] * S + k v^T          o = S^T q

Each head's ``o`` is divided by its root mean square (no weight), the heads side by side are multiplied by
``silu(g)``, and ``W_o`` maps them back to the width.  The four projections are one matrix product; everything
between it and ``W_o`` is 32-bit (``csrc/kernels/retention.hip``).  The state ``[heads, dim, vdim]`` lives in the
engine's state slots: zero at a request's position 0, carried from step to step, so a prompt may be cut anywhere.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..kernels import ops
from ..weights.loader import fused_rows
from .base import BuildContext, Part, PartSpec, SlotState, TensorSpec, make_part, register_part
from .linear import Weight, linear


class Retention(Part):
    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}
    FUSED = ("q", "k", "v", "g")

    def __init__(self, hidden_size: int, heads: int, head_dim: int, value_dim: int, decay: Sequence[float], norm_eps: float,
                 position: Optional[PartSpec] = None, key_scale: Optional[float] = None, names: Optional[Dict[str, str]] = None):
        """``decay``: one factor per head.  ``key_scale``: what the keys are multiplied by after the rotation
        (default ``head_dim ** -0.5``).  ``position``: a rotation (or none)."""
        self.hidden_size, self.heads, self.head_dim, self.value_dim = int(hidden_size), int(heads), int(head_dim), int(value_dim)
        self.decay = [float(x) for x in decay]
        if len(self.decay) != self.heads:
            raise ValueError(f"retention: {len(self.decay)} decays for {self.heads} heads")
        if self.head_dim > 256:
            raise ValueError(f"retention: head_dim {head_dim} is not supported by the kernel (at most 256)")
        self.norm_eps = float(norm_eps)
        self.key_scale = float(key_scale) if key_scale is not None else float(head_dim) ** -0.5
        self.names = dict(self.NAMES, **(names or {}))
        self.position = make_part("position", position or PartSpec("none"))
        self.graph_safe = self.position.graph_safe
        self.w_in = self.w_o = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, hk, hv, nm = self.hidden_size, self.heads * self.head_dim, self.heads * self.value_dim, self.names
        return {nm["q"]: TensorSpec((hk, d)), nm["k"]: TensorSpec((hk, d)), nm["v"]: TensorSpec((hv, d)),
                nm["g"]: TensorSpec((hv, d)), nm["o"]: TensorSpec((d, hv))}

    def fused_groups(self, dtype, device):
        return [(tuple(self.names[k] for k in self.FUSED), 0)]

    def cache_need(self):
        return SlotState((self.heads, self.head_dim, self.value_dim), torch.float32)

    def load(self, tensors, build: BuildContext) -> None:
        nm, hk, hv = self.names, self.heads * self.head_dim, self.heads * self.value_dim
        self.w_in = Weight(fused_rows([tensors[nm[k]] for k in self.FUSED]), build)
        self.offsets = {"q": 0, "k": hk, "v": 2 * hk, "g": 2 * hk + hv}
        self.w_o = Weight(tensors[nm["o"]], build)
        self.decay_vec = torch.tensor(self.decay, dtype=torch.float32, device=build.device)
        self.position.load({}, build)
        if type(self.position).apply is not Part.apply or self.position.score_slopes() is not None:
            raise ValueError("retention: the position part must be a rotation or none")
        self.dtype = build.dtype

    def forward(self, h, step, cache, out_dtype=None, state: Optional[torch.Tensor] = None):
        state = state if state is not None else cache.state
        if state is None:
            raise ops.KernelError("retention: the layer was given no state slots")
        rot = self.position.rotary_tables()
        cos, sin, rot_dim, pairing = rot if rot is not None else (None, None, 0, 0)
        rows = linear(h, self.w_in, out_dtype=torch.float32)
        y = ops.retention(rows, self.offsets, self.decay_vec, state, step, self.heads, self.head_dim, self.value_dim,
                          self.key_scale, self.norm_eps, self.dtype, cos=cos, sin=sin, rot_dim=rot_dim, pairing=pairing)
        return linear(y, self.w_o, out_dtype=out_dtype or self.dtype)


register_part("mixer", "retention", Retention)
