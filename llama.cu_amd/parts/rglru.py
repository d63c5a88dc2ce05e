"""A recurrent block around a real-gated linear recurrent unit.

Two branches of ``width`` channels read the mixer's input ``h``:

    y = gelu_tanh(W_y h + b_y)
    u = conv(W_x h + b_x)                 a causal convolution over time on each channel, with a bias
    r = sigmoid(A u + b_a),  i = sigmoid(I u + b_i)      A, I block-diagonal: the channels in ``blocks`` equal parts
    a = exp(-c * r * softplus(lam)),      S <- a * S + sqrt(1 - a^2) * i * u         (from S = 0, the first token too)
    out = W_o (S * y)

The two input projections are one matrix product with 32-bit output; the convolution, the gates, the decay and the
recurrence are 32-bit (``csrc/kernels/rglru.hip``).  Per request the engine's state slot holds ``[taps, width]``
floats: the last ``taps - 1`` inputs of the convolution and ``S``; both start at zero at position 0.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import fused_rows
from .base import BuildContext, Part, SlotState, TensorSpec, register_part
from .linear import Weight, linear


class RGLRU(Part):
    graph_safe = True
    NAMES = {"y": "y", "y_bias": "y.b", "x": "x", "x_bias": "x.b", "conv": "conv", "conv_bias": "conv.b", "a_gate": "ra",
             "a_gate_bias": "ra.b", "i_gate": "ri", "i_gate_bias": "ri.b", "lam": "lam", "o": "o"}

    def __init__(self, hidden_size: int, width: int, blocks: int, taps: int, decay_exponent: float = 8.0,
                 names: Optional[Dict[str, str]] = None):
        """``decay_exponent``: the ``c`` of ``a = exp(-c r softplus(lam))``."""
        self.hidden_size, self.width, self.blocks, self.taps = int(hidden_size), int(width), int(blocks), int(taps)
        if self.width % self.blocks:
            raise ValueError(f"rglru: width {width} is no multiple of {blocks} blocks")
        if self.width // self.blocks > 1024 or not 1 <= self.taps <= 16:
            raise ValueError(f"rglru: blocks of {self.width // self.blocks} channels or {taps} taps are not supported (at most 1024; 1 to 16)")
        self.c = float(decay_exponent)
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, w, b, nm = self.hidden_size, self.width, self.blocks, self.names
        bs = w // b
        return {nm["y"]: TensorSpec((w, d)), nm["y_bias"]: TensorSpec((w,)), nm["x"]: TensorSpec((w, d)), nm["x_bias"]: TensorSpec((w,)),
                nm["conv"]: TensorSpec((w, self.taps)), nm["conv_bias"]: TensorSpec((w,)),
                nm["a_gate"]: TensorSpec((b, bs, bs)), nm["a_gate_bias"]: TensorSpec((b, bs)),
                nm["i_gate"]: TensorSpec((b, bs, bs)), nm["i_gate_bias"]: TensorSpec((b, bs)),
                nm["lam"]: TensorSpec((w,)), nm["o"]: TensorSpec((d, w))}

    def fused_groups(self, dtype, device):
        return [((self.names["y"], self.names["x"]), 0)]

    def cache_need(self):
        return SlotState((self.taps, self.width), torch.float32)

    def load(self, tensors, build: BuildContext) -> None:
        nm, w = self.names, self.width
        self.w_in = Weight(fused_rows([tensors[nm["y"]], tensors[nm["x"]]]), build)
        self.w_o = Weight(tensors[nm["o"]], build)
        f32 = lambda name: tensors[nm[name]].float().contiguous()
        # what enters the recurrence is 32-bit whatever the file holds; the gates' matrices transposed ([block][in][out])
        self.bias = torch.cat([f32("y_bias"), f32("x_bias")]).contiguous()
        self.conv_w, self.conv_b = f32("conv"), f32("conv_bias")
        self.wa_t = f32("a_gate").transpose(1, 2).contiguous()
        self.wi_t = f32("i_gate").transpose(1, 2).contiguous()
        self.ba, self.bi = f32("a_gate_bias").reshape(w).contiguous(), f32("i_gate_bias").reshape(w).contiguous()
        self.lam = f32("lam")
        self.dtype = build.dtype

    def forward(self, h, step, cache, out_dtype=None, state: Optional[torch.Tensor] = None):
        state = state if state is not None else cache.state
        if state is None:
            raise ops.KernelError("rglru: the layer was given no state slots")
        rows = linear(h, self.w_in, out_dtype=torch.float32)
        y = ops.rglru(rows, 0, self.width, self.bias, self.conv_w, self.conv_b, self.wa_t, self.wi_t, self.ba, self.bi,
                      self.lam, self.c, state, step, self.dtype)
        return linear(y, self.w_o, out_dtype=out_dtype or self.dtype)


register_part("mixer", "rglru", RGLRU)
