"""A feed-forward of many small experts of which every token uses a few.

    z = W_router h (32-bit),  s = sigmoid(z)
    the ``top`` experts with the largest scores are chosen (ties: the lower index), with s itself as weight (the weights of a token are not made to add up to one)
    out = sum over the chosen e of  W_down[e] act(W_up[e] (s_e * h))        act: the exact (erf) gelu

The weight scales what goes INTO the expert, not what comes out.  Routing, grouping by expert and the experts' products all run on
the device (``csrc/kernels/moe.hip``): nothing about which expert a token uses comes back to the host, so a
step's launches depend on its sizes alone.  The experts' matrices are laid out side by side by the loader, so
that an expert is an index.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import fused_rows
from .base import BuildContext, Part, TensorSpec, register_part


class SigmoidMoE(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, expert_size: int, experts: int, top: int, router: str = "router",
                 up: str = "e{}.up", down: str = "e{}.down"):
        """``router``, ``up``, ``down``: the tensors' names under the part's own (``{}``: the expert's index)."""
        self.hidden_size, self.expert_size = int(hidden_size), int(expert_size)
        self.experts, self.top = int(experts), int(top)
        if not 1 <= self.top <= self.experts or self.experts > 1024:
            raise ValueError(f"moe: top {top} of {experts} experts is not supported (1 <= top <= experts <= 1024)")
        self.router_name, self.up_name, self.down_name = router, up, down
        self.router = self.w_up = self.w_down = None

    def _ups(self):
        return [self.up_name.format(e) for e in range(self.experts)]

    def _downs(self):
        return [self.down_name.format(e) for e in range(self.experts)]

    def tensors(self) -> Dict[str, TensorSpec]:
        d, ff = self.hidden_size, self.expert_size
        t = {self.router_name: TensorSpec((self.experts, d))}
        for n in self._ups():
            t[n] = TensorSpec((ff, d))
        for n in self._downs():
            t[n] = TensorSpec((d, ff))
        return t

    def fused_groups(self, dtype, device):
        return [(tuple(self._ups()), 0), (tuple(self._downs()), 0)]

    def load(self, tensors, build: BuildContext) -> None:
        d, ff, n = self.hidden_size, self.expert_size, self.experts
        self.router = tensors[self.router_name].float().contiguous()        # the router is 32-bit
        self.w_up = fused_rows([tensors[k] for k in self._ups()]).view(n, ff, d)
        self.w_down = fused_rows([tensors[k] for k in self._downs()]).view(n, d, ff)
        if ff % 8:
            # the products load 16 bytes at a time along k: an expert whose size is no multiple of 8 gets rows of zeros
            # in its up matrix and the columns of zeros that meet them in its down matrix (gelu(0) = 0: nothing changes)
            pad = 8 - ff % 8
            self.w_up = torch.cat([self.w_up, self.w_up.new_zeros(n, pad, d)], dim=1).contiguous()
            self.w_down = torch.cat([self.w_down, self.w_down.new_zeros(n, d, pad)], dim=2).contiguous()
        self.dtype = build.dtype

    def forward(self, h, add_to: Optional[torch.Tensor] = None):
        """``add_to``: float32 ``[n, d]`` that takes the output in (and is returned); without it the output comes
        back in the compute type."""
        ids, wts = ops.moe_route(h, self.router, self.top)
        out = add_to if add_to is not None else torch.zeros((h.shape[0], self.hidden_size), dtype=torch.float32, device=h.device)
        ops.moe_experts(h, ids, wts, self.w_up, self.w_down, out)
        return out if add_to is not None else out.to(self.dtype)


register_part("ffn", "sigmoid_moe", SigmoidMoE)
