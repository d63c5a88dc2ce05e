"""Several mixers side by side: all read the same input, and the mixer's output is the sum of theirs, each times a
factor: ``out = sum_i scale_i * mixer_i(h)``.  Each mixer keeps its own tensors under its own name and its own cache
need; at most one of them may hold keys and values in pages (``SeveralNeeds``).  The sum is 32-bit.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from ..kernels import ops
from .base import BuildContext, Part, PartSpec, SeveralNeeds, TensorSpec, make_part, prefixed, register_part


class SideBySide(Part):
    def __init__(self, mixers: Sequence[PartSpec], scales: Sequence[float]):
        if len(mixers) != len(scales) or not mixers:
            raise ValueError("side_by_side: one scale for every mixer, and at least one mixer")
        self.specs = list(mixers)
        self.mixers = [make_part("mixer", m) for m in mixers]
        self.scales = [float(x) for x in scales]
        self.graph_safe = all(m.graph_safe for m in self.mixers)
        # under which name each mixer with a need finds a state of its own in the one LayerCache (SeveralNeeds)
        self._state_of, kept = {}, 0
        for i, m in enumerate(self.mixers):
            if m.cache_need() is not None:
                self._state_of[i] = f"state{kept}"
                kept += 1

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {}
        for spec, m in zip(self.specs, self.mixers):
            for k, v in m.tensors().items():
                out[prefixed(spec.name, k)] = v
        return out

    def fused_groups(self, dtype, device):
        out = []
        for spec, m in zip(self.specs, self.mixers):
            out += [(tuple(prefixed(spec.name, n) for n in names), pad) for names, pad in m.fused_groups(dtype, device)]
        return out

    def load(self, tensors, build: BuildContext) -> None:
        for spec, m in zip(self.specs, self.mixers):
            pre = spec.name + "." if spec.name else ""
            m.load({k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}, build)
        self.dtype = build.dtype

    def cache_need(self):
        kept = [n for n in (m.cache_need() for m in self.mixers) if n is not None]
        return SeveralNeeds(tuple(kept)) if kept else None

    def prepare(self, step) -> None:
        for m in self.mixers:
            m.prepare(step)

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        return max(int(m.decode_splits(batch, max_ctx_len)) for m in self.mixers)

    def forward(self, h, step, cache, out_dtype=None):
        total = None
        for i, (m, scale) in enumerate(zip(self.mixers, self.scales)):
            kw = {}
            name = self._state_of.get(i)
            if name is not None and name in cache.more:
                kw["state"] = cache.more[name]
            out = m.forward(h, step, cache, out_dtype=torch.float32, **kw)
            total = ops.scaled_sum(total, out, scale)
        return total


register_part("mixer", "side_by_side", SideBySide)
