"""Two mixers side by side: both read the same rows, and the result is
``left_scale * left(h) + right_scale * right(h)``.  The sum is left to whoever takes the result
(``parts.base.WeightedTerms``: a norm on the sublayer's output adds the two in float32 while it
normalises).  Each mixer keeps its own cache: the pair asks for a bundle with the members "left"
and "right" (a member that is a bundle itself is taken apart: "left.<name>")."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..cache.manager import BundleView
from ..cache.specs import CacheBundle
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import Mixer, WeightedTerms, register_part


class ParallelMixer(Mixer):
    def __init__(self, left: Mixer, right: Mixer, left_scale: float = 1.0,
                 right_scale: float = 1.0):
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)

    def _sides(self):
        return (("left", self.left), ("right", self.right))

    @property
    def capturable(self) -> bool:
        return self.left.capturable and self.right.capturable

    @property
    def step_tables(self):
        asked = []
        for _, m in self._sides():
            t = getattr(m, "step_tables", None)
            if t is not None:
                asked += list(t) if isinstance(t, (list, tuple)) else [t]
        return asked or None

    def cache_spec(self):
        members = []
        for side, m in self._sides():
            spec = m.cache_spec()
            if isinstance(spec, CacheBundle):
                members += [(f"{side}.{name}", s) for name, s in spec.parts]
            elif spec is not None:
                members.append((side, spec))
        return CacheBundle(tuple(members)) if members else None

    @staticmethod
    def _view(cache, side: str, mixer: Mixer):
        spec = mixer.cache_spec()
        if spec is None:
            return None
        if isinstance(spec, CacheBundle):
            return BundleView({name: cache.part(f"{side}.{name}") for name, _ in spec.parts})
        return cache.part(side)

    def tensor_specs(self) -> List[TensorSpec]:
        return self.left.tensor_specs() + self.right.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.left.bind(tensors)
        self.right.bind(tensors)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a pair of mixers does not read another layer's cache")
        out = []
        for side, m in self._sides():
            y = m.forward(x, batch, self._view(cache, side, m))
            if isinstance(y, torch.Tensor) and y.dim() == 3:
                y = ops.sum_partial_sums(y)
            out.append(y)
        if out[0].dtype != out[1].dtype:
            out = [y if y.dtype == torch.float32 else ops.cast(y, torch.float32) for y in out]
        return WeightedTerms(out[0], self.left_scale, out[1], self.right_scale)

    def weight_bytes(self) -> int:
        return self.left.weight_bytes() + self.right.weight_bytes()


register_part("mixer", "parallel", ParallelMixer)
