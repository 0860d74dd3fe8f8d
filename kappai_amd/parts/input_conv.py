"""A short causal convolution in front of a sublayer: what the sublayer reads, ``h``, becomes
``h + conv(h)`` with ``conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j]`` on every channel by
itself, zeros before the sequence's start.  The last ``taps - 1`` inputs are a request's state."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.specs import FixedState
from ..kernels import ops, profile
from ..weights.spec import INIT_SMALL, VECTOR, TensorSpec
from .base import Part


class ShortInputConv(Part):
    def __init__(self, name: str, width: int, taps: int, dtype: torch.dtype):
        if not 1 <= taps <= ops.CANON_MAX_TAPS:
            raise ValueError(f"{name}: {taps} taps; the kernel takes 1 to {ops.CANON_MAX_TAPS}")
        self.name, self.width, self.n_taps, self.dtype = name, width, int(taps), dtype
        self.taps: Optional[torch.Tensor] = None

    def cache_spec(self):
        return FixedState((self.n_taps - 1, self.width), "float32")

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.width, self.n_taps), VECTOR, INIT_SMALL)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.taps = tensors[self.name].to(torch.float32).contiguous()

    def forward(self, h: torch.Tensor, batch, cache) -> torch.Tensor:
        """``h``: float32 rows [T, width]; returns ``h + conv(h)`` in the compute dtype and
        brings the state of every request of the step up to date."""
        with profile.scope("short_conv"):
            return ops.canon_conv(h, self.taps, cache.state, batch.row_pos, batch.row_seg,
                                  batch.seg_start, batch.seg_slot, self.dtype)

    def weight_bytes(self) -> int:
        return self.width * self.n_taps * 4
