"""RMS norm in groups: the row is cut into ``groups`` equal consecutive parts, each divided by its
own ``sqrt(mean(part^2) + eps)``, and the whole multiplied by the weight.  One group is the plain
RMS norm.  Computed in float32 and fused with the residual sum that precedes it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile
from ..weights.spec import INIT_ONES, VECTOR, TensorSpec
from .base import Norm, register_part


class GroupRMSNorm(Norm):
    takes_partial_sums = True      # the kernel adds [S, T, width] partial sums itself, in order
    takes_out_dtype = True         # add_norm(..., out_dtype=torch.float32) hands out 32-bit rows

    def __init__(self, name: str, width: int, eps: float, groups: int, dtype: torch.dtype,
                 suffix: str = ".weight"):
        if groups < 1 or width % groups:
            raise ValueError(f"{name}: a width of {width} cannot be cut into {groups} equal groups")
        self.name, self.width, self.eps, self.groups, self.dtype = (
            name, width, float(eps), int(groups), dtype)
        self.tensor_name = name + suffix
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.tensor_name, (self.width,), VECTOR, INIT_ONES)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tensor_name].to(torch.float32).contiguous()

    def add_norm(self, resid, delta, rows=None, out_dtype=None):
        if isinstance(delta, ops.Added):
            delta = None             # the sum is in ``resid`` already
        with profile.scope("rmsnorm" if rows is None else "logits_norm"):
            return ops.add_group_rmsnorm(resid, delta, self.weight, self.eps, self.groups,
                                         out_dtype or self.dtype, rows=rows,
                                         write_resid=rows is None)

    def add_norm_conv_step(self, resid, delta, conv, batch, cache):
        """The norm and the short convolution behind it (``parts.input_conv.ShortInputConv``) in
        one kernel, for a step whose segments are single rows."""
        if isinstance(delta, ops.Added):
            delta = None
        with profile.scope("rmsnorm"):
            return ops.add_group_rmsnorm_canon_step(
                resid, delta, self.weight, self.eps, self.groups, conv.taps, cache.state,
                batch.row_pos, batch.seg_slot, conv.dtype)

    def weight_bytes(self) -> int:
        return self.width * 4


register_part("norm", "group_rmsnorm", GroupRMSNorm)
