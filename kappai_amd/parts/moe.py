"""Mixture of experts: ``experts`` small gated feed-forward layers, of which every token uses
``top``.  Router logits ``W_router h`` in float32; the ``top`` largest are chosen and their
weights are the softmax over the chosen logits alone; the output is the weighted sum of the
chosen experts' ``W_down (silu(W_gate h) * W_up h)``.  Experts have no biases.

The step's (row, choice) pairs are sorted by expert on the GPU and the experts' products run
over that order tile by tile, so nothing of the routing is read by the host.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_NORMAL, MATRIX, TensorSpec
from .base import FeedForward, register_part


class MixtureOfExperts(FeedForward):
    def __init__(self, prefix: str, width: int, hidden: int, experts: int, top: int,
                 dtype: torch.dtype, names=None, weight_suffix: str = ".weight"):
        n = {"router": "router", "expert": "e{}.", "gate": "gate", "up": "up", "down": "down"}
        n.update(names or {})
        if not 1 <= top <= min(experts, ops.MOE_MAX_TOP):
            raise ValueError(f"{prefix}: {top} of {experts} experts a token; the kernels take 1 to "
                             f"{ops.MOE_MAX_TOP}")
        self.prefix, self.width, self.hidden, self.dtype = prefix, width, hidden, dtype
        self.E, self.top = int(experts), int(top)
        self._router = prefix + n["router"] + weight_suffix
        self._expert = [{k: prefix + n["expert"].format(e) + n[k] + weight_suffix
                         for k in ("gate", "up", "down")} for e in range(self.E)]
        self.router: Optional[torch.Tensor] = None
        self.w_gate = self.w_up = self.w_down = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self._router, (self.E, self.width), MATRIX, INIT_NORMAL)]
        for names in self._expert:
            specs.append(TensorSpec(names["gate"], (self.hidden, self.width), MATRIX, INIT_NORMAL))
            specs.append(TensorSpec(names["up"], (self.hidden, self.width), MATRIX, INIT_NORMAL))
            specs.append(TensorSpec(names["down"], (self.width, self.hidden), MATRIX, INIT_NORMAL))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.router = tensors[self._router].to(torch.float32).contiguous()

        def stacked(key):
            w = torch.stack([tensors[names[key]].to(self.dtype) for names in self._expert]
                            ).contiguous()
            # bfloat16 matrices whose shape allows it are kept in the order the matrix-core
            # kernel loads them, and only so
            if w.is_cuda and tuning.FRAGMENT_ORDER and ops.ExpertFragments.fits(w):
                return ops.ExpertFragments.of(w)
            return w
        up = stacked("up")
        self.w_gate = stacked("gate")
        self.w_up = up
        self.w_down = stacked("down")

    def forward(self, x, batch):
        with profile.scope("router"):
            chosen, weights = ops.moe_route(x, self.router, self.top)
            plan = ops.moe_plan(chosen, self.E)
        with profile.scope("matmul_ffn_gate_up", 0):
            act = ops.moe_experts_gated(x, self.w_gate, self.w_up, plan)
        with profile.scope("matmul_ffn_down", 0):
            y = ops.moe_experts_down(act, self.w_down, plan)
            return ops.moe_combine(y, weights, plan)

    def weight_bytes(self) -> int:
        """What a step of one row reads: the router and ``top`` experts."""
        per_expert = 3 * self.hidden * self.width * self.w_gate.element_size()
        return self.router.numel() * 4 + self.top * per_expert


register_part("feed_forward", "moe", MixtureOfExperts)
