"""minGRU: a gated recurrence whose gates read the current token only.

``z = sigmoid(W_z h + b_z)``, ``u = W_x h + b_x``; the candidate is ``u + 1/2`` where ``u >= 0``
and ``sigmoid(u)`` below; element by element ``S_t = (1 - z) S_(t-1) + z * candidate`` from a zero
state; the output is ``W_o (S_t * silu(W_g h))``.  The three input products run as one; gates,
candidates and the state are float32 (computed from the products' results as they are stored), the state a slot
of ``inner`` floats a request.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List

import numpy as np
import torch

from ..cache.specs import FixedState
from ..kernels import ops, profile, tuning
from ..weights.spec import TensorSpec
from .base import Mixer, StepTables, register_part
from .linear import Linear


@dataclass(frozen=True)
class ScanChunks(StepTables):
    """The segments of a step cut into runs of at most ``rows`` rows for a scan in passes:
    ``scan_chunks`` [chunks, 3] = (segment, first row, rows) and ``scan_seg_chunk0`` [S + 1], the
    first chunk of every segment."""
    rows: int

    family = "scan_chunks"
    decode_constant = True

    def combine(self, others):
        return ScanChunks(min([self.rows] + [o.rows for o in others]))

    def build(self, step):
        seg_start = step.arrays["seg_start"].astype(np.int64)
        n = seg_start[1:] - seg_start[:-1]
        per = (n + self.rows - 1) // self.rows
        first = np.zeros(n.shape[0] + 1, dtype=np.int64)
        np.cumsum(per, out=first[1:])
        seg = np.repeat(np.arange(n.shape[0], dtype=np.int64), per)
        k = np.arange(int(per.sum()), dtype=np.int64) - np.repeat(first[:-1], per)
        row0 = seg_start[seg] + k * self.rows
        rows = np.minimum(self.rows, n[seg] - k * self.rows)
        return ({"scan_chunks": np.stack([seg, row0, rows], axis=1).astype(np.int32),
                 "scan_seg_chunk0": first.astype(np.int32)}, {})


class MinGRU(Mixer):
    def __init__(self, prefix: str, width: int, inner: int, dtype: torch.dtype, names=None,
                 weight_suffix: str = ".weight", bias_suffix: str = ".bias"):
        n = {"z": "z", "x": "x", "g": "g", "o": "o"}
        n.update(names or {})
        self.prefix, self.width, self.inner, self.dtype = prefix, width, inner, dtype
        self.gates = Linear([prefix + n["z"], prefix + n["x"], prefix + n["g"]], width,
                            [inner, inner, inner], bias=[True, True, False],
                            stage="matmul_in_proj", weight_suffix=weight_suffix,
                            bias_suffix=bias_suffix)
        self.out = Linear([prefix + n["o"]], inner, [width], stage="matmul_out_proj",
                          weight_suffix=weight_suffix)

    @property
    def step_tables(self) -> ScanChunks:
        return ScanChunks(tuning.SCAN_CHUNK_ROWS)

    def cache_spec(self):
        return FixedState((self.inner,), "float32")

    def tensor_specs(self) -> List[TensorSpec]:
        return self.gates.tensor_specs() + self.out.tensor_specs()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.gates.bind(tensors)
        self.out.bind(tensors)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        if shared_cache:
            raise ValueError("a recurrent state cannot be read by another layer")
        # (the products' results are stored in the compute dtype, as every other product's; what
        # the recurrence makes of them is float32)
        proj = self.gates.forward(x)
        chunked = batch.max_segment_rows > tuning.SCAN_CHUNKS_FROM_ROWS
        with profile.scope("scan"):
            y = ops.mingru_scan(proj, cache.state, batch.seg_start, batch.seg_pos0,
                                batch.seg_slot, self.dtype,
                                chunks=batch.extra.get("scan_chunks") if chunked else None,
                                seg_chunk0=batch.extra.get("scan_seg_chunk0") if chunked else None)
        return self.out.forward(y, partial_sums=True)

    def weight_bytes(self) -> int:
        return self.gates.weight_bytes() + self.out.weight_bytes()


register_part("mixer", "mingru", MinGRU)
