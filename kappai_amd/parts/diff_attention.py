"""Differential attention over the paged cache, with a sliding window.

A head has two score maps over the same values.  With a1, a2 the maps' outputs,
``o = a1 - lambda a2``; every head's ``o`` is divided by its own root mean square (no weight) and
multiplied by ``1 - diff``; ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff`` is one number a
layer.  Scores are ``q . k * scale`` with an ordinary softmax over the keys a position sees:
itself and the ``window - 1`` before it (``window`` None: all).  Nothing rotates here; a position
encoding, if any, belongs to the model.  Query head h reads kv head ``h // (H / G)``.

The maps run as heads of their own through the framework's paged attention kernels (see
``ops.diff_store``): 2H heads on 2G kv heads of one size that holds queries, keys and values.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..cache.specs import PagedKV
from ..kernels import ops, profile, tuning
from ..weights.spec import INIT_SMALL, VECTOR, TensorSpec
from .attention import AttentionTiles
from .base import Mixer, register_part
from .linear import Linear


class DifferentialAttention(Mixer):
    def __init__(self, prefix: str, width: int, num_heads: int, num_kv_heads: int, dim: int,
                 vdim: int, scale: float, diff: float, norm_eps: float, dtype: torch.dtype,
                 window: Optional[int] = None, names=None, weight_suffix: str = ".weight"):
        n = {"q": "q", "k": "k", "v": "v", "o": "o", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2",
             "lk2": "lk2"}
        n.update(names or {})
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads cannot be shared out over {num_kv_heads} kv heads")
        self.prefix, self.width, self.dtype = prefix, width, dtype
        self.H, self.G, self.d, self.dv = num_heads, num_kv_heads, dim, vdim
        self.head_size = 16 * ((max(dim, vdim) + 15) // 16)      # one size for the kernels' heads
        self.scale, self.diff, self.norm_eps = float(scale), float(diff), float(norm_eps)
        self.window = int(window) if window else None
        self.qkv = Linear([prefix + n["q"], prefix + n["k"], prefix + n["v"]], width,
                          [num_heads * 2 * dim, num_kv_heads * 2 * dim, num_kv_heads * vdim],
                          stage="matmul_qkv", weight_suffix=weight_suffix)
        self.out = Linear([prefix + n["o"]], num_heads * vdim, [width], stage="matmul_attn_out",
                          weight_suffix=weight_suffix)
        self._lambda_names = [prefix + n[k] for k in ("lq1", "lk1", "lq2", "lk2")]
        self.lam: Optional[float] = None

    @property
    def step_tables(self) -> AttentionTiles:
        ok = (self.dtype == torch.bfloat16 and self.H // self.G <= 16 and self.head_size <= 256)
        return AttentionTiles(ops.ATTENTION_TILE_ROWS,
                              tuning.LONE_ROWS_FROM if ok and tuning.LONE_ROWS_FROM else None)

    def cache_spec(self):
        return PagedKV(2 * self.G, self.head_size, self.window)

    def tensor_specs(self) -> List[TensorSpec]:
        return (self.qkv.tensor_specs() + self.out.tensor_specs()
                + [TensorSpec(name, (self.d,), VECTOR, INIT_SMALL) for name in self._lambda_names])

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.qkv.bind(tensors)
        self.out.bind(tensors)
        lq1, lk1, lq2, lk2 = (tensors[name].to(torch.float32).cpu() for name in self._lambda_names)
        self.lam = (math.exp(float((lq1 * lk1).sum())) - math.exp(float((lq2 * lk2).sum()))
                    + self.diff)

    def forward(self, x, batch, cache, shared_cache: bool = False):
        H, G, D = self.H, self.G, self.head_size
        proj = self.qkv.forward(x)
        tables = batch.block_tables[cache.group]
        k_pool, v_pool = cache.pool("k"), cache.pool("v")
        with profile.scope("rope_kvput"):
            q = ops.diff_store(proj, H, G, self.d, self.dv, D, k_pool, v_pool, batch.row_pos,
                               batch.row_seg, tables, cache.page_size, store_kv=not shared_cache)
        with profile.scope("attn"):
            ctx = ops.paged_attention(q, 2 * H, 2 * G, D, k_pool, v_pool, batch.row_pos,
                                      batch.row_seg, tables, cache.page_size, self.scale,
                                      window=self.window or 0,
                                      q_tiles=batch.extra.get("q_tiles"),
                                      single_rows=batch.max_segment_rows == 1,
                                      max_position=batch.max_position,
                                      lone_rows=batch.extra.get("lone_rows"),
                                      max_lone_position=batch.numbers.get("max_lone_position",
                                                                          -1))
            o = ops.diff_combine(ctx, H, G, self.dv, D, self.lam, self.norm_eps, 1.0 - self.diff)
        return self.out.forward(o, partial_sums=True)

    def weight_bytes(self) -> int:
        return self.qkv.weight_bytes() + self.out.weight_bytes()


register_part("mixer", "differential_attention", DifferentialAttention)
