"""Grouped-head softmax attention over a row-per-token cache: every token
owns one paged cache row [keys of all kv heads | values of all kv heads], and
one kernel (ops.row_attention) serves prompt portions and decode rows alike,
reading keys and values from the cache only, so a position's result does not
depend on how its prompt was cut or batched. Queries are prepared in fp32 by
ops.qkv_store, which also scatters the step's keys and values; scores,
softmax and the per-head post-processing are fp32.

Two mixers are built on it:

DifferentialAttention — every head has TWO query/key maps over the same
values. With a1, a2 the two softmax results, o = a1 - lambda * a2, then o is
divided by its RMS over the value width and multiplied by (1 - diff);
lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff is one learned number per
layer. Full causal mask, no rotation; the queries are multiplied by a
position-dependent temperature 1 + coef * ln(floor((p + 1) / every) + 1).
Biases on q, k, v.

PooledWindowAttention — queries and keys are divided by their per-head RMS
(no weight), the values ARE the keys as projected (before that norm), scores
pass a tanh soft cap, and the mask is a sliding window plus pooled blocks:
beyond the window a token sees one mean key / mean value per block of `pool`
consecutive positions that lies wholly outside the window, in the same
softmax. The means are kept in the cache's pooled rows (fp32), written by
ops.pool_cache_update when a block's last token is stored.

Either mixer may read ANOTHER layer's cache rows (`owns_cache=False`) with
its own queries. All sizes and constants are constructor arguments.
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.comm import get_comm
from ..parallel.layers import MergedColumnParallelLinear, RowParallelLinear
from .forward_meta import ForwardMeta


class _RowAttentionBase(nn.Module):
    maps = 1

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, norm_eps: float,
                 cache_layer_idx: int, owns_cache: bool, bias: bool,
                 separate_values: bool):
        super().__init__()
        if get_comm().tp_size != 1:
            raise NotImplementedError(
                "row-cache attention keeps all kv heads of a token in one "
                "cache row; tensor parallelism is not wired up for it")
        if heads % kv_heads != 0:
            raise ValueError(f"{heads} query heads do not divide into "
                             f"{kv_heads} key/value heads")
        self.heads, self.kv_heads = heads, kv_heads
        self.dim, self.vdim = dim, value_dim
        self.scale, self.eps = float(scale), float(norm_eps)
        self.cache_layer_idx, self.owns_cache = cache_layer_idx, owns_cache
        sizes = [heads * self.maps * dim]
        if owns_cache:
            sizes.append(kv_heads * self.maps * dim)
            if separate_values:
                sizes.append(kv_heads * value_dim)
        self.in_proj = MergedColumnParallelLinear(hidden_size, sizes, bias=bias)
        self.o_proj = RowParallelLinear(heads * value_dim, hidden_size)

    def _project(self, x: torch.Tensor):
        parts = self.in_proj.split_output(self.in_proj(x))
        return parts + [None] * (3 - len(parts))


class DifferentialAttention(_RowAttentionBase):
    maps = 2

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, diff: float, temp_coef: float,
                 temp_every: int, norm_eps: float, cache_layer_idx: int,
                 owns_cache: bool = True, bias: bool = True):
        super().__init__(hidden_size, heads, kv_heads, dim, value_dim, scale,
                         norm_eps, cache_layer_idx, owns_cache, bias, True)
        self.diff = float(diff)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        for name in ("lq1", "lk1", "lq2", "lk2"):
            setattr(self, name, nn.Parameter(torch.empty(dim), requires_grad=False))
        self._lam: Optional[float] = None

    @property
    def lam(self) -> float:
        if self._lam is None:
            d1 = float((self.lq1.double() * self.lk1.double()).sum())
            d2 = float((self.lq2.double() * self.lk2.double()).sum())
            self._lam = math.exp(d1) - math.exp(d2) + self.diff
        return self._lam

    def invalidate_constants(self) -> None:
        self._lam = None

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        q, k, v = self._project(x)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        q32 = ops.qkv_store(q, k, v, meta.positions, meta.slot_mapping, cache,
                            self.dim, None, self.temp_coef, self.temp_every)
        o = ops.row_attention(
            q32, cache, None, meta.block_tables, meta.token_seq(),
            meta.positions, self.heads, self.kv_heads, 2, self.dim, self.vdim,
            0, 0, self.scale, 0.0, self.lam, self.eps, 1.0 - self.diff,
            x.dtype, max_seq_len=meta.max_seq_len,
            query_bounds=meta.query_bounds(),
        )
        return self.o_proj(o)


class PooledWindowAttention(_RowAttentionBase):
    maps = 1

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, softcap: float, window: int,
                 pool: int, norm_eps: float, cache_layer_idx: int,
                 owns_cache: bool = True):
        if value_dim != dim:
            raise ValueError("the values are the projected keys: value width "
                             f"{value_dim} must equal the key width {dim}")
        super().__init__(hidden_size, heads, kv_heads, dim, value_dim, scale,
                         norm_eps, cache_layer_idx, owns_cache, False, False)
        self.softcap = float(softcap)
        self.window, self.pool = int(window), int(pool)
        if self.window < 1:
            raise ValueError("window size must be at least 1")

    def invalidate_constants(self) -> None:
        pass

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        q, k, _ = self._project(x)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        pool = meta.mla_cache.pool_layer(self.cache_layer_idx) \
            if self.pool > 0 else None
        q32 = ops.qkv_store(q, k, None, meta.positions, meta.slot_mapping,
                            cache, self.dim, self.eps, 0.0, 0)
        if pool is not None and self.owns_cache:
            ops.pool_cache_update(cache, pool, meta.block_tables,
                                  meta.token_seq(), meta.positions,
                                  meta.slot_mapping, self.pool)
        o = ops.row_attention(
            q32, cache, pool, meta.block_tables, meta.token_seq(),
            meta.positions, self.heads, self.kv_heads, 1, self.dim, self.vdim,
            self.window, self.pool, self.scale, self.softcap, 0.0, None, 1.0,
            x.dtype, max_seq_len=meta.max_seq_len,
            query_bounds=meta.query_bounds(),
        )
        return self.o_proj(o)
