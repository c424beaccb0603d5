"""Paged KV cache tensors, MI355X-first layout.

Layout choice (differs from the reference's vLLM-packed Metal layout,
src/parallax/server/cache/kv_cache.py:84-193): K uses
``[num_blocks, num_kv_heads, block_size, head_dim]`` (token-major rows: a
QK^T A-fragment is 8 consecutive d of one token) and V is stored TRANSPOSED,
``[num_blocks, num_kv_heads, head_dim, block_size]`` (d-major rows: a PV
A-fragment is 8 consecutive tokens of one d) — so BOTH decode-attention MFMA
operands are direct 16 B HBM loads with no LDS transpose staging, and the
prefill kernel stages V^T as plain vectorized row copies. The cache write
pays a per-element transpose scatter once per token instead. 288 GB HBM3E
means block count is sized generously from a memory fraction rather than
packed tightly.

Also here: ``MLAKVCache`` — DeepSeek-style compressed latent cache (kv_lora_rank
latent + rope dims per token, no per-head expansion), and ``LinearStateCache`` —
slot-based conv/recurrent state for hybrid linear-attention stacks.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch


@dataclass
class KVCacheSpec:
    num_layers: int
    num_kv_heads: int
    head_dim: int
    block_size: int
    dtype: torch.dtype = torch.bfloat16
    # sparse-attention indexer keys: one index_dim vector per token per layer
    # (minimax-m3 MSA; dtype follows the main cache but never fp8)
    index_dim: int = 0

    @property
    def bytes_per_token_per_layer(self) -> int:
        return (2 * self.num_kv_heads * self.head_dim + self.index_dim) \
            * self.dtype.itemsize

    def bytes_per_block(self) -> int:
        return self.block_size * self.bytes_per_token_per_layer * self.num_layers


class PagedKVCache:
    """Per-shard paged KV storage: one K and one V tensor per local layer."""

    def __init__(self, spec: KVCacheSpec, num_blocks: int, device: torch.device):
        self.spec = spec
        self.num_blocks = num_blocks
        self.device = device
        # K rows are tokens (QK^T fragments read 8 consecutive d per token);
        # V is stored TRANSPOSED [.., D, block] so PV fragments read 8
        # consecutive tokens per d straight from HBM — the decode/prefill
        # kernels consume V^T without any LDS transpose staging
        k_shape = (num_blocks, spec.num_kv_heads, spec.block_size, spec.head_dim)
        v_shape = (num_blocks, spec.num_kv_heads, spec.head_dim, spec.block_size)
        self.k_caches: List[torch.Tensor] = [
            torch.zeros(k_shape, dtype=spec.dtype, device=device)
            for _ in range(spec.num_layers)
        ]
        self.v_caches: List[torch.Tensor] = [
            torch.zeros(v_shape, dtype=spec.dtype, device=device)
            for _ in range(spec.num_layers)
        ]
        idx_dtype = spec.dtype if spec.dtype != torch.float8_e4m3fn \
            else torch.bfloat16
        # +1 trash block for graph-safe pad-token stores (see MLAKVCache)
        self.index_caches: List[torch.Tensor] = (
            [
                torch.zeros((num_blocks + 1, spec.block_size, spec.index_dim),
                            dtype=idx_dtype, device=device)
                for _ in range(spec.num_layers)
            ]
            if spec.index_dim > 0 else []
        )

    def layer(self, idx: int):
        return self.k_caches[idx], self.v_caches[idx]

    def index_layer(self, idx: int) -> torch.Tensor:
        return self.index_caches[idx]

    @staticmethod
    def num_blocks_for_bytes(spec: KVCacheSpec, budget_bytes: int) -> int:
        return max(0, budget_bytes // spec.bytes_per_block())


class MLAKVCache:
    """Compressed MLA cache: per token one latent vector (kv_lora_rank) plus the
    decoupled rope key (qk_rope_head_dim) — reference dsa_cache.py:8 behavior,
    laid out ``[num_blocks, block_size, kv_lora_rank + rope_dim]`` so decode
    reads one contiguous row per token."""

    def __init__(
        self,
        num_layers: int,
        kv_lora_rank: int,
        rope_dim: int,
        block_size: int,
        num_blocks: int,
        device: torch.device,
        dtype: torch.dtype = torch.bfloat16,
        index_dim: int = 0,
        pool_tokens=None,
    ):
        # kv_lora_rank / rope_dim may be per-layer sequences (stacks whose
        # latent layers differ in size); scalars mean every layer is alike
        ranks = list(kv_lora_rank) if isinstance(kv_lora_rank, (list, tuple)) \
            else [kv_lora_rank] * num_layers
        ropes = list(rope_dim) if isinstance(rope_dim, (list, tuple)) \
            else [rope_dim] * num_layers
        assert len(ranks) == len(ropes) == num_layers
        self.kv_lora_rank = ranks[0] if ranks else 0
        self.rope_dim = ropes[0] if ropes else 0
        self.layer_ranks = ranks
        self.layer_rope_dims = ropes
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.entry_dim = self.kv_lora_rank + self.rope_dim
        self.caches: List[torch.Tensor] = [
            torch.zeros((num_blocks, block_size, r + d), dtype=dtype, device=device)
            for r, d in zip(ranks, ropes)
        ]
        # DSA (DeepSeek-V3.2): one indexer key per token per layer, shared
        # across indexer query heads (reference dsa_cache.py)
        self.index_dim = index_dim
        idx_dtype = dtype if dtype != torch.float8_e4m3fn else torch.bfloat16
        # +1 trash block at the end: graph-safe indexer-cache stores write
        # pad tokens (slot -1) there instead of branching (see
        # ops.reference.store_indexer_cache)
        self.index_caches: List[torch.Tensor] = (
            [
                torch.zeros((num_blocks + 1, block_size, index_dim),
                            dtype=idx_dtype, device=device)
                for _ in range(num_layers)
            ]
            if index_dim > 0
            else []
        )

        # pooled rows: a layer with pool_tokens[i] = P > 0 also keeps the mean
        # of every P consecutive rows of a sequence (fp32, whatever the cache
        # dtype). Pooled block b of a sequence lives in the sequence's page
        # b // per_page at offset b % per_page with per_page = ceil(block_size
        # / P), so the ordinary block table addresses it: block b is complete
        # only once b * P + P tokens exist, and then that page is allocated.
        self.pool_tokens: List[int] = list(pool_tokens) if pool_tokens \
            else [0] * num_layers
        assert len(self.pool_tokens) == num_layers
        self.pools: List[Optional[torch.Tensor]] = [
            torch.zeros((num_blocks, self.pool_rows_per_block(block_size, p), r + d),
                        dtype=torch.float32, device=device) if p > 0 else None
            for p, r, d in zip(self.pool_tokens, ranks, ropes)
        ]

    @staticmethod
    def pool_rows_per_block(block_size: int, pool_tokens: int) -> int:
        return (block_size + pool_tokens - 1) // pool_tokens

    def layer(self, idx: int) -> torch.Tensor:
        return self.caches[idx]

    def pool_layer(self, idx: int) -> Optional[torch.Tensor]:
        return self.pools[idx]

    def index_layer(self, idx: int) -> torch.Tensor:
        return self.index_caches[idx]

    @staticmethod
    def bytes_per_block(
        num_layers: int, kv_lora_rank, rope_dim, block_size: int,
        dtype: torch.dtype = torch.bfloat16, index_dim: int = 0,
        pool_tokens=None,
    ) -> int:
        if isinstance(kv_lora_rank, (list, tuple)):
            width = sum(kv_lora_rank) + sum(rope_dim) + index_dim * num_layers
            pooled = sum(
                MLAKVCache.pool_rows_per_block(block_size, p) * (r + d) * 4
                for p, r, d in zip(pool_tokens or [], kv_lora_rank, rope_dim)
                if p > 0
            )
            return block_size * width * dtype.itemsize + pooled
        return num_layers * block_size * (kv_lora_rank + rope_dim + index_dim) * dtype.itemsize


class LinearStateCache:
    """Slot-based state for linear-attention / SSM hybrid layers (reference
    cache/linear_cache.py): per slot a conv window state and a recurrent state,
    with snapshot/restore for prefix reuse."""

    def __init__(
        self,
        num_layers: int,
        conv_state_shape: tuple,
        recurrent_state_shape: tuple,
        num_slots: int,
        device: torch.device,
        dtype: torch.dtype = torch.bfloat16,
    ):
        self.num_slots = num_slots
        # a list of shapes = one per layer (layers of unequal size)
        conv_shapes = list(conv_state_shape) \
            if conv_state_shape and isinstance(conv_state_shape[0], (list, tuple)) \
            else [conv_state_shape] * num_layers
        rec_shapes = list(recurrent_state_shape) \
            if recurrent_state_shape and isinstance(recurrent_state_shape[0], (list, tuple)) \
            else [recurrent_state_shape] * num_layers
        assert len(conv_shapes) == len(rec_shapes) == num_layers
        self.conv_states: List[torch.Tensor] = [
            torch.zeros((num_slots, *shape), dtype=dtype, device=device)
            for shape in conv_shapes
        ]
        self.recurrent_states: List[torch.Tensor] = [
            torch.zeros((num_slots, *shape), dtype=torch.float32, device=device)
            for shape in rec_shapes
        ]

    def reset_slot(self, slot: int) -> None:
        for c in self.conv_states:
            c[slot].zero_()
        for r in self.recurrent_states:
            r[slot].zero_()

    def snapshot(self, slot: int):
        return (
            [c[slot].clone() for c in self.conv_states],
            [r[slot].clone() for r in self.recurrent_states],
        )

    def restore(self, slot: int, snap) -> None:
        conv, rec = snap
        for dst, src in zip(self.conv_states, conv):
            dst[slot].copy_(src)
        for dst, src in zip(self.recurrent_states, rec):
            dst[slot].copy_(src)


def build_block_table_tensor(
    block_tables: List[List[int]], device: torch.device, pad: int = 0
) -> torch.Tensor:
    """Pad ragged per-request block tables into an int32 [batch, max_blocks] tensor."""
    max_len = max((len(bt) for bt in block_tables), default=1)
    max_len = max(max_len, 1)
    out = torch.full((len(block_tables), max_len), pad, dtype=torch.int32)
    for i, bt in enumerate(block_tables):
        if bt:
            out[i, : len(bt)] = torch.tensor(bt, dtype=torch.int32)
    return out.to(device)


def slot_mapping_for_positions(
    block_table: List[int], start_pos: int, num_tokens: int, block_size: int
) -> List[int]:
    """Flat cache-slot index (block_id * block_size + offset) for each new token."""
    out = []
    for pos in range(start_pos, start_pos + num_tokens):
        out.append(block_table[pos // block_size] * block_size + pos % block_size)
    return out
