"""Compressed KV store: owns the quantised history of one sequence of one layer.

Mirrors turboquant/store.py of the reference (`FlatCache`, `CompressedKVStore`
with `quantizer`, `num_tokens`, `num_chunks`, `append_chunk`, `get_flat_cache`,
`memory_bytes`, `reset`; store.py:19-134).  Where the reference appends chunk
tensors to python lists and concatenates them on every read (store.py:92-114),
this store writes each chunk straight into a paged pool with the fused quantise
kernel; the flat (H, N, ...) tensors of the reference are produced on demand by
a gather kernel and cached until the next write.
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from .kv_cache import ValueQuantized
from .paged import PAGE_TOKENS, PagedKVPool
from .quantizer import ProdQuantized, TurboQuantProd


class FlatCache(NamedTuple):
    """Flat view of the compressed history, tensors shaped (num_kv_heads, total_tokens, ...)."""
    prod_q: ProdQuantized
    value_q: ValueQuantized
    num_tokens: int


class CompressedKVStore:
    _INITIAL_PAGES = 64

    def __init__(self, head_dim: int, num_kv_heads: int, key_bits: int = 3, value_bits: int = 2,
                 value_group_size: int = 32, device=None, layer_idx: int = 0):
        self.head_dim = head_dim
        self.num_kv_heads = num_kv_heads
        self.key_bits = key_bits
        self.value_bits = value_bits
        self.value_group_size = min(value_group_size, head_dim)
        self.device = device or torch.device("cuda")
        self.layer_idx = layer_idx
        # per-layer seed, as the reference draws it (store.py:52-57)
        self.quantizer = TurboQuantProd(dim=head_dim, bits=key_bits, device=self.device, seed=42 + layer_idx * 7)
        self._chunk_lengths: list[int] = []
        self._pool: Optional[PagedKVPool] = None
        self._block_table: Optional[torch.Tensor] = None
        self._flat: Optional[FlatCache] = None

    # ---- bookkeeping ---------------------------------------------------------------
    @property
    def num_tokens(self) -> int:
        return sum(self._chunk_lengths)

    @property
    def num_chunks(self) -> int:
        return len(self._chunk_lengths)

    @property
    def pool(self) -> Optional[PagedKVPool]:
        return self._pool

    @property
    def block_table(self) -> Optional[torch.Tensor]:
        """(1, num_pages) int32: this sequence's pages, in order."""
        return self._block_table

    def ensure_pool(self, dtype: torch.dtype, min_tokens: int = 0) -> PagedKVPool:
        need = max(self._INITIAL_PAGES, (min_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS)
        if self._pool is None:
            self._pool = PagedKVPool(self.quantizer, self.num_kv_heads, need, self.value_bits, self.value_group_size,
                                     dtype=dtype, device=self.device)
        elif need > self._pool.num_pages:
            self._pool.grow(max(need, 2 * self._pool.num_pages))
        if self._block_table is None or self._block_table.shape[1] != self._pool.num_pages:
            self._block_table = torch.arange(self._pool.num_pages, dtype=torch.int32, device=self._pool.device)[None, :]
        return self._pool

    # ---- write -----------------------------------------------------------------------
    def append_chunk(self, key: torch.Tensor, value: torch.Tensor):
        """Quantise and store key/value (chunk_len, num_kv_heads, head_dim)."""
        chunk_len = key.shape[0]
        if chunk_len == 0:
            return
        start = self.num_tokens
        pool = self.ensure_pool(key.dtype, start + chunk_len)
        if key.dtype != pool.dtype:
            raise TypeError(f"store holds {pool.dtype} pages; got a {key.dtype} chunk")
        start_pos = torch.tensor([start], dtype=torch.int32, device=pool.device)
        pool.append(key.unsqueeze(0), value.unsqueeze(0), self._block_table, start_pos)
        self._chunk_lengths.append(chunk_len)
        self._flat = None

    def append_chunk_from_blocks(self, key_cache: torch.Tensor, value_cache: torch.Tensor, src_blocks: torch.Tensor,
                                 chunk_len: int):
        """Quantise the first chunk_len tokens of a sequence straight out of a paged exact cache
        ((num_blocks, 16, H, d) tensors, the sequence's blocks in src_blocks) into an EMPTY store:
        the gather and the quantisation are one pass over the cache."""
        if chunk_len == 0:
            return
        if self.num_tokens != 0:
            raise RuntimeError("append_chunk_from_blocks fills an empty store (source and store positions coincide)")
        pool = self.ensure_pool(key_cache.dtype, chunk_len)
        if key_cache.dtype != pool.dtype:
            raise TypeError(f"store holds {pool.dtype} pages; got a {key_cache.dtype} cache")
        src = src_blocks.to(device=pool.device, dtype=torch.int32).reshape(1, -1).contiguous()
        pool.append_from_blocks(key_cache, value_cache, src, self._block_table,
                                torch.tensor([chunk_len], dtype=torch.int32), max_tokens=chunk_len)
        self._chunk_lengths.append(chunk_len)
        self._flat = None

    # ---- read ------------------------------------------------------------------------
    def get_flat_cache(self) -> Optional[FlatCache]:
        """The reference's flat tensors; None while the store is empty."""
        if not self._chunk_lengths:
            return None
        if self._flat is None:
            n = self.num_tokens
            idx, signs, norms, rnorms, v_data, v_scales, v_zeros = self._pool.export_flat(self._block_table[0], n)
            self._flat = FlatCache(
                prod_q=ProdQuantized(mse_indices=idx, qjl_signs=signs, residual_norms=rnorms, norms=norms,
                                     mse_bits=self.key_bits - 1),
                value_q=ValueQuantized(data=v_data, scales=v_scales, zeros=v_zeros, bits=self.value_bits),
                num_tokens=n)
        return self._flat

    def memory_bytes(self) -> int:
        """Compressed bytes with norms, residual norms, scales and zeros counted
        at 2 bytes each (the reference's accounting, store.py:116-128)."""
        mb = self.key_bits - 1
        stored = 1 if mb == 1 else (2 if mb == 2 else (4 if mb <= 4 else 8))
        per_byte = 8 // stored
        d = self.head_dim
        key_bytes = (d + per_byte - 1) // per_byte + (d + 7) // 8 + 2 + 2
        val_bytes = d * self.value_bits // 8 + 2 * 2 * (d // self.value_group_size)
        return self.num_tokens * self.num_kv_heads * (key_bytes + val_bytes)

    def reset(self):
        self._chunk_lengths.clear()
        self._flat = None
