"""Write-side policy: exact ring of recent tokens + when to compress.

Mirrors turboquant/capture.py of the reference (`RingBuffer`, capture.py:21-131;
`KVCaptureEngine`, capture.py:134-240) with the same methods and the same token
routing: prefill compresses everything but the newest `ring_capacity` tokens,
decode tokens land in the ring, and a write that finds the ring full first
drains the whole ring into the compressed store.  This is host bookkeeping
around two device tensors; the quantisation itself happens in
`CompressedKVStore.append_chunk`.
"""

from __future__ import annotations

from typing import TYPE_CHECKING, Optional, Tuple

import torch

from .paged import PAGE_TOKENS

if TYPE_CHECKING:
    from .store import CompressedKVStore

KVPair = Tuple[torch.Tensor, torch.Tensor]


class RingBuffer:
    """`capacity` exact tokens, (capacity, num_kv_heads, head_dim) per tensor."""

    __slots__ = ("capacity", "num_kv_heads", "head_dim", "device", "dtype", "_k", "_v", "_pos", "_total_written")

    def __init__(self, capacity: int, num_kv_heads: int, head_dim: int, device, dtype: torch.dtype = torch.bfloat16):
        self.capacity = capacity
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.device = device
        self.dtype = dtype
        self._k = torch.zeros(capacity, num_kv_heads, head_dim, device=device, dtype=dtype)
        self._v = torch.zeros(capacity, num_kv_heads, head_dim, device=device, dtype=dtype)
        self._pos = 0
        self._total_written = 0

    @property
    def size(self) -> int:
        return self._pos

    @property
    def is_full(self) -> bool:
        return self._pos >= self.capacity

    @property
    def total_written(self) -> int:
        return self._total_written

    def write(self, key: torch.Tensor, value: torch.Tensor, num_tokens: int) -> Optional[KVPair]:
        """Append num_tokens tokens.  Whenever the ring is full at the moment a
        token needs room, everything in it is drained first; the drained tokens
        come back (oldest first) as (k, v), or None if nothing was drained."""
        spilled_k, spilled_v = [], []
        done = 0
        while done < num_tokens:
            if self._pos >= self.capacity:
                spilled_k.append(self._k[: self._pos].clone())
                spilled_v.append(self._v[: self._pos].clone())
                self._pos = 0
            take = min(num_tokens - done, self.capacity - self._pos)
            self._k[self._pos: self._pos + take] = key[done: done + take]
            self._v[self._pos: self._pos + take] = value[done: done + take]
            self._pos += take
            done += take
        self._total_written += num_tokens
        if not spilled_k:
            return None
        return torch.cat(spilled_k, dim=0), torch.cat(spilled_v, dim=0)

    def drain(self) -> Optional[KVPair]:
        if self._pos == 0:
            return None
        pair = (self._k[: self._pos].clone(), self._v[: self._pos].clone())
        self._pos = 0
        return pair

    def peek(self) -> Optional[KVPair]:
        if self._pos == 0:
            return None
        return self._k[: self._pos], self._v[: self._pos]

    def reset(self):
        self._pos = 0
        self._total_written = 0


class KVCaptureEngine:
    """Routes K/V of one layer into the ring and the compressed store."""

    def __init__(self, store: "CompressedKVStore", ring_capacity: int = 128, device=None,
                 dtype: torch.dtype = torch.bfloat16):
        self.store = store
        self.ring = RingBuffer(capacity=ring_capacity, num_kv_heads=store.num_kv_heads, head_dim=store.head_dim,
                               device=device or store.device, dtype=dtype)
        self._prefill_done = False

    @property
    def total_compressed_tokens(self) -> int:
        return self.store.num_tokens

    @property
    def total_buffered_tokens(self) -> int:
        return self.ring.size

    @property
    def total_tokens(self) -> int:
        return self.total_compressed_tokens + self.total_buffered_tokens

    def ingest_prefill(self, key: torch.Tensor, value: torch.Tensor, num_tokens: int):
        """key/value (num_tokens, num_kv_heads, head_dim).  The newest
        ring_capacity tokens stay exact; older ones are compressed in one chunk.
        As in the reference, whatever the ring spills while taking the tail is
        not forwarded to the store (capture.py:176,180)."""
        cap = self.ring.capacity
        if num_tokens <= cap:
            self.ring.write(key[:num_tokens], value[:num_tokens], num_tokens)
        else:
            head = num_tokens - cap
            self.store.append_chunk(key[:head], value[:head])
            self.ring.write(key[head:num_tokens], value[head:num_tokens], cap)
        self._prefill_done = True

    def ingest_prefill_from_paged_cache(self, kv_cache_tensor: torch.Tensor, num_tokens: int,
                                        block_table: torch.Tensor, block_size: int):
        """Prefill from a paged exact cache (2, num_blocks, block_size, heads, dim)
        through `block_table` (logical -> physical block).  With 16-token blocks and an empty
        store the part to compress is quantised in place (gather and quantisation in one
        kernel pass); only the ring's tail is gathered."""
        n_blocks = (num_tokens + block_size - 1) // block_size
        phys = block_table[:n_blocks].to(device=kv_cache_tensor.device, dtype=torch.long)
        cap = self.ring.capacity
        in_place = (block_size == PAGE_TOKENS and num_tokens > cap and self.store.num_tokens == 0 and
                    kv_cache_tensor.is_cuda and kv_cache_tensor.dim() == 5 and kv_cache_tensor[0].stride(-1) == 1 and
                    kv_cache_tensor[0].stride() == kv_cache_tensor[1].stride())
        if not in_place:
            k = kv_cache_tensor[0].index_select(0, phys).reshape(n_blocks * block_size, *kv_cache_tensor.shape[3:])
            v = kv_cache_tensor[1].index_select(0, phys).reshape(n_blocks * block_size, *kv_cache_tensor.shape[3:])
            self.ingest_prefill(k[:num_tokens], v[:num_tokens], num_tokens)
            return
        head = num_tokens - cap
        self.store.append_chunk_from_blocks(kv_cache_tensor[0], kv_cache_tensor[1], phys, head)
        pos = torch.arange(head, num_tokens, device=kv_cache_tensor.device)
        blk = phys[pos // block_size]
        self.ring.write(kv_cache_tensor[0][blk, pos % block_size], kv_cache_tensor[1][blk, pos % block_size], cap)
        self._prefill_done = True

    def ingest_decode(self, key: torch.Tensor, value: torch.Tensor, num_tokens: int):
        """Decode tokens go to the ring; what the ring drains is compressed."""
        spilled = self.ring.write(key[:num_tokens], value[:num_tokens], num_tokens)
        if spilled is not None:
            self.store.append_chunk(*spilled)

    def flush(self):
        """Compress whatever the ring holds."""
        pair = self.ring.drain()
        if pair is not None:
            self.store.append_chunk(*pair)

    def reset(self):
        self.ring.reset()
        self.store.reset()
        self._prefill_done = False
