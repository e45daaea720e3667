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
    """The newest exact tokens of one layer: one (2, capacity, num_kv_heads, head_dim) tensor, keys in plane 0
    and values in plane 1, filled from the front.  Same interface and token routing as the reference's ring
    (capture.py:21-131): a write that needs room while the ring is full first hands back everything in it."""

    def __init__(self, capacity: int, num_kv_heads: int, head_dim: int, device, dtype: torch.dtype = torch.bfloat16):
        self.capacity = capacity
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.device = device
        self.dtype = dtype
        self._rows = torch.zeros(2, capacity, num_kv_heads, head_dim, device=device, dtype=dtype)
        self._fill = 0          # tokens held
        self._seen = 0          # tokens ever written

    @property
    def size(self) -> int:
        return self._fill

    @property
    def is_full(self) -> bool:
        return self._fill >= self.capacity

    @property
    def total_written(self) -> int:
        return self._seen

    def _take_all(self) -> torch.Tensor:
        held = self._rows[:, : self._fill].clone()
        self._fill = 0
        return held

    def write(self, key: torch.Tensor, value: torch.Tensor, num_tokens: int) -> Optional[KVPair]:
        """Append num_tokens tokens; returns what had to leave the ring on the way (oldest first) as (k, v),
        or None.  The ring is emptied, completely, each time a token arrives while it is full."""
        handed_back = []
        src = 0
        while src < num_tokens:
            if self.is_full:
                handed_back.append(self._take_all())
            n = min(num_tokens - src, self.capacity - self._fill)
            self._rows[0, self._fill: self._fill + n] = key[src: src + n]
            self._rows[1, self._fill: self._fill + n] = value[src: src + n]
            self._fill += n
            src += n
        self._seen += num_tokens
        if not handed_back:
            return None
        out = handed_back[0] if len(handed_back) == 1 else torch.cat(handed_back, dim=1)
        return out[0], out[1]

    def drain(self) -> Optional[KVPair]:
        if self._fill == 0:
            return None
        held = self._take_all()
        return held[0], held[1]

    def peek(self) -> Optional[KVPair]:
        if self._fill == 0:
            return None
        return self._rows[0, : self._fill], self._rows[1, : self._fill]

    def reset(self):
        self._fill = 0
        self._seen = 0


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
