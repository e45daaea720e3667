"""Paged compressed KV pool for batches of sequences (new design).

The reference keeps one python list of chunk tensors per layer and therefore
one sequence (store.py:59-63; integration/vllm.py:139-145).  This module is the
batch-aware store underneath: a pool of 16-token pages per layer, block tables
and sequence lengths, written by the fused quantise kernel and read by the fused
decode-attention kernel.  `CompressedKVStore` (store.py mirror) is a
single-sequence view over it.
"""

from __future__ import annotations

import ctypes as C
import math
from typing import Optional

import torch

from . import _ffi
from .quantizer import TurboQuantProd

PAGE_TOKENS = _ffi.TQ_PAGE_TOKENS


class PagedKVPool:
    """(num_pages, num_kv_heads, page_bytes) uint8 pool + its geometry."""

    def __init__(self, quantizer: TurboQuantProd, num_kv_heads: int, num_pages: int, value_bits: int = 2,
                 value_group_size: int = 32, dtype: torch.dtype = torch.bfloat16, device=None):
        self.quantizer = quantizer
        self.head_dim = quantizer.dim
        self.num_kv_heads = num_kv_heads
        self.value_bits = value_bits
        self.value_group_size = min(value_group_size, self.head_dim)
        self.dtype = dtype
        self.device = torch.device(device) if device is not None else quantizer.S.device
        if self.device.type != "cuda":
            raise RuntimeError("PagedKVPool needs a GPU device: the TurboQuant kernels have no CPU path")
        self.layout = _ffi.make_page_layout(self.head_dim, quantizer.bits - 1, value_bits, self.value_group_size, dtype)
        self.num_pages = int(num_pages)
        self.data = torch.zeros(self.num_pages, num_kv_heads, self.layout.page_bytes, dtype=torch.uint8,
                                device=self.device)

    @property
    def page_bytes(self) -> int:
        return self.layout.page_bytes

    def grow(self, num_pages: int):
        """Enlarge the pool, keeping existing pages."""
        if num_pages <= self.num_pages:
            return
        bigger = torch.zeros(num_pages, self.num_kv_heads, self.layout.page_bytes, dtype=torch.uint8, device=self.device)
        bigger[: self.num_pages] = self.data
        self.data, self.num_pages = bigger, int(num_pages)

    # ---- write ------------------------------------------------------------------
    def append(self, key: torch.Tensor, value: torch.Tensor, block_table: torch.Tensor,
               start_pos: Optional[torch.Tensor] = None):
        """Quantise key/value (B, T, H, d) and store token t of sequence b at
        logical position start_pos[b] + t through block_table (B, max_pages) int32."""
        _ffi.require_gpu(key, "key")
        if key.dim() != 4 or key.shape != value.shape:
            raise ValueError("key and value must both be (B, T, H, d)")
        B, T, H, d = key.shape
        if H != self.num_kv_heads or d != self.head_dim:
            raise ValueError(f"expected (B, T, {self.num_kv_heads}, {self.head_dim}), got {tuple(key.shape)}")
        if key.dtype != self.dtype or value.dtype != self.dtype:
            raise TypeError(f"pool was laid out for {self.dtype}")
        if key.stride(-1) != 1 or value.stride(-1) != 1 or key.stride() != value.stride():
            key, value = key.contiguous(), value.contiguous()
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.shape[0] != B:
            raise ValueError("block_table must be int32 (B, max_pages)")
        block_table = block_table.contiguous()
        if start_pos is not None:
            start_pos = start_pos.to(device=self.device, dtype=torch.int32).contiguous()
        ly = self.quantizer._layer()
        with _ffi.on_device(self.device):
            _ffi.check(_ffi.lib().tq_append_kv_paged(
                key.data_ptr(), value.data_ptr(), _ffi.dtype_tag(self.dtype), B, T, H, key.stride(0), key.stride(1),
                key.stride(2), _ffi.ptr(start_pos), block_table.data_ptr(), block_table.shape[1], C.byref(ly),
                C.byref(self.layout), self.data.data_ptr(), self.num_pages, _ffi.stream_ptr(self.device)),
                "tq_append_kv_paged")

    def append_from_blocks(self, key_cache: torch.Tensor, value_cache: torch.Tensor, src_table: torch.Tensor,
                           block_table: torch.Tensor, run_len: torch.Tensor, start_pos: Optional[torch.Tensor] = None,
                           max_tokens: Optional[int] = None):
        """Quantise tokens that sit in a paged exact cache, without gathering them first.
        key_cache / value_cache (num_blocks, 16, H, d); sequence b's positions start_pos[b] ..
        start_pos[b] + run_len[b] - 1 are read through src_table (B, n) (position p -> block
        src_table[b, p // 16], slot p % 16) and written through block_table (B, max_pages)."""
        _ffi.require_gpu(key_cache, "key_cache")
        if key_cache.dim() != 4 or key_cache.shape != value_cache.shape or key_cache.shape[1] != PAGE_TOKENS:
            raise ValueError("key_cache and value_cache must both be (num_blocks, 16, H, d)")
        if key_cache.shape[2] != self.num_kv_heads or key_cache.shape[3] != self.head_dim:
            raise ValueError(f"expected (num_blocks, 16, {self.num_kv_heads}, {self.head_dim})")
        if key_cache.dtype != self.dtype or value_cache.dtype != self.dtype:
            raise TypeError(f"pool was laid out for {self.dtype}")
        if key_cache.stride(-1) != 1 or key_cache.stride() != value_cache.stride():
            raise ValueError("key_cache and value_cache need the same strides and a contiguous last dimension")
        B = src_table.shape[0]
        for t in (src_table, block_table):
            if t.dtype != torch.int32 or t.dim() != 2 or t.shape[0] != B:
                raise ValueError("src_table and block_table must be int32 (B, n)")
        src_table, block_table = src_table.contiguous(), block_table.contiguous()
        run_len = run_len.to(device=self.device, dtype=torch.int32).contiguous()
        if start_pos is not None:
            start_pos = start_pos.to(device=self.device, dtype=torch.int32).contiguous()
        if max_tokens is None:
            max_tokens = int(run_len.max())
        ly = self.quantizer._layer()
        with _ffi.on_device(self.device):
            _ffi.check(_ffi.lib().tq_append_kv_from_blocks(
                key_cache.data_ptr(), value_cache.data_ptr(), _ffi.dtype_tag(self.dtype), B, int(max_tokens),
                self.num_kv_heads, key_cache.stride(0), key_cache.stride(1), key_cache.stride(2), src_table.data_ptr(),
                src_table.shape[1], _ffi.ptr(start_pos), run_len.data_ptr(), block_table.data_ptr(),
                block_table.shape[1], C.byref(ly), C.byref(self.layout), self.data.data_ptr(), self.num_pages,
                _ffi.stream_ptr(self.device)), "tq_append_kv_from_blocks")

    def append_ragged(self, key: torch.Tensor, value: torch.Tensor, row0: torch.Tensor, run_len: torch.Tensor,
                      start_pos: torch.Tensor, block_table: torch.Tensor, max_run: int):
        """Quantise a ragged batch of runs in one call: key / value (rows, H, d) hold the rows of all
        sequences one after another; sequence b owns rows row0[b] .. row0[b] + run_len[b] - 1, which become
        its tokens start_pos[b] .. in the pages of block_table[b].  row0 / run_len / start_pos are (B,) device
        tensors (nothing is read back to the host); max_run bounds every run_len."""
        _ffi.require_gpu(key, "key")
        if key.dim() != 3 or key.shape != value.shape or tuple(key.shape[1:]) != (self.num_kv_heads, self.head_dim):
            raise ValueError(f"expected key and value of shape (rows, {self.num_kv_heads}, {self.head_dim})")
        if key.dtype != self.dtype or value.dtype != self.dtype:
            raise TypeError(f"pool was laid out for {self.dtype}")
        if key.stride(-1) != 1 or key.stride() != value.stride():
            key, value = key.contiguous(), value.contiguous()
        if block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise ValueError("block_table must be int32 (B, max_pages)")
        B = block_table.shape[0]
        block_table = block_table.contiguous()
        arrs = [t.to(device=self.device, dtype=torch.int32).contiguous() for t in (row0, run_len, start_pos)]
        if any(t.shape != (B,) for t in arrs):
            raise ValueError("row0, run_len and start_pos must have one entry per row of block_table")
        ly = self.quantizer._layer()
        with _ffi.on_device(self.device):
            _ffi.check(_ffi.lib().tq_append_kv_ragged(
                key.data_ptr(), value.data_ptr(), _ffi.dtype_tag(self.dtype), B, int(max_run), self.num_kv_heads,
                key.stride(0), key.stride(1), arrs[0].data_ptr(), arrs[1].data_ptr(), arrs[2].data_ptr(),
                block_table.data_ptr(), block_table.shape[1], C.byref(ly), C.byref(self.layout),
                self.data.data_ptr(), self.num_pages, _ffi.stream_ptr(self.device)), "tq_append_kv_ragged")

    # ---- read -------------------------------------------------------------------
    def export_flat(self, block_table_row: torch.Tensor, n_tok: int):
        """Gather one sequence's pages into the reference's flat tensors
        (H, n_tok, ...): idx, signs, norms, rnorms, v_data, v_scales, v_zeros."""
        H, d, dev = self.num_kv_heads, self.head_dim, self.device
        mb = self.quantizer.bits - 1
        eff = 1 if mb == 1 else (2 if mb == 2 else 4)
        ng = d // self.value_group_size
        idx = torch.empty(H, n_tok, d * eff // 8, dtype=torch.uint8, device=dev)
        signs = torch.empty(H, n_tok, d // 8, dtype=torch.uint8, device=dev)
        norms = torch.empty(H, n_tok, dtype=self.dtype, device=dev)
        rnorms = torch.empty(H, n_tok, dtype=torch.float32, device=dev)
        v_data = torch.empty(H, n_tok, d * self.value_bits // 8, dtype=torch.uint8, device=dev)
        v_scales = torch.empty(H, n_tok, ng, dtype=self.dtype, device=dev)
        v_zeros = torch.empty(H, n_tok, ng, dtype=self.dtype, device=dev)
        bt = block_table_row.to(device=dev, dtype=torch.int32).contiguous()
        with torch.cuda.device(dev):
            _ffi.check(_ffi.lib().tq_pool_export(
                self.data.data_ptr(), self.num_pages, H, bt.data_ptr(), n_tok, C.byref(self.layout), idx.data_ptr(),
                signs.data_ptr(), norms.data_ptr(), rnorms.data_ptr(), v_data.data_ptr(), v_scales.data_ptr(),
                v_zeros.data_ptr(), _ffi.stream_ptr(dev)), "tq_pool_export")
        return idx, signs, norms, rnorms, v_data, v_scales, v_zeros

    def page_kernel(self) -> int:
        """Which page kernel the library runs for this pool's layer (tq_decode_page_kernel): 0 the general
        vector-ALU kernel, 1 the matrix-core kernel of head_dim 64 / 128 / 256, 2 the matrix-core kernel of the
        head sizes above 256."""
        ly = self.quantizer._layer()
        rc = _ffi.lib().tq_decode_page_kernel(C.byref(ly), C.byref(self.layout))
        if rc < 0:
            _ffi.check(rc, "tq_decode_page_kernel")
        return int(rc)

    def _matrix_core_shape(self, Hq: Optional[int]) -> bool:
        """Whether decode runs on the matrix-core page kernel (head_dim 64 / 128 / 256, 16-bit pools, up to 4-bit
        keys - 5-bit at head_dim 128 -, at most 128 query heads per KV head); only the split heuristic depends on it."""
        if self.head_dim not in (64, 128, 256) or self.dtype not in (torch.bfloat16, torch.float16):
            return False
        if self.quantizer.bits - 1 > 4 or self.value_bits not in (2, 4, 8) or self.value_group_size not in (32, 64):
            return False
        if self.value_bits == 8 and (self.quantizer.bits != 3 or self.value_group_size != 32):
            return False
        if self.quantizer.bits == 5 and (self.head_dim != 128 or self.value_group_size != 32):
            return False                                     # 5-bit keys: head_dim 128 only
        if Hq is None:
            return True
        return max(1, Hq // self.num_kv_heads) <= 128       # (more than 8 heads per KV head: groups of at most 8)

    def default_splits(self, B: int, max_len: int, Hq: Optional[int] = None) -> int:
        """Split count of the page-streaming kernel.  Matrix-core kernel: its workgroups (4 wavefronts,
        one per SIMD, each walking 64-token blocks) should number about two per CU (256 CUs) while every
        wavefront still gets several blocks, because each wavefront first builds its query operands.
        General kernel: it hides its memory latency by occupancy, so about eight workgroups per CU, each
        with at least one 256-token chunk."""
        pairs = max(1, B * self.num_kv_heads)
        if self.head_dim > 256 and self.page_kernel() == 2:
            # head sizes above 256: one workgroup per compute unit, a block of 32 tokens at a time; each workgroup
            # first packs its query operands, so it should have at least 16 blocks
            if Hq is not None:
                pairs *= (Hq // self.num_kv_heads + 7) // 8
            blocks = max(1, (max_len + 31) // 32)
            return int(max(1, min(max(1, 256 // pairs), max(1, blocks // 16), 512)))
        if not self._matrix_core_shape(Hq):
            chunks = max(1, (max_len + 255) // 256)
            return int(max(1, min(2048 // pairs, chunks, 512)))
        blocks = max(1, (max_len + 63) // 64)
        # (more than 8 query heads per KV head: ceil(G / 8) workgroups per split read a KV head's pages;
        # 16 x 8192 with 128 q / 8 KV heads: 57.0 us with 4 splits, 48.3 us with 2)
        if Hq is not None:
            pairs *= (Hq // self.num_kv_heads + 7) // 8
        want = max(1, 512 // pairs)
        longest = max(1, blocks // 16)          # keep >= 4 blocks per wavefront
        return int(max(1, min(want, longest, 512)))

    def workspace(self, B: int, Hq: int, n_split: int) -> torch.Tensor:
        nbytes = _ffi.lib().tq_decode_workspace_bytes(B, Hq, self.head_dim, n_split)
        return torch.empty(nbytes // 4, dtype=torch.float32, device=self.device)

    def decode_attention(self, query: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor,
                         scale: Optional[float] = None, recent_k: Optional[torch.Tensor] = None,
                         recent_v: Optional[torch.Tensor] = None, recent_len: Optional[torch.Tensor] = None,
                         n_split: Optional[int] = None, workspace: Optional[torch.Tensor] = None,
                         out: Optional[torch.Tensor] = None, max_len: Optional[int] = None,
                         stages: int = 7, static_scratch: bool = False) -> torch.Tensor:
        """softmax(scale * [scores_hist ; q k_recent^T]) [v_hist ; v_recent] for one
        query token per sequence.  query (B, Hq, d);
        block_table (B, max_pages) or (max_pages,) shared; seq_lens (B,) int32;
        recent_k / recent_v (B, R, H, d) exact tokens, recent_len (B,) valid rows.
        `stages` (bit 0 query rotation, bit 1 page kernel, bit 2 merge) exists for
        timing the stages apart; 7 runs the whole thing.  `static_scratch` runs the library's entry
        point that allocates nothing (tq_decode_attn_paged_noalloc): no workspace tensor, the partials live
        in a fixed device array inside the library (16 MiB; larger calls raise), shared by all calls on
        this GPU - pass `out` as well and the call touches no allocator at all."""
        _ffi.require_gpu(query, "query")
        B, Hq, d = query.shape
        if d != self.head_dim or Hq % self.num_kv_heads:
            raise ValueError(f"Incompatible GQA shapes: Q={Hq}, H_kv={self.num_kv_heads}, d={d}")
        query = query.contiguous()
        if scale is None:
            scale = 1.0 / math.sqrt(d)
        bt = block_table.contiguous()
        bt_stride = -bt.shape[0] if bt.dim() == 1 else bt.shape[1]      # negative: one shared row of that length
        seq_lens = seq_lens.to(device=self.device, dtype=torch.int32).contiguous()
        if n_split is None:
            if max_len is None:
                max_len = (bt.shape[-1]) * PAGE_TOKENS
            n_split = self.default_splits(B, max_len, Hq)
        if static_scratch:
            if workspace is not None or stages != 7:
                raise ValueError("static_scratch takes no workspace and runs all stages")
        elif workspace is None:
            workspace = self.workspace(B, Hq, n_split)
        if out is None:
            out = torch.empty_like(query)
        rk_ptr = rv_ptr = rl_ptr = None
        rows = 0
        rs = (0, 0, 0)
        if recent_k is not None and recent_k.shape[1] > 0:
            if recent_k.dtype != query.dtype or recent_v.dtype != query.dtype:
                raise TypeError("recent_k / recent_v must have the query's dtype")
            if recent_k.stride(-1) != 1 or recent_k.stride() != recent_v.stride():
                recent_k, recent_v = recent_k.contiguous(), recent_v.contiguous()
            rows = recent_k.shape[1]
            rs = (recent_k.stride(0), recent_k.stride(1), recent_k.stride(2))
            rk_ptr, rv_ptr = recent_k.data_ptr(), recent_v.data_ptr()
            if recent_len is not None:
                recent_len = recent_len.to(device=self.device, dtype=torch.int32).contiguous()
                rl_ptr = recent_len.data_ptr()
        ly = self.quantizer._layer()
        if static_scratch:
            with _ffi.on_device(self.device):
                _ffi.check(_ffi.lib().tq_decode_attn_paged_noalloc(
                    query.data_ptr(), _ffi.dtype_tag(query.dtype), B, Hq, self.num_kv_heads, self.data.data_ptr(),
                    self.num_pages, bt.data_ptr(), bt_stride, seq_lens.data_ptr(), float(scale), C.byref(ly),
                    C.byref(self.layout), rk_ptr, rv_ptr, rows, rs[0], rs[1], rs[2], rl_ptr, out.data_ptr(),
                    n_split, _ffi.stream_ptr(self.device)), "tq_decode_attn_paged_noalloc")
            return out
        with _ffi.on_device(self.device):
            _ffi.check(_ffi.lib().tq_decode_attn_paged_stages(
                query.data_ptr(), _ffi.dtype_tag(query.dtype), B, Hq, self.num_kv_heads, self.data.data_ptr(),
                self.num_pages, bt.data_ptr(), bt_stride, seq_lens.data_ptr(), float(scale), C.byref(ly),
                C.byref(self.layout), rk_ptr, rv_ptr, rows, rs[0], rs[1], rs[2], rl_ptr, out.data_ptr(),
                workspace.data_ptr(), n_split, stages, _ffi.stream_ptr(self.device)), "tq_decode_attn_paged")
        return out

    @staticmethod
    def ring_cache_ok(key_cache: torch.Tensor, value_cache: torch.Tensor) -> bool:
        """Whether decode_attention_ring can read this paged exact cache in place: (blocks, 16, H, d) with
        contiguous channels, equal strides, and (16-bit types) even strides and 4-byte aligned bases."""
        if key_cache.dim() != 4 or key_cache.shape != value_cache.shape or key_cache.shape[1] != PAGE_TOKENS:
            return False
        if key_cache.stride() != value_cache.stride() or key_cache.stride(-1) != 1 or key_cache.dtype != value_cache.dtype:
            return False
        if key_cache.element_size() == 2:
            if any(st % 2 for st in key_cache.stride()[:3]) or key_cache.data_ptr() % 4 or value_cache.data_ptr() % 4:
                return False
        return True

    def decode_attention_ring(self, query: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor,
                              key_cache: torch.Tensor, value_cache: torch.Tensor, ring_rows: int,
                              scale: Optional[float] = None, n_split: Optional[int] = None,
                              workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                              max_len: Optional[int] = None) -> torch.Tensor:
        """Hybrid attention of one query token per sequence (score.py:99-111) with the exact tokens read in
        place: the newest min(seq_lens[b], ring_rows) tokens of sequence b come from the engine's paged exact
        cache key_cache / value_cache (blocks, 16, H, d) through `block_table`, the tokens before them from
        this pool's pages of the same numbers.  seq_lens counts all tokens.  Same result as decode_attention
        with those rows gathered into recent_k / recent_v."""
        _ffi.require_gpu(query, "query")
        B, Hq, d = query.shape
        if d != self.head_dim or Hq % self.num_kv_heads:
            raise ValueError(f"Incompatible GQA shapes: Q={Hq}, H_kv={self.num_kv_heads}, d={d}")
        if key_cache.dtype != query.dtype:
            raise TypeError("the exact cache must have the query's dtype")
        if tuple(key_cache.shape[2:]) != (self.num_kv_heads, d) or not self.ring_cache_ok(key_cache, value_cache):
            raise ValueError("decode_attention_ring needs a (blocks, 16, H_kv, d) cache with contiguous channels, "
                             "equal key / value strides and word-aligned rows")
        query = query.contiguous()
        if scale is None:
            scale = 1.0 / math.sqrt(d)
        bt = block_table.contiguous()
        bt_stride = -bt.shape[0] if bt.dim() == 1 else bt.shape[1]      # negative: one shared row of that length
        seq_lens = seq_lens.to(device=self.device, dtype=torch.int32).contiguous()
        if n_split is None:
            if max_len is None:
                max_len = (bt.shape[-1]) * PAGE_TOKENS
            n_split = self.default_splits(B, max_len, Hq)
        if workspace is None:
            workspace = self.workspace(B, Hq, n_split)
        if out is None:
            out = torch.empty_like(query)
        ly = self.quantizer._layer()
        with _ffi.on_device(self.device):
            _ffi.check(_ffi.lib().tq_decode_attn_paged_ring(
                query.data_ptr(), _ffi.dtype_tag(query.dtype), B, Hq, self.num_kv_heads, self.data.data_ptr(),
                self.num_pages, bt.data_ptr(), bt_stride, seq_lens.data_ptr(), float(scale), C.byref(ly),
                C.byref(self.layout), key_cache.data_ptr(), value_cache.data_ptr(), key_cache.stride(0),
                key_cache.stride(1), key_cache.stride(2), int(ring_rows), out.data_ptr(), workspace.data_ptr(),
                n_split, _ffi.stream_ptr(self.device)), "tq_decode_attn_paged_ring")
        return out
