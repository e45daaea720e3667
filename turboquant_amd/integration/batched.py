"""Batch-aware attention hooks over the paged compressed pool (new design).

The reference's hooks keep ONE sequence per layer: one store and one ring, and
"prefill vs decode" is `num_tokens > 1` (integration/vllm.py:130-145); that is
what `turboquant_amd.integration.vllm` mirrors.  A serving engine decodes many
sequences per step through block tables.  This module is the batch-aware
counterpart on the same duck-typed contract (integration/vllm.py:361-441):
every hooked standard-attention layer owns a `PagedKVPool` whose page numbers
ARE the engine's block numbers (block size 16 = page size), written from the
K/V tensors of every step and read by the fused decode kernel with the engine's
own block table and sequence lengths.

Besides `num_actual_tokens` and `max_query_len`, `attn_metadata` must carry

  seq_lens        (B,)   int32  length of each sequence INCLUDING this step's tokens
  block_table     (B, max_blocks) int32
  query_start_loc (B+1,) int32  row range of each sequence in the step's token-major tensors

(optionally `seq_lens_cpu` / `query_start_loc_cpu`, which spare a device read on
prefill steps).  Modes are those of `integration.vllm`:

  off           nothing is written, the backend answers
  capture_only  pages are written, the backend answers
  hybrid        decode steps are answered from the pool, the last `ring_capacity`
                tokens of each sequence exactly from the engine's paged cache
                (layout (2, num_blocks, 16, H_kv, d)); prefill by the backend
  full_tq       decode steps are answered from the pool alone; prefill by the
                backend, or by dense causal attention over the step's own K/V
                when the engine's cache was never allocated (`no_alloc`)
"""

from __future__ import annotations

import logging
import math
from dataclasses import dataclass
from typing import Dict, Optional

import torch
import torch.nn.functional as F

from ..paged import PAGE_TOKENS, PagedKVPool
from ..quantizer import TurboQuantProd
from . import vllm as _single
from .vllm import (MODE_CAPTURE_ONLY, MODE_HYBRID, MODE_OFF, LayerConfig, _bind, _is_mla_impl, _query_heads_of,
                   _unbound)

logger = logging.getLogger("turboquant.integration.batched")


def _host_list(meta, name):
    cpu = getattr(meta, name + "_cpu", None)
    t = cpu if cpu is not None else getattr(meta, name)
    return [int(x) for x in t.tolist()]


@dataclass
class BatchedLayerState:
    """One attention layer: its quantiser and the compressed pool that shadows the engine's blocks."""
    config: LayerConfig
    quantizer: TurboQuantProd
    pool: PagedKVPool
    tokens_written: int = 0
    decode_steps: int = 0

    @property
    def supports_hybrid(self) -> bool:
        return True

    # ---- write -------------------------------------------------------------------
    def write(self, key: torch.Tensor, value: torch.Tensor, meta) -> None:
        """Quantise this step's tokens (n, H_kv, d) into the pages their sequences own."""
        cfg = self.config
        n = int(meta.num_actual_tokens)
        k = key[:n].reshape(n, cfg.num_kv_heads, cfg.head_dim)
        v = value[:n].reshape(n, cfg.num_kv_heads, cfg.head_dim)
        table = meta.block_table
        if int(meta.max_query_len) == 1:                       # one token per sequence: a single batched append
            start = meta.seq_lens.to(torch.int32) - 1
            self.pool.append(k[:, None], v[:, None], table, start_pos=start)
        else:                                                  # ragged rows: still one call, nothing read back
            qsl = meta.query_start_loc.to(device=k.device, dtype=torch.int32)
            run = qsl[1:] - qsl[:-1]
            start = meta.seq_lens.to(device=k.device, dtype=torch.int32) - run
            self.pool.append_ragged(k, v, qsl[:-1], run, start, table, max_run=int(meta.max_query_len))
        self.tokens_written += n

    def ingest_paged_cache(self, kv_cache: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor,
                           max_tokens: Optional[int] = None) -> None:
        """Compress what the engine's exact paged cache (2, num_blocks, 16, H_kv, d) already holds for the
        sequences of `block_table`: tokens [0, seq_lens[b]) of every sequence, read in place through the
        block table and written to the pages of the same numbers (the batch counterpart of
        capture.py:187-217, without the gather copy)."""
        self.pool.append_from_blocks(kv_cache[0], kv_cache[1], block_table, block_table, seq_lens,
                                     max_tokens=max_tokens)
        self.tokens_written += int(seq_lens.sum())

    # ---- read --------------------------------------------------------------------
    def _exact_tail(self, kv_cache, meta):
        """The last `ring_capacity` tokens of every sequence from the engine's paged cache:
        (B, R, H_kv, d) keys and values, their valid counts, and the compressed lengths."""
        cfg = self.config
        R = cfg.ring_capacity
        ok = (torch.is_tensor(kv_cache) and kv_cache.dim() == 5 and kv_cache.shape[0] == 2 and
              kv_cache.shape[2] == PAGE_TOKENS and kv_cache.shape[3] == cfg.num_kv_heads and
              kv_cache.shape[4] == cfg.head_dim)
        if not ok or R <= 0:
            return None
        seq = meta.seq_lens.to(torch.int64)
        tail = torch.clamp(seq, max=R)                                          # (B,)
        pos = (seq - tail)[:, None] + torch.arange(R, device=seq.device)[None]  # (B, R) token positions
        pos = torch.minimum(pos, (seq - 1).clamp_min(0)[:, None])
        blocks = torch.gather(meta.block_table.to(torch.int64), 1, pos // PAGE_TOKENS)
        slot = blocks * PAGE_TOKENS + pos % PAGE_TOKENS
        flat_k = kv_cache[0].reshape(-1, cfg.num_kv_heads, cfg.head_dim)
        flat_v = kv_cache[1].reshape(-1, cfg.num_kv_heads, cfg.head_dim)
        return flat_k[slot], flat_v[slot], tail.to(torch.int32), (seq - tail).to(torch.int32)

    def attend(self, query: torch.Tensor, meta, scale: Optional[float] = None, kv_cache=None,
               hybrid: bool = False) -> torch.Tensor:
        """One query token per sequence, (B, H_q, d) -> (B, H_q, d)."""
        self.decode_steps += 1
        cfg = self.config
        if (hybrid and cfg.ring_capacity > 0 and torch.is_tensor(kv_cache) and kv_cache.dim() == 5 and
                kv_cache.shape[0] == 2 and tuple(kv_cache.shape[2:]) == (PAGE_TOKENS, cfg.num_kv_heads, cfg.head_dim) and
                kv_cache.dtype == query.dtype and cfg.ring_capacity <= 1024 and
                self.pool.ring_cache_ok(kv_cache[0], kv_cache[1])):
            # the exact tokens are read in place from the engine's cache, through the step's block table
            return self.pool.decode_attention_ring(query, meta.block_table, meta.seq_lens, kv_cache[0], kv_cache[1],
                                                   cfg.ring_capacity, scale=scale,
                                                   max_len=getattr(meta, "max_seq_len", None))
        recent = self._exact_tail(kv_cache, meta) if hybrid else None
        if recent is None:
            return self.pool.decode_attention(query, meta.block_table, meta.seq_lens, scale=scale,
                                              max_len=getattr(meta, "max_seq_len", None))
        rk, rv, rlen, hist = recent
        return self.pool.decode_attention(query, meta.block_table, hist, scale=scale, recent_k=rk, recent_v=rv,
                                          recent_len=rlen, max_len=getattr(meta, "max_seq_len", None))

    def memory_bytes(self) -> int:
        return self.pool.data.numel()


class _BatchedLayerHooks:
    """Replacement methods of one standard attention layer (impl first, like the unbound originals)."""

    def __init__(self, state: BatchedLayerState, orig_forward, orig_update, no_alloc: bool):
        self.state, self.orig_forward, self.orig_update, self.no_alloc = state, orig_forward, orig_update, no_alloc

    def kv_update(self, impl, layer, key, value, kv_cache, slot_mapping):
        if not self.no_alloc:                                  # the engine's exact cache stays current
            self.orig_update(impl, layer, key, value, kv_cache, slot_mapping)

    def _deliver(self, result, query, output, n):
        cfg = self.state.config
        flat = result.reshape(n, cfg.num_query_heads * cfg.head_dim).to(query.dtype)
        if output is not None:
            dst = output[:n]
            dst.copy_((result if dst.dim() == 3 else flat).to(dst.dtype))
            return output
        return result.to(query.dtype) if query.dim() == 3 else flat

    def _dense_prefill(self, impl, query, key, value, meta, n):
        """Causal attention of every sequence over its own rows of this step (first chunk of a
        sequence only: there is no exact cache to read earlier tokens from)."""
        cfg = self.state.config
        q = query[:n].reshape(n, cfg.num_query_heads, cfg.head_dim)
        k = key[:n].reshape(n, cfg.num_kv_heads, cfg.head_dim)
        v = value[:n].reshape(n, cfg.num_kv_heads, cfg.head_dim)
        rep = cfg.num_query_heads // cfg.num_kv_heads
        scale = getattr(impl, "scale", 1.0 / math.sqrt(cfg.head_dim))
        out = torch.empty_like(q)
        lens, qsl = _host_list(meta, "seq_lens"), _host_list(meta, "query_start_loc")
        for b in range(len(lens)):
            r0, r1 = qsl[b], qsl[b + 1]
            if r1 <= r0:
                continue
            if lens[b] != r1 - r0:
                raise RuntimeError("chunked prefill needs the engine's paged cache (hooks installed with no_alloc)")
            kb, vb = k[r0:r1].repeat_interleave(rep, 1), v[r0:r1].repeat_interleave(rep, 1)
            o = F.scaled_dot_product_attention(q[r0:r1].transpose(0, 1)[None], kb.transpose(0, 1)[None],
                                               vb.transpose(0, 1)[None], is_causal=True, scale=scale)
            out[r0:r1] = o[0].transpose(0, 1)
        return out

    def forward(self, impl, layer, query, key, value, kv_cache, attn_metadata, output=None, output_scale=None,
                output_block_scale=None):
        mode = _single.get_mode()
        passthrough = lambda: self.orig_forward(impl, layer, query, key, value, kv_cache, attn_metadata, output,
                                                output_scale, output_block_scale)
        if mode == MODE_OFF or attn_metadata is None:          # None = the engine's profiling pass
            return passthrough()
        self.state.write(key, value, attn_metadata)
        n = int(attn_metadata.num_actual_tokens)
        if mode == MODE_CAPTURE_ONLY:
            return passthrough()
        if int(attn_metadata.max_query_len) > 1:               # prefill (or a mixed step): exact attention
            if not self.no_alloc:
                return passthrough()
            return self._deliver(self._dense_prefill(impl, query, key, value, attn_metadata, n), query, output, n)
        cfg = self.state.config
        q = query[:n].reshape(n, cfg.num_query_heads, cfg.head_dim)
        result = self.state.attend(q, attn_metadata, scale=getattr(impl, "scale", None), kv_cache=kv_cache,
                                   hybrid=(mode == MODE_HYBRID and not self.no_alloc))
        return self._deliver(result, query, output, n)


def install_batched_hooks(model_runner, num_blocks: int, key_bits: int = 3, value_bits: int = 2,
                          value_group_size: int = 32, ring_capacity: int = 128, initial_layers_count: int = 4,
                          initial_layers_key_bits: Optional[int] = None, mode: str = MODE_CAPTURE_ONLY,
                          no_alloc: bool = False, dtype: torch.dtype = torch.bfloat16) -> Dict[str, BatchedLayerState]:
    """Hook every standard attention layer of `model_runner` with a compressed pool of `num_blocks`
    16-token pages (the engine's block count); returns {layer name: BatchedLayerState}.  Bit widths are
    assigned as by `install_hooks` (integration/vllm.py:333-359).  Latent-attention layers are left alone."""
    _single.set_mode(mode)
    if initial_layers_key_bits is None:
        initial_layers_key_bits = min(key_bits + 1, 4)
    states: Dict[str, BatchedLayerState] = {}
    device = torch.device(model_runner.device)
    idx = 0
    for name, module in model_runner.compilation_config.static_forward_context.items():
        impl = getattr(module, "impl", None)
        if impl is None or getattr(impl, "num_kv_heads", None) is None or not hasattr(impl, "head_size"):
            continue
        if _is_mla_impl(impl):
            continue
        head_dim = int(impl.head_size)
        cfg = LayerConfig(head_dim=head_dim, num_kv_heads=int(impl.num_kv_heads),
                          num_query_heads=_query_heads_of(module, impl),
                          key_bits=initial_layers_key_bits if idx < initial_layers_count else key_bits,
                          value_bits=value_bits, value_group_size=min(value_group_size, head_dim),
                          ring_capacity=ring_capacity, layer_idx=idx, backend_kind="flash", device=device)
        tq = TurboQuantProd(head_dim, bits=cfg.key_bits, device=device, seed=42 + 7 * idx)
        pool = PagedKVPool(tq, cfg.num_kv_heads, num_blocks, value_bits=value_bits,
                           value_group_size=cfg.value_group_size, dtype=dtype, device=device)
        state = BatchedLayerState(config=cfg, quantizer=tq, pool=pool)
        states[name] = state
        has_update = hasattr(impl, "do_kv_cache_update")
        hooks = _BatchedLayerHooks(state, _unbound(impl.forward),
                                   _unbound(impl.do_kv_cache_update) if has_update else None, no_alloc)
        if has_update:
            impl.do_kv_cache_update = _bind(impl, hooks.kv_update)
        impl.forward = _bind(impl, hooks.forward)
        impl._tq_layer_state = state
        idx += 1
    model_runner._tq_layer_states = states
    model_runner._tq_no_alloc = no_alloc
    logger.info("[TurboQuant] Batched hooks on %d layers (mode=%s, no_alloc=%s)", len(states), mode, no_alloc)
    return states


def get_batched_stats(model_runner) -> dict:
    states = getattr(model_runner, "_tq_layer_states", None) or {}
    return {"num_layers": len(states),
            "tokens_written_per_layer": max((s.tokens_written for s in states.values()), default=0),
            "decode_steps": max((s.decode_steps for s in states.values()), default=0),
            "total_memory_bytes": sum(s.memory_bytes() for s in states.values()),
            "mode": _single.get_mode()}
