"""Attention-layer hooks for a vLLM-style model runner.

Mirrors turboquant/integration/vllm.py of the reference: the same modes
(`off | capture_only | hybrid | full_tq`, :36-52), `LayerConfig` / `LayerState`
(:55-85), `install_hooks` (:333-446), `free_kv_cache` (:449-501) and `get_stats`
(:504-528), against the same duck-typed contract:

  model_runner.compilation_config.static_forward_context : {layer name -> attention module}
  module.impl with num_kv_heads, head_size (or kv_lora_rank), optional num_heads / scale,
  bound methods impl.forward(layer, query, key, value, kv_cache, attn_metadata,
  output=None, output_scale=None, output_block_scale=None) and, when the backend has
  one, impl.do_kv_cache_update(layer, key, value, kv_cache, slot_mapping);
  attn_metadata.num_actual_tokens and .max_query_len.

vLLM itself is never imported.  Writes go through `KVCaptureEngine` into the
paged compressed store (one fused quantise call per chunk); decode steps in
hybrid mode are answered by the fused decode-attention kernel over the store
plus the exact ring.  As in the reference, a layer state holds ONE sequence.
"""

from __future__ import annotations

import logging
import math
import types
from dataclasses import dataclass, field
from typing import Dict, Optional

import torch
import torch.nn.functional as F

from ..capture import KVCaptureEngine
from ..score import MIN_HISTORY_FOR_TQ, compute_hybrid_attention
from ..store import CompressedKVStore

logger = logging.getLogger("turboquant.integration.vllm")

MODE_OFF = "off"
MODE_CAPTURE_ONLY = "capture_only"
MODE_HYBRID = "hybrid"
MODE_FULL_TQ = "full_tq"
_VALID_MODES = (MODE_OFF, MODE_CAPTURE_ONLY, MODE_HYBRID, MODE_FULL_TQ)

_GLOBAL_MODE = MODE_CAPTURE_ONLY


def set_mode(mode: str):
    global _GLOBAL_MODE
    assert mode in _VALID_MODES, f"Invalid mode: {mode}. Valid: {_VALID_MODES}"
    _GLOBAL_MODE = mode
    logger.info("[TurboQuant] Mode set to: %s", mode)


def get_mode() -> str:
    return _GLOBAL_MODE


@dataclass
class LayerConfig:
    head_dim: int
    num_kv_heads: int
    num_query_heads: int
    key_bits: int = 3
    value_bits: int = 2
    value_group_size: int = 32
    ring_capacity: int = 128
    layer_idx: int = 0
    backend_kind: str = "flash"          # "flash" | "mla"
    device: torch.device = field(default_factory=lambda: torch.device("cuda"))


@dataclass
class LayerState:
    """Run-time state of one attention layer: its compressed store and capture engine."""
    config: LayerConfig
    store: CompressedKVStore
    engine: KVCaptureEngine
    _log_count: int = 0

    @property
    def supports_hybrid(self) -> bool:
        return self.config.backend_kind == "flash"

    def reset(self):
        self.engine.reset()
        self._log_count = 0


def _new_state(cfg: LayerConfig) -> LayerState:
    store = CompressedKVStore(head_dim=cfg.head_dim, num_kv_heads=cfg.num_kv_heads, key_bits=cfg.key_bits,
                              value_bits=cfg.value_bits, value_group_size=cfg.value_group_size, device=cfg.device,
                              layer_idx=cfg.layer_idx)
    return LayerState(config=cfg, store=store,
                      engine=KVCaptureEngine(store=store, ring_capacity=cfg.ring_capacity, device=cfg.device))


def _query_heads_of(attn_module, impl) -> int:
    for owner, name in ((attn_module, "num_heads"), (attn_module, "num_attention_heads"), (impl, "num_heads")):
        n = getattr(owner, name, None)
        if n:
            return int(n)
    return int(impl.num_kv_heads)


def _is_mla_impl(impl) -> bool:
    """Latent-attention backends expose forward_mqa + do_kv_cache_update and no forward (:113-118)."""
    return hasattr(impl, "forward_mqa") and hasattr(impl, "do_kv_cache_update") and not hasattr(impl, "forward")


class _FlashLayerHooks:
    """The replacement methods of one standard attention layer.  `forward` and
    `kv_update` take the impl as first argument, like the unbound originals."""

    def __init__(self, state: LayerState, orig_forward, orig_update, no_alloc: bool):
        self.state = state
        self.orig_forward = orig_forward
        self.orig_update = orig_update
        self.no_alloc = no_alloc
        self.capture_in_forward = orig_update is None      # backends that write the cache inside forward()

    # ---- capture -----------------------------------------------------------------
    def _ingest(self, key, value, num_tokens: int):
        eng = self.state.engine
        if num_tokens <= 1:
            eng.ingest_decode(key[:num_tokens], value[:num_tokens], num_tokens)
        else:
            eng.ingest_prefill(key[:num_tokens], value[:num_tokens], num_tokens)

    def kv_update(self, impl, layer, key, value, kv_cache, slot_mapping):
        if not self.no_alloc:                              # keep the engine's own paged cache up to date
            self.orig_update(impl, layer, key, value, kv_cache, slot_mapping)
        if _GLOBAL_MODE == MODE_OFF:
            return
        self._ingest(key, value, int(slot_mapping.shape[0]))

    # ---- attention ---------------------------------------------------------------
    def _shape_q(self, query, n):
        cfg = self.state.config
        q = query[:n]
        return q.view(n, cfg.num_query_heads, cfg.head_dim) if q.dim() == 2 else q

    def _deliver(self, result, query, output, n):
        """Hand back `result` (n, Hq, d) the way the backend's forward does: into
        output[:n] when given, else shaped like the query (:282-288)."""
        cfg = self.state.config
        flat = result.reshape(n, cfg.num_query_heads * cfg.head_dim).to(query.dtype)
        if output is not None:
            dst = output[:n]
            dst.copy_((result if dst.dim() == 3 else flat).to(dst.dtype))
            return output
        return result.to(query.dtype) if query.dim() == 3 else flat

    def _dense_causal_prefill(self, impl, query, key, value, n):
        """Prefill attention when the engine's paged cache is not allocated (:148-180)."""
        cfg = self.state.config
        q = self._shape_q(query, n)
        k, v = key[:n], value[:n]
        if k.dim() == 2:
            k = k.view(n, cfg.num_kv_heads, cfg.head_dim)
            v = v.view(n, cfg.num_kv_heads, cfg.head_dim)
        rep = cfg.num_query_heads // cfg.num_kv_heads
        if rep > 1:
            k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
        scale = getattr(impl, "scale", 1.0 / math.sqrt(cfg.head_dim))
        out = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                             v.transpose(0, 1)[None], is_causal=True, scale=scale)
        return out[0].transpose(0, 1)

    def forward(self, impl, layer, query, key, value, kv_cache, attn_metadata, output=None, output_scale=None,
                output_block_scale=None):
        mode = _GLOBAL_MODE
        passthrough = lambda: self.orig_forward(impl, layer, query, key, value, kv_cache, attn_metadata, output,
                                                output_scale, output_block_scale)
        if self.capture_in_forward and mode != MODE_OFF and attn_metadata is not None:
            self._ingest(key, value, int(getattr(attn_metadata, "num_actual_tokens", key.shape[0])))
        if mode in (MODE_OFF, MODE_CAPTURE_ONLY) or attn_metadata is None:      # None = the engine's profiling pass
            return passthrough()

        state = self.state
        if attn_metadata.max_query_len > 1:                                     # prefill
            if not self.no_alloc:
                return passthrough()
            n = attn_metadata.num_actual_tokens
            return self._deliver(self._dense_causal_prefill(impl, query, key, value, n), query, output, n)

        if mode == MODE_HYBRID and state.supports_hybrid and state.store.num_tokens >= MIN_HISTORY_FOR_TQ:
            n = attn_metadata.num_actual_tokens
            recent = state.engine.ring.peek()
            result = compute_hybrid_attention(query=self._shape_q(query, n), store=state.store,
                                              recent_k=recent[0] if recent else None,
                                              recent_v=recent[1] if recent else None,
                                              num_query_heads=state.config.num_query_heads,
                                              scale=getattr(impl, "scale", None))
            return self._deliver(result, query, output, n)

        if self.no_alloc:                                   # nothing to attend through: zeros, as the reference (:301-311)
            n = getattr(attn_metadata, "num_actual_tokens", query.shape[0])
            if query.dim() == 3:
                return torch.zeros_like(query[:n])
            cfg = state.config
            return torch.zeros(n, cfg.num_query_heads * cfg.head_dim, dtype=query.dtype, device=query.device)
        return passthrough()


class _MlaLayerHooks:
    """Latent-attention layers are observed, not captured (:321-340 of the reference)."""

    def __init__(self, state: LayerState, orig_forward_mqa, orig_update):
        self.state, self.orig_forward_mqa, self.orig_update = state, orig_forward_mqa, orig_update

    def kv_update(self, impl, kv_c_normed, k_pe, kv_cache, slot_mapping, kv_cache_dtype, k_scale):
        self.orig_update(impl, kv_c_normed, k_pe, kv_cache, slot_mapping, kv_cache_dtype, k_scale)
        if self.state._log_count < 1:
            logger.info("[TurboQuant] MLA update observed on layer %d; the compressed MLA path is not built.",
                        self.state.config.layer_idx)
            self.state._log_count += 1

    def forward_mqa(self, impl, q, kv_c_and_k_pe_cache, attn_metadata, layer):
        return self.orig_forward_mqa(impl, q, kv_c_and_k_pe_cache, attn_metadata, layer)


def _bind(impl, fn):
    """Bound method on `impl` that calls fn(impl, *args, **kwargs)."""
    return types.MethodType(lambda self, *a, _fn=fn, **kw: _fn(self, *a, **kw), impl)


def _unbound(method):
    return getattr(method, "__func__", None) or (lambda self, *a, _m=method, **kw: _m(*a, **kw))


def install_hooks(model_runner, key_bits: int = 3, value_bits: int = 2, value_group_size: int = 32,
                  ring_capacity: int = 128, initial_layers_count: int = 4,
                  initial_layers_key_bits: Optional[int] = None, mode: str = MODE_CAPTURE_ONLY,
                  no_alloc: bool = False) -> Dict[str, LayerState]:
    """Hook every attention layer of `model_runner`; returns {layer name: LayerState}.
    The first `initial_layers_count` layers get `initial_layers_key_bits` (default
    min(key_bits + 1, 4)) key bits."""
    global _GLOBAL_MODE
    _GLOBAL_MODE = mode
    if initial_layers_key_bits is None:
        initial_layers_key_bits = min(key_bits + 1, 4)

    states: Dict[str, LayerState] = {}
    device = model_runner.device
    idx = 0
    for name, module in model_runner.compilation_config.static_forward_context.items():
        impl = getattr(module, "impl", None)
        if impl is None or getattr(impl, "num_kv_heads", None) is None:
            continue
        if hasattr(impl, "head_size"):
            head_dim = int(impl.head_size)
        elif hasattr(impl, "kv_lora_rank"):
            head_dim = int(impl.kv_lora_rank)
        else:
            continue
        kind = "mla" if _is_mla_impl(impl) else "flash"
        cfg = LayerConfig(head_dim=head_dim, num_kv_heads=int(impl.num_kv_heads),
                          num_query_heads=_query_heads_of(module, impl),
                          key_bits=initial_layers_key_bits if idx < initial_layers_count else key_bits,
                          value_bits=value_bits, value_group_size=min(value_group_size, head_dim),
                          ring_capacity=ring_capacity, layer_idx=idx, backend_kind=kind, device=device)
        state = _new_state(cfg)
        states[name] = state

        if kind == "flash":
            has_update = hasattr(impl, "do_kv_cache_update")
            hooks = _FlashLayerHooks(state, _unbound(impl.forward),
                                     _unbound(impl.do_kv_cache_update) if has_update else None, no_alloc)
            if has_update:
                impl.do_kv_cache_update = _bind(impl, hooks.kv_update)
            elif idx == 0:
                logger.info("[TurboQuant] backend has no do_kv_cache_update; capturing K/V in forward()")
            impl.forward = _bind(impl, hooks.forward)
        else:
            hooks = _MlaLayerHooks(state, _unbound(impl.forward_mqa) if hasattr(impl, "forward_mqa") else None,
                                   _unbound(impl.do_kv_cache_update))
            impl.do_kv_cache_update = _bind(impl, hooks.kv_update)
            if hooks.orig_forward_mqa is not None:
                impl.forward_mqa = _bind(impl, hooks.forward_mqa)
        impl._tq_layer_state = state
        idx += 1

    model_runner._tq_layer_states = states
    model_runner._tq_no_alloc = no_alloc
    logger.info("[TurboQuant] Hooks on %d layers (mode=%s, no_alloc=%s)", len(states), mode, no_alloc)
    return states


def _release_paged_caches(model_runner, states) -> int:
    """Swap the engine's exact paged KV tensors of the hooked standard layers for a
    one-byte placeholder; returns the bytes released."""
    ctx = model_runner.compilation_config.static_forward_context
    tiny = torch.zeros(1, dtype=torch.int8, device=model_runner.device)
    released, freed = set(), 0
    for name, state in states.items():
        if not getattr(state, "supports_hybrid", False) or name not in ctx:
            continue
        kv_list = getattr(ctx[name], "kv_cache", None)
        if kv_list and hasattr(kv_list[0], "data_ptr"):
            old = kv_list[0]
            released.add(old.data_ptr())
            freed += old.nelement() * old.element_size()
            kv_list[0] = tiny
    caches = getattr(model_runner, "kv_caches", [])
    for i, entry in enumerate(caches):
        if isinstance(entry, list):
            for j, t in enumerate(entry):
                if hasattr(t, "data_ptr") and t.data_ptr() in released:
                    entry[j] = tiny
        elif hasattr(entry, "data_ptr") and entry.data_ptr() in released:
            caches[i] = tiny
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return freed


def free_kv_cache(model_runner) -> int:
    """Free the exact paged KV cache of the hooked standard-attention layers
    (latent-attention layers keep theirs).  Returns the bytes freed."""
    states = getattr(model_runner, "_tq_layer_states", None)
    if not states:
        logger.warning("[TurboQuant] No layer states found, nothing to free")
        return 0
    freed = _release_paged_caches(model_runner, states)
    logger.info("[TurboQuant] Freed %.0f MB KV cache (%d layers)", freed / 1e6, len(states))
    return freed


def get_stats(model_runner) -> dict:
    states = getattr(model_runner, "_tq_layer_states", None)
    if not states:
        return {}
    n = max(len(states), 1)
    return {
        "num_layers": len(states),
        "total_compressed_tokens": sum(s.store.num_tokens for s in states.values()) // n,
        "total_buffered_tokens": sum(s.engine.ring.size for s in states.values()) // n,
        "total_memory_bytes": sum(s.store.memory_bytes() for s in states.values()),
        "mode": _GLOBAL_MODE,
    }
