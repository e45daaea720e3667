"""Legacy entry points of the attention-backend shim.

Mirrors turboquant/vllm_attn_backend.py of the reference: the three legacy mode
names (:16-26), `install_turboquant_hooks` (:41-70), `free_kv_cache` (:216-264)
and `enable_no_alloc` (:76-213), all delegating to `integration.vllm`.
"""

from __future__ import annotations

import logging
from typing import Optional

from .integration import vllm as _backend

logger = logging.getLogger("turboquant.attn")

MODE_SHADOW = "shadow"
MODE_ACCUMULATE = "accumulate"
MODE_ACTIVE = "active"
_VALID_MODES = (MODE_SHADOW, MODE_ACCUMULATE, MODE_ACTIVE)

_LEGACY_TO_NEW = {
    MODE_SHADOW: _backend.MODE_CAPTURE_ONLY,
    MODE_ACCUMULATE: _backend.MODE_CAPTURE_ONLY,
    MODE_ACTIVE: _backend.MODE_HYBRID,
}

_GLOBAL_MODE = MODE_ACCUMULATE
_TQ_NO_ALLOC_CONFIG: Optional[dict] = None


def set_mode(mode: str):
    global _GLOBAL_MODE
    assert mode in _VALID_MODES
    _GLOBAL_MODE = mode
    _backend.set_mode(_LEGACY_TO_NEW[mode])


def get_mode() -> str:
    return _GLOBAL_MODE


def install_turboquant_hooks(model_runner, key_bits: int = 3, value_bits: int = 2, value_group_size: int = 32,
                             buffer_size: int = 128, initial_layers_count: int = 4,
                             initial_layers_key_bits: Optional[int] = None, mode: str = MODE_ACCUMULATE,
                             no_alloc: bool = False):
    global _GLOBAL_MODE
    states = _backend.install_hooks(model_runner, key_bits=key_bits, value_bits=value_bits,
                                    value_group_size=value_group_size, ring_capacity=buffer_size,
                                    initial_layers_count=initial_layers_count,
                                    initial_layers_key_bits=initial_layers_key_bits,
                                    mode=_LEGACY_TO_NEW.get(mode, _backend.MODE_CAPTURE_ONLY), no_alloc=no_alloc)
    _GLOBAL_MODE = mode
    model_runner._tq_states = states
    model_runner._tq_no_alloc = no_alloc
    return states


def free_kv_cache(model_runner) -> int:
    if getattr(model_runner, "_tq_layer_states", None):
        return _backend.free_kv_cache(model_runner)
    states = getattr(model_runner, "_tq_states", None)
    if not states:
        return 0
    return _backend._release_paged_caches(model_runner, states)


def enable_no_alloc(key_bits: int = 3, value_bits: int = 2, buffer_size: int = 128, initial_layers_count: int = 4):
    """Arrange for the hooks to be installed on every worker while the engine
    starts, before it sizes its KV cache.  Call before creating `vllm.LLM`.
    Needs vLLM's v1 executor classes; raises ImportError when vLLM is absent."""
    global _TQ_NO_ALLOC_CONFIG
    _TQ_NO_ALLOC_CONFIG = dict(key_bits=key_bits, value_bits=value_bits, buffer_size=buffer_size,
                               initial_layers_count=initial_layers_count)
    from vllm.v1.executor.abstract import Executor      # noqa: deferred, optional dependency

    if getattr(Executor, "_tq_patched", False):
        return
    original = Executor.get_kv_cache_specs

    def _install_on_worker(worker):
        cfg = _TQ_NO_ALLOC_CONFIG
        states = install_turboquant_hooks(worker.model_runner, key_bits=cfg["key_bits"],
                                          value_bits=cfg["value_bits"], buffer_size=cfg["buffer_size"],
                                          initial_layers_count=cfg["initial_layers_count"], mode=MODE_ACTIVE,
                                          no_alloc=True)
        return {"hooks": len(states),
                "flash_layers": sum(1 for s in states.values() if s.supports_hybrid)}

    def get_kv_cache_specs(self):
        if _TQ_NO_ALLOC_CONFIG is not None:
            report = self.collective_rpc(_install_on_worker)
            logger.info("[TurboQuant] Installed no_alloc hooks: %s", report)
        return original(self)

    Executor.get_kv_cache_specs = get_kv_cache_specs
    Executor._tq_patched = True
