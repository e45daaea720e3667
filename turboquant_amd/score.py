"""Read path: decode attention over compressed history + exact recent tokens.

Mirrors turboquant/score.py of the reference (`MIN_HISTORY_FOR_TQ`,
`compute_hybrid_attention`, score.py:26-81).  The reference de-quantises the
whole history to fp32 and runs dense attention on every decode step
(score.py:84-173); here one fused kernel streams the packed pages, scores them
with the rotated / sketched query and accumulates values with an online
softmax, the exact recent tokens being one more partial in the same merge.
"""

from __future__ import annotations

import logging
import math
from typing import Optional

import torch

from .store import CompressedKVStore

logger = logging.getLogger("turboquant.score")

MIN_HISTORY_FOR_TQ = 16


def compute_hybrid_attention(query: torch.Tensor, store: CompressedKVStore, recent_k: Optional[torch.Tensor],
                             recent_v: Optional[torch.Tensor], num_query_heads: int,
                             scale: Optional[float] = None) -> torch.Tensor:
    """query (num_tokens, num_query_heads, head_dim); recent_k / recent_v
    (recent_len, num_kv_heads, head_dim) or None.  Every query token attends to
    all compressed tokens (only if there are at least MIN_HISTORY_FOR_TQ of
    them) followed by all recent tokens, without a mask.  Returns
    (num_tokens, num_query_heads, head_dim) in query's dtype; zeros when there
    is nothing to attend to."""
    head_dim, num_kv_heads = store.head_dim, store.num_kv_heads
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    n_hist = store.num_tokens
    has_history = n_hist >= MIN_HISTORY_FOR_TQ
    has_recent = recent_k is not None and recent_k.shape[0] > 0
    if not has_history and not has_recent:
        return torch.zeros(query.shape[0], num_query_heads, head_dim, device=query.device, dtype=query.dtype)

    gqa_ratio = num_query_heads // num_kv_heads
    T, Q, D = query.shape
    if Q != num_kv_heads * gqa_ratio:
        raise ValueError(f"Incompatible GQA shapes: Q={Q}, H_kv={num_kv_heads}, gqa_ratio={gqa_ratio}")

    # the kernel reads q and the recent tokens in one dtype; mixed inputs are widened to fp32 (lossless)
    work_dtype = query.dtype
    if has_recent and (recent_k.dtype != work_dtype or recent_v.dtype != work_dtype):
        work_dtype = torch.float32
    q = query.to(work_dtype)
    pool = store.ensure_pool(store.pool.dtype if store.pool is not None else
                             (recent_k.dtype if has_recent else query.dtype))
    seq_lens = torch.full((T,), n_hist if has_history else 0, dtype=torch.int32, device=pool.device)
    rk = rv = None
    if has_recent:
        rk = recent_k.to(work_dtype).unsqueeze(0).expand(T, *recent_k.shape)
        rv = recent_v.to(work_dtype).unsqueeze(0).expand(T, *recent_v.shape)
    out = pool.decode_attention(q, store.block_table[0], seq_lens, scale=scale, recent_k=rk, recent_v=rv,
                                max_len=max(n_hist, 1))
    return out.to(query.dtype)
