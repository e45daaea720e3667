"""A minimal decoder-only transformer behind the attention-backend contract.

Not a model family: just enough of a dense pre-norm transformer (RMSNorm, rotary
Q/K, grouped-query attention, SwiGLU FFN, random bf16 weights) and of a model
runner (`compilation_config.static_forward_context`, per-layer attention modules
with an `impl` that has `do_kv_cache_update` / `forward`, paged exact KV cache,
attention metadata) to drive the hooks of `integration.vllm` / `integration.batched`
end to end the way a serving engine would: a full decode step of a batch of
sequences through every layer.  The dense parts are plain torch; the attention
backend is where the compressed path plugs in.
"""

from __future__ import annotations

import math
import types
from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F

BLOCK = 16            # tokens per KV block of the runner = tokens per compressed page


@dataclass
class StepMetadata:
    """What the attention backends read (the fields of vLLM's attention metadata used here)."""
    num_actual_tokens: int
    max_query_len: int
    max_seq_len: int
    seq_lens: torch.Tensor            # (B,) int32, device
    query_start_loc: torch.Tensor     # (B+1,) int32, device
    block_table: torch.Tensor         # (B, max_blocks) int32, device
    slot_mapping: torch.Tensor        # (T,) int64, device
    seq_lens_cpu: torch.Tensor
    query_start_loc_cpu: torch.Tensor


class DenseBackend:
    """Exact attention over a paged cache (2, num_blocks, BLOCK, H_kv, d): the stand-in for the engine's
    own backend.  Sequence by sequence, causal inside the step's rows."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_size: int):
        self.num_heads, self.num_kv_heads, self.head_size = num_heads, num_kv_heads, head_size
        self.scale = 1.0 / math.sqrt(head_size)

    def do_kv_cache_update(self, layer, key, value, kv_cache, slot_mapping):
        n = slot_mapping.shape[0]
        kv_cache[0].view(-1, self.num_kv_heads, self.head_size)[slot_mapping] = key[:n].view(n, self.num_kv_heads, -1)
        kv_cache[1].view(-1, self.num_kv_heads, self.head_size)[slot_mapping] = value[:n].view(n, self.num_kv_heads, -1)

    def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, output_scale=None,
                output_block_scale=None):
        m = attn_metadata
        n = m.num_actual_tokens
        q = query[:n].view(n, self.num_heads, self.head_size)
        out = torch.empty_like(q)
        rep = self.num_heads // self.num_kv_heads
        fk = kv_cache[0].view(-1, self.num_kv_heads, self.head_size)
        fv = kv_cache[1].view(-1, self.num_kv_heads, self.head_size)
        lens, qsl = m.seq_lens_cpu.tolist(), m.query_start_loc_cpu.tolist()
        for b, L in enumerate(lens):
            r0, r1 = qsl[b], qsl[b + 1]
            if r1 <= r0:
                continue
            pos = torch.arange(L, device=q.device)
            slot = m.block_table[b].long()[pos // BLOCK] * BLOCK + pos % BLOCK
            k = fk[slot].float().repeat_interleave(rep, 1)                  # (L, Hq, d)
            v = fv[slot].float().repeat_interleave(rep, 1)
            s = torch.einsum("thd,nhd->htn", q[r0:r1].float(), k) * self.scale
            t = r1 - r0
            mask = pos[None, :] > (L - t + torch.arange(t, device=q.device))[:, None]
            s = s.masked_fill(mask[None], float("-inf"))
            out[r0:r1] = torch.einsum("htn,nhd->thd", s.softmax(-1), v).to(q.dtype)
        res = out if query.dim() == 3 else out.reshape(n, -1)
        if output is not None:
            output[:n].copy_(res.reshape(output[:n].shape))
            return output
        return res


class AttentionModule:
    def __init__(self, impl, kv_cache: Optional[torch.Tensor]):
        self.impl = impl
        self.kv_cache = [kv_cache]
        self.num_heads = impl.num_heads


def _rms(x, w, eps=1e-6):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


def _rope(x, positions, theta=10000.0):
    """Rotary embedding on (T, H, d), rotate-half convention."""
    d = x.shape[-1]
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, device=x.device, dtype=torch.float32) / d))
    ang = positions.float()[:, None] * inv[None]                            # (T, d/2)
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., : d // 2].float(), x[..., d // 2:].float()
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], -1).to(x.dtype)


class MinimalRunner:
    """Random-init dense transformer + paged KV bookkeeping for a fixed batch of sequences.

    `num_blocks` blocks of 16 tokens are shared by all sequences; sequence b owns the blocks
    block_table[b].  With `exact_cache=False` no exact KV cache is allocated (the compressed pool is
    then the only KV storage and the hooks must run in `full_tq` mode with `no_alloc=True`)."""

    def __init__(self, n_layers: int, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int, ffn: int,
                 vocab: int, batch: int, max_seq_len: int, device, exact_cache: bool = True, seed: int = 0,
                 dtype: torch.dtype = torch.bfloat16):
        self.device = torch.device(device)
        self.n_layers, self.hidden, self.hq, self.hkv, self.d, self.vocab = n_layers, hidden, num_heads, num_kv_heads, head_dim, vocab
        self.batch, self.dtype = batch, dtype
        g = torch.Generator(device=self.device).manual_seed(seed)
        w = lambda *shape: (torch.randn(*shape, generator=g, device=self.device, dtype=torch.float32) * 0.02).to(dtype)
        self.embed = w(vocab, hidden)
        self.lm_head = w(hidden, vocab)
        self.final_norm = torch.ones(hidden, dtype=dtype, device=self.device)
        self.layers = []
        self.blocks_per_seq = (max_seq_len + BLOCK - 1) // BLOCK
        self.num_blocks = batch * self.blocks_per_seq
        ctx = {}
        self.kv_caches: List[torch.Tensor] = []
        for i in range(n_layers):
            impl = DenseBackend(num_heads, num_kv_heads, head_dim)
            cache = (torch.zeros(2, self.num_blocks, BLOCK, num_kv_heads, head_dim, dtype=dtype, device=self.device)
                     if exact_cache else None)
            mod = AttentionModule(impl, cache)
            ctx[f"model.layers.{i}.self_attn.attn"] = mod
            if cache is not None:
                self.kv_caches.append(cache)
            self.layers.append(types.SimpleNamespace(
                attn=mod, ln1=torch.ones(hidden, dtype=dtype, device=self.device),
                ln2=torch.ones(hidden, dtype=dtype, device=self.device),
                wqkv=w(hidden, (num_heads + 2 * num_kv_heads) * head_dim), wo=w(num_heads * head_dim, hidden),
                w_gate_up=w(hidden, 2 * ffn), w_down=w(ffn, hidden)))
        self.compilation_config = types.SimpleNamespace(static_forward_context=ctx)
        # sequence b owns a shuffled set of blocks, as a block allocator would hand them out
        perm = torch.randperm(self.num_blocks, generator=torch.Generator().manual_seed(seed + 1))
        self.block_table = perm.view(batch, self.blocks_per_seq).to(torch.int32).to(self.device)
        self.seq_lens = [0] * batch

    # ---- metadata ------------------------------------------------------------------
    def metadata(self, new_tokens: Sequence[int]) -> StepMetadata:
        """Metadata of a step that appends new_tokens[b] tokens to sequence b."""
        lens = [s + t for s, t in zip(self.seq_lens, new_tokens)]
        qsl = [0]
        slots = []
        for b, t in enumerate(new_tokens):
            qsl.append(qsl[-1] + t)
            pos = torch.arange(self.seq_lens[b], lens[b])
            slots.append(self.block_table[b].cpu().long()[pos // BLOCK] * BLOCK + pos % BLOCK)
        lens_t, qsl_t = torch.tensor(lens, dtype=torch.int32), torch.tensor(qsl, dtype=torch.int32)
        return StepMetadata(num_actual_tokens=qsl[-1], max_query_len=max(new_tokens), max_seq_len=max(lens),
                            seq_lens=lens_t.to(self.device), query_start_loc=qsl_t.to(self.device),
                            block_table=self.block_table, slot_mapping=torch.cat(slots).to(self.device),
                            seq_lens_cpu=lens_t, query_start_loc_cpu=qsl_t)

    def decode_metadata(self) -> StepMetadata:
        """One new token per sequence, built without host loops (seq_lens advance on the device)."""
        lens_t = torch.tensor([s + 1 for s in self.seq_lens], dtype=torch.int32)
        dev_lens = lens_t.to(self.device)
        pos = (dev_lens - 1).long()
        slot = torch.gather(self.block_table.long(), 1, (pos // BLOCK)[:, None])[:, 0] * BLOCK + pos % BLOCK
        qsl = torch.arange(self.batch + 1, dtype=torch.int32)
        return StepMetadata(num_actual_tokens=self.batch, max_query_len=1, max_seq_len=int(lens_t.max()),
                            seq_lens=dev_lens, query_start_loc=qsl.to(self.device), block_table=self.block_table,
                            slot_mapping=slot, seq_lens_cpu=lens_t, query_start_loc_cpu=qsl)

    # ---- one model step ------------------------------------------------------------
    def step(self, tokens: torch.Tensor, meta: StepMetadata, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        """tokens (T,) of the step (token-major over sequences) -> logits of each sequence's last token
        (B, vocab); advances the sequence lengths."""
        T = tokens.shape[0]
        if positions is None:
            lens, qsl = meta.seq_lens_cpu.tolist(), meta.query_start_loc_cpu.tolist()
            positions = torch.cat([torch.arange(L - (qsl[b + 1] - qsl[b]), L) for b, L in enumerate(lens)]).to(self.device)
        x = self.embed[tokens]
        hq, hkv, d = self.hq, self.hkv, self.d
        for lay in self.layers:
            h = _rms(x, lay.ln1)
            qkv = h @ lay.wqkv
            q, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)
            q = _rope(q.view(T, hq, d), positions).reshape(T, hq * d)
            k = _rope(k.view(T, hkv, d), positions)
            v = v.view(T, hkv, d).contiguous()
            impl, cache = lay.attn.impl, lay.attn.kv_cache[0]
            if hasattr(impl, "do_kv_cache_update"):
                impl.do_kv_cache_update(lay.attn, k, v, cache, meta.slot_mapping)
            attn = impl.forward(lay.attn, q, k, v, cache, meta)
            x = x + attn.reshape(T, hq * d) @ lay.wo
            h = _rms(x, lay.ln2)
            gate, up = (h @ lay.w_gate_up).chunk(2, dim=-1)
            x = x + (F.silu(gate) * up) @ lay.w_down
        last = meta.query_start_loc[1:].long() - 1
        logits = _rms(x[last], self.final_norm) @ self.lm_head
        self.seq_lens = meta.seq_lens_cpu.tolist()
        return logits

    def decode_step(self, tokens: torch.Tensor) -> torch.Tensor:
        """tokens (B,): one new token per sequence."""
        meta = self.decode_metadata()
        return self.step(tokens, meta, positions=(meta.seq_lens - 1).long())

    # ---- the decode step as a HIP graph ----------------------------------------------
    def capture_decode_step(self, max_seq_len: int, first_tokens: torch.Tensor):
        """Run one decode step eagerly on `first_tokens` (that settles launch attributes and the allocator),
        capture the step (lengths advance on the device, slots and positions are derived from them inside
        the graph) and return (replay, logits of the first step); replay(tokens) -> logits runs the next
        step.  The sequences may grow up to `max_seq_len` tokens under this graph; it is meant for the
        exact-cache-free compressed path (backends whose forward reads host copies of the metadata cannot
        be captured)."""
        dev = self.device
        tokens = first_tokens.to(device=dev, dtype=torch.long).clone()
        lens = torch.tensor(self.seq_lens, dtype=torch.int32, device=dev)
        qsl = torch.arange(self.batch + 1, dtype=torch.int32)
        meta = StepMetadata(num_actual_tokens=self.batch, max_query_len=1, max_seq_len=max_seq_len, seq_lens=lens,
                            query_start_loc=qsl.to(dev), block_table=self.block_table,
                            slot_mapping=torch.zeros(self.batch, dtype=torch.long, device=dev),
                            seq_lens_cpu=torch.tensor(self.seq_lens, dtype=torch.int32), query_start_loc_cpu=qsl)

        def body():
            lens.add_(1)
            pos = (lens - 1).long()
            meta.slot_mapping.copy_(torch.gather(self.block_table.long(), 1, (pos // BLOCK)[:, None])[:, 0] * BLOCK
                                    + pos % BLOCK)
            return self.step(tokens, meta, positions=pos)

        host_lens = list(self.seq_lens)
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            first_logits = body().clone()
        torch.cuda.current_stream(dev).wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = body()
        # the graph's kernels address `lens` and the metadata tensors directly: they must live as long as it does
        state = {"steps": 1, "keep": (lens, meta, body)}

        def replay(new_tokens: torch.Tensor) -> torch.Tensor:
            tokens.copy_(new_tokens)
            graph.replay()
            state["steps"] += 1
            self.seq_lens = [n + state["steps"] for n in host_lens]
            return logits

        self.seq_lens = [n + 1 for n in host_lens]
        return replay, first_logits
