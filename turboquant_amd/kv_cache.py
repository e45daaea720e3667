"""Value group quantiser and the stand-alone TurboQuant KV cache object.

Mirrors turboquant/kv_cache.py of the reference: `ValueQuantized`,
`unpack_values`, `quantize_values`, `dequantize_values` (kv_cache.py:20-116) and
`TurboQuantKVCache` (kv_cache.py:119-349) with the same arguments, layouts and
dtypes; the arithmetic runs in libtq_hip.so.
"""

from __future__ import annotations

import math
from typing import NamedTuple, Optional

import torch

from . import _ffi
from .quantizer import ProdQuantized, TurboQuantProd


class ValueQuantized(NamedTuple):
    """Bit-packed group-quantised values."""
    data: torch.Tensor       # (..., n_tokens, d*bits/8) uint8
    scales: torch.Tensor     # (..., n_tokens, n_groups) input dtype
    zeros: torch.Tensor      # (..., n_tokens, n_groups) input dtype
    bits: int = 2


def unpack_values(vq: ValueQuantized) -> torch.Tensor:
    """One uint8 code per element (layout helper; kernels read the packed form)."""
    bits = vq.bits if len(vq) > 3 else 2
    packed = vq.data
    if bits not in (2, 4):
        return packed
    per_byte = 8 // bits
    fields = [(packed >> (bits * s)) & ((1 << bits) - 1) for s in range(per_byte)]
    return torch.stack(fields, dim=-1).reshape(*packed.shape[:-1], packed.shape[-1] * per_byte)


def quantize_values(v: torch.Tensor, bits: int = 2, group_size: int = 32) -> ValueQuantized:
    """Asymmetric per-group min/max quantisation of (..., seq_len, d) values to
    2, 4 or 8 bits, computed with the rounding of v's dtype."""
    _ffi.require_gpu(v, "v")
    d = v.shape[-1]
    assert d % group_size == 0, f"head_dim {d} must be divisible by group_size {group_size}"
    rows = v.reshape(-1, d)
    if rows.stride(-1) != 1 or (rows.shape[0] > 1 and rows.stride(0) < d):
        rows = rows.contiguous()
    n = rows.shape[0]
    stride = rows.stride(0) if n > 1 else d
    n_groups = d // group_size
    data = torch.empty(n, d * bits // 8, dtype=torch.uint8, device=v.device)
    scales = torch.empty(n, n_groups, dtype=v.dtype, device=v.device)
    zeros = torch.empty(n, n_groups, dtype=v.dtype, device=v.device)
    with torch.cuda.device(v.device):
        _ffi.check(_ffi.lib().tq_quantize_values(
            rows.data_ptr(), _ffi.dtype_tag(v.dtype), n, stride, d, group_size, bits, data.data_ptr(),
            scales.data_ptr(), zeros.data_ptr(), _ffi.stream_ptr(v.device)), "tq_quantize_values")
    lead = v.shape[:-1]
    return ValueQuantized(data=data.reshape(*lead, -1), scales=scales.reshape(*lead, n_groups),
                          zeros=zeros.reshape(*lead, n_groups), bits=bits)


def dequantize_values(vq: ValueQuantized, group_size: int = 32) -> torch.Tensor:
    """fp32 code * scale + zero, (..., seq_len, d)."""
    bits = vq.bits if len(vq) > 3 else 2
    data = _ffi.require_gpu(vq.data, "data").contiguous()
    scales, zeros = vq.scales.contiguous(), vq.zeros.contiguous()
    d = data.shape[-1] * 8 // bits
    n = data.numel() // data.shape[-1]
    out = torch.empty(*data.shape[:-1], d, dtype=torch.float32, device=data.device)
    with torch.cuda.device(data.device):
        _ffi.check(_ffi.lib().tq_dequant_values(
            data.data_ptr(), scales.data_ptr(), zeros.data_ptr(), _ffi.dtype_tag(scales.dtype), n, d, group_size, bits,
            out.data_ptr(), _ffi.stream_ptr(data.device)), "tq_dequant_values")
    return out


class TurboQuantKVCache:
    """Self-contained cache: the newest `buffer_size` tokens stay exact, older
    ones are TurboQuant keys + group-quantised values.  Tensors are
    (batch, heads, seq, head_dim)."""

    def __init__(self, head_dim: int, key_bits: int = 3, value_bits: int = 2, value_group_size: int = 32,
                 buffer_size: int = 128, device=None, dtype: torch.dtype = torch.float16, layer_idx: int = 0):
        self.head_dim = head_dim
        self.key_bits = key_bits
        self.value_bits = value_bits
        self.value_group_size = value_group_size
        self.buffer_size = buffer_size
        self.device = device or torch.device("cuda")
        self.dtype = dtype
        self.layer_idx = layer_idx
        self.key_quantizer = TurboQuantProd(dim=head_dim, bits=key_bits, device=self.device, seed=42 + layer_idx * 7)
        self.seq_len = 0
        self.key_quantized: Optional[ProdQuantized] = None
        self.value_quantized: Optional[ValueQuantized] = None
        self.key_buffer: Optional[torch.Tensor] = None
        self.value_buffer: Optional[torch.Tensor] = None

    def _compress(self, keys: torch.Tensor, values: torch.Tensor):
        kq = self.key_quantizer.quantize(keys)
        vq = quantize_values(values, bits=self.value_bits, group_size=self.value_group_size)
        if self.key_quantized is None:
            self.key_quantized, self.value_quantized = kq, vq
            return
        old_k, old_v = self.key_quantized, self.value_quantized
        self.key_quantized = ProdQuantized(
            mse_indices=torch.cat([old_k.mse_indices, kq.mse_indices], dim=-2),
            qjl_signs=torch.cat([old_k.qjl_signs, kq.qjl_signs], dim=-2),
            residual_norms=torch.cat([old_k.residual_norms, kq.residual_norms], dim=-1),
            norms=torch.cat([old_k.norms, kq.norms], dim=-1),
            mse_bits=kq.mse_bits)
        self.value_quantized = ValueQuantized(
            data=torch.cat([old_v.data, vq.data], dim=-2),
            scales=torch.cat([old_v.scales, vq.scales], dim=-2),
            zeros=torch.cat([old_v.zeros, vq.zeros], dim=-2),
            bits=self.value_bits)

    def prefill(self, keys: torch.Tensor, values: torch.Tensor):
        """All but the newest buffer_size tokens are compressed at once."""
        total = keys.shape[-2]
        self.seq_len = total
        if total <= self.buffer_size:
            self.key_buffer, self.value_buffer = keys, values
            return
        cut = total - self.buffer_size
        self.key_buffer, self.value_buffer = keys[..., cut:, :], values[..., cut:, :]
        self.key_quantized = self.value_quantized = None
        self._compress(keys[..., :cut, :], values[..., :cut, :])

    def append(self, key: torch.Tensor, value: torch.Tensor):
        """One decode token (batch, heads, 1, head_dim); the oldest buffered
        tokens spill into the compressed part once the buffer overflows."""
        self.seq_len += 1
        if self.key_buffer is None:
            self.key_buffer, self.value_buffer = key, value
        else:
            self.key_buffer = torch.cat([self.key_buffer, key], dim=-2)
            self.value_buffer = torch.cat([self.value_buffer, value], dim=-2)
        extra = self.key_buffer.shape[-2] - self.buffer_size
        if extra > 0:
            spill_k, spill_v = self.key_buffer[..., :extra, :], self.value_buffer[..., :extra, :]
            self.key_buffer, self.value_buffer = self.key_buffer[..., extra:, :], self.value_buffer[..., extra:, :]
            self._compress(spill_k, spill_v)

    def attention_scores(self, query: torch.Tensor, scale: float = None) -> torch.Tensor:
        """scale * <q, k> over [compressed ; buffer]: (batch, heads, n_q, seq_len)."""
        if scale is None:
            scale = 1.0 / math.sqrt(self.head_dim)
        pieces = []
        if self.key_quantized is not None:
            pieces.append(self.key_quantizer.attention_score(query, self.key_quantized) * scale)
        if self.key_buffer is not None:
            pieces.append(torch.matmul(query, self.key_buffer.transpose(-2, -1)) * scale)
        return torch.cat(pieces, dim=-1)

    def attend(self, attn_weights: torch.Tensor) -> torch.Tensor:
        """softmaxed weights (batch, heads, n_q, seq_len) -> (batch, heads, n_q, head_dim)."""
        result = None
        col = 0
        if self.value_quantized is not None:
            n_c = self.value_quantized.data.shape[-2]
            dense = dequantize_values(self.value_quantized, self.value_group_size)
            result = torch.matmul(attn_weights[..., col:col + n_c], dense)
            col += n_c
        if self.value_buffer is not None:
            n_b = self.value_buffer.shape[-2]
            part = torch.matmul(attn_weights[..., col:col + n_b], self.value_buffer)
            result = part if result is None else result + part
        return result

    def memory_bytes(self) -> dict:
        """Bytes held, counting norms / scales / zeros at 2 bytes each."""
        info = {"quantized_keys": 0, "quantized_values": 0, "buffer": 0, "total": 0}
        if self.key_quantized is not None:
            kq = self.key_quantized
            info["quantized_keys"] = (kq.mse_indices.nelement() + kq.qjl_signs.nelement()
                                      + 2 * kq.residual_norms.nelement() + 2 * kq.norms.nelement())
        if self.value_quantized is not None:
            vq = self.value_quantized
            info["quantized_values"] = vq.data.nelement() + 2 * vq.scales.nelement() + 2 * vq.zeros.nelement()
        for buf in (self.key_buffer, self.value_buffer):
            if buf is not None:
                info["buffer"] += 2 * buf.nelement()
        info["total"] = info["quantized_keys"] + info["quantized_values"] + info["buffer"]
        return info

    def get_seq_length(self) -> int:
        return self.seq_len
