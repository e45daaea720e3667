"""TurboQuant key quantisers on the MI355X kernels.

Mirrors turboquant/quantizer.py of the reference: `MSEQuantized`,
`ProdQuantized`, `_pack_indices`, `_unpack_indices`, `TurboQuantMSE` (Alg. 1,
quantizer.py:93-169) and `TurboQuantProd` (Alg. 2, quantizer.py:172-306) keep
their names, constructor arguments, buffers, tensor layouts and dtypes.  The
arithmetic runs in libtq_hip.so; inputs must be GPU tensors.
"""

from __future__ import annotations

import ctypes as C
import math
from typing import NamedTuple, Optional

import torch
import torch.nn.functional as F

from . import _ffi
from .codebook import get_codebook_tensors
from .rotation import generate_qjl_matrix, generate_rotation_matrix


class MSEQuantized(NamedTuple):
    """Output of TurboQuantMSE.quantize."""
    indices: torch.Tensor       # (..., packed_len) uint8 bit-packed indices
    norms: torch.Tensor         # (...,) L2 norms in the input dtype
    bits: int


class ProdQuantized(NamedTuple):
    """Output of TurboQuantProd.quantize."""
    mse_indices: torch.Tensor     # (..., packed_len) uint8
    qjl_signs: torch.Tensor       # (..., ceil(d/8)) uint8
    residual_norms: torch.Tensor  # (...,) fp32
    norms: torch.Tensor           # (...,) input dtype
    mse_bits: int


def _packing(bits: int):
    """(stored bits per index, indices per byte): 3-bit indices travel as nibbles."""
    if bits == 1:
        return 1, 8
    if bits == 2:
        return 2, 4
    if bits <= 4:
        return 4, 2
    return 8, 1


def _pack_indices(indices: torch.Tensor, bits: int) -> torch.Tensor:
    """Little-end-first packing of integer indices into bytes (layout helper;
    the quantise kernels emit this layout directly)."""
    width, per_byte = _packing(bits)
    if per_byte == 1:
        return indices.to(torch.uint8)
    d = indices.shape[-1]
    tail = (-d) % per_byte
    body = indices.to(torch.uint8)
    if tail:
        body = F.pad(body, (0, tail), value=0)
    lanes = body.reshape(*indices.shape[:-1], -1, per_byte).to(torch.int32)
    out = torch.zeros(lanes.shape[:-1], dtype=torch.int32, device=indices.device)
    for slot in range(per_byte):
        out |= lanes[..., slot] << (width * slot)
    return (out & 0xFF).to(torch.uint8)


def _unpack_indices(packed: torch.Tensor, bits: int, d: int) -> torch.Tensor:
    """Inverse of _pack_indices; returns int64 indices (..., d)."""
    width, per_byte = _packing(bits)
    if per_byte == 1:
        return packed.long()
    wide = packed.to(torch.int32)
    fields = [(wide >> (width * slot)) & ((1 << width) - 1) for slot in range(per_byte)]
    return torch.stack(fields, dim=-1).reshape(*packed.shape[:-1], -1)[..., :d].long()


def _rows(x: torch.Tensor):
    """View (..., d) as (n_vec, d) with a constant row stride, copying only if needed."""
    d = x.shape[-1]
    flat = x.reshape(-1, d)
    if flat.stride(-1) != 1 or (flat.shape[0] > 1 and flat.stride(0) < d):
        flat = flat.contiguous()
    return flat, (flat.stride(0) if flat.shape[0] > 1 else d)


class TurboQuantMSE(torch.nn.Module):
    """Algorithm 1: normalise, rotate by Pi, bucketise every coordinate against
    the Lloyd-Max thresholds, bit-pack.  De-quantise: centroid lookup, rotate
    back, rescale by the stored norm."""

    def __init__(self, dim: int, bits: int = 3, device=None, dtype: torch.dtype = torch.float32, seed: int = 42):
        super().__init__()
        self.dim = dim
        self.bits = bits
        self.n_clusters = 2 ** bits
        self.device = device or torch.device("cuda" if torch.cuda.is_available() else "cpu")

        self.register_buffer("Pi", generate_rotation_matrix(dim, self.device, dtype, seed=seed))
        centroids, boundaries = get_codebook_tensors(dim, bits, self.device, dtype)
        self.register_buffer("centroids", centroids)
        self.register_buffer("boundaries", boundaries)
        self.register_buffer("decision_boundaries", boundaries[1:-1].contiguous())
        # kernel-side companions (not part of the reference's state dict)
        self.register_buffer("_PiT", self.Pi.T.contiguous(), persistent=False)
        self._centroids_host = centroids.detach().float().cpu()
        self._splits = None           # (Pi, Pi^T[, S, S^T]) as bf16 term triples, built on first GPU use
        self._layer_cache = None      # (key, TqLayer): the descriptor of the buffers as they are now

    # -- library plumbing ---------------------------------------------------------
    def _layer(self, S: Optional[torch.Tensor] = None, ST: Optional[torch.Tensor] = None) -> _ffi.TqLayer:
        # One descriptor per state of the buffers: building it costs more host time than a decode call has to
        # spare (a dozen buffer look-ups and a library call), so it is kept until a buffer moves or is written.
        Pi, cen, thr = self.Pi, self.centroids, self.decision_boundaries
        state = (Pi.data_ptr(), Pi._version, cen.data_ptr(), cen._version, thr.data_ptr(), thr._version,
                 None if S is None else (S.data_ptr(), S._version, None if ST is None else ST.data_ptr()))
        cached = self._layer_cache
        if cached is not None and cached[0] == state:
            return cached[1]
        ly = self._build_layer(S, ST)
        self._layer_cache = (state, ly)
        return ly

    def _build_layer(self, S: Optional[torch.Tensor] = None, ST: Optional[torch.Tensor] = None) -> _ffi.TqLayer:
        if self.Pi.dtype != torch.float32:
            raise TypeError("the kernels need float32 rotation / codebook buffers")
        if self._PiT.device != self.Pi.device or self._PiT.data_ptr() == 0:
            self._PiT = self.Pi.T.contiguous()
            self._splits = None
        key = (self.Pi.data_ptr(), self.Pi._version, None if S is None else (S.data_ptr(), S._version))
        if self._splits is None or self._splits[0] != key:
            self._PiT = self.Pi.T.contiguous()
            # head_dim 128 / 256 have matrix-core quantise / de-quantise kernels; the head sizes of the wide-head decode
            # kernel (320 ... 704 in steps of 64) rotate their queries on the matrix cores, which takes Pi and S only
            wide = self.dim % 64 == 0 and 320 <= self.dim <= 704
            mk = _ffi.split_bf16x3 if (self.dim in (128, 256) or wide) else (lambda m: None)
            mkt = (lambda m: None) if wide else mk
            # head_dim 128: Pi^T also as fp6 terms, for the centroid contraction on the block-scaled MFMA
            fp6 = _ffi.split_fp6x5(self._PiT) if (self.dim == 128 and S is not None) else None
            self._splits = (key, (mk(self.Pi), mkt(self._PiT), None if S is None else mk(S),
                                  None if ST is None else mkt(ST), fp6))
        qc = None
        if S is not None:
            if getattr(self, "_query_consts", None) is None or self._query_consts[0] != key:
                self._query_consts = (key, (self.Pi.sum(dim=0).contiguous(), S.sum(dim=0).contiguous(),
                                            float(S.norm(dim=1).max())))
            qc = self._query_consts[1]
        return _ffi.make_layer(self.dim, self.bits, self.Pi, self._PiT, self.centroids, self.decision_boundaries,
                               S, ST, centroids_host=self._centroids_host, splits=self._splits[1], query_consts=qc)

    def quantize(self, x: torch.Tensor) -> MSEQuantized:
        """x (..., d) -> packed indices (..., d*eff/8) and norms (...) in x's dtype."""
        _ffi.require_gpu(x, "x")
        rows, stride = _rows(x)
        n = rows.shape[0]
        width, per_byte = _packing(self.bits)
        packed = torch.empty(n, (self.dim + per_byte - 1) // per_byte, dtype=torch.uint8, device=x.device)
        norms = torch.empty(n, dtype=x.dtype, device=x.device)
        ly = self._layer()
        with torch.cuda.device(x.device):
            _ffi.check(_ffi.lib().tq_quantize_keys(
                rows.data_ptr(), _ffi.dtype_tag(x.dtype), n, stride, C.byref(ly), packed.data_ptr(), None,
                norms.data_ptr(), None, None, None, 1, _ffi.stream_ptr(x.device)), "tq_quantize_keys")
        lead = x.shape[:-1]
        return MSEQuantized(indices=packed.reshape(*lead, -1), norms=norms.reshape(lead), bits=self.bits)

    def dequantize(self, q: MSEQuantized) -> torch.Tensor:
        """(centroids[idx] @ Pi) * norm, fp32 (..., d)."""
        idx = _ffi.require_gpu(q.indices, "indices").contiguous()
        norms = q.norms.contiguous()
        lead = norms.shape
        n = norms.numel()
        out = torch.empty(n, self.dim, dtype=torch.float32, device=idx.device)
        ly = self._layer()
        with torch.cuda.device(idx.device):
            _ffi.check(_ffi.lib().tq_dequant_keys(
                idx.data_ptr(), None, norms.data_ptr(), _ffi.dtype_tag(norms.dtype), None, n, C.byref(ly),
                out.data_ptr(), _ffi.stream_ptr(idx.device)), "tq_dequant_keys")
        return out.reshape(*lead, self.dim)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.dequantize(self.quantize(x))


class TurboQuantProd(torch.nn.Module):
    """Algorithm 2: (bits-1)-bit TurboQuantMSE, then a 1-bit QJL sketch
    sign(S r) of the residual r = x - x_mse with ||r||.  The inner-product
    estimate <q, x_mse> + ||r|| * sqrt(pi/2)/d * <S q, sign(S r)> is unbiased."""

    def __init__(self, dim: int, bits: int = 3, device=None, dtype: torch.dtype = torch.float32, seed: int = 42):
        super().__init__()
        self.dim = dim
        self.bits = bits
        self.device = device or torch.device("cuda" if torch.cuda.is_available() else "cpu")
        assert bits >= 2, "Inner product TurboQuant requires at least 2 bits (1 for MSE + 1 for QJL)"
        self.mse_quantizer = TurboQuantMSE(dim=dim, bits=bits - 1, device=self.device, dtype=dtype, seed=seed)
        self.register_buffer("S", generate_qjl_matrix(dim, self.device, dtype, seed=seed + 1000))
        self.register_buffer("_ST", self.S.T.contiguous(), persistent=False)
        self.qjl_scale = math.sqrt(math.pi / 2.0) / dim

    def _layer(self) -> _ffi.TqLayer:
        if self._ST.device != self.S.device or getattr(self, "_ST_version", None) != self.S._version:
            self._ST = self.S.T.contiguous()
            self._ST_version = self.S._version
        return self.mse_quantizer._layer(self.S, self._ST)

    def quantize(self, x: torch.Tensor) -> ProdQuantized:
        _ffi.require_gpu(x, "x")
        rows, stride = _rows(x)
        n, d = rows.shape[0], self.dim
        mb = self.bits - 1
        width, per_byte = _packing(mb)
        packed = torch.empty(n, (d + per_byte - 1) // per_byte, dtype=torch.uint8, device=x.device)
        signs = torch.empty(n, (d + 7) // 8, dtype=torch.uint8, device=x.device)
        norms = torch.empty(n, dtype=x.dtype, device=x.device)
        rnorms = torch.empty(n, dtype=torch.float32, device=x.device)
        ly = self._layer()
        with torch.cuda.device(x.device):
            _ffi.check(_ffi.lib().tq_quantize_keys(
                rows.data_ptr(), _ffi.dtype_tag(x.dtype), n, stride, C.byref(ly), packed.data_ptr(), signs.data_ptr(),
                norms.data_ptr(), rnorms.data_ptr(), None, None, 0, _ffi.stream_ptr(x.device)), "tq_quantize_keys")
        lead = x.shape[:-1]
        return ProdQuantized(mse_indices=packed.reshape(*lead, -1), qjl_signs=signs.reshape(*lead, -1),
                             residual_norms=rnorms.reshape(lead), norms=norms.reshape(lead), mse_bits=mb)

    def quantize_traced(self, x: torch.Tensor):
        """quantize() plus the two fp32 intermediates the packing consumes: the
        rotated unit vectors y and the projected residual p (both (..., d))."""
        _ffi.require_gpu(x, "x")
        rows, stride = _rows(x)
        n, d = rows.shape[0], self.dim
        mb = self.bits - 1
        width, per_byte = _packing(mb)
        dev = x.device
        packed = torch.empty(n, (d + per_byte - 1) // per_byte, dtype=torch.uint8, device=dev)
        signs = torch.empty(n, (d + 7) // 8, dtype=torch.uint8, device=dev)
        norms = torch.empty(n, dtype=x.dtype, device=dev)
        rnorms = torch.empty(n, dtype=torch.float32, device=dev)
        y = torch.empty(n, d, dtype=torch.float32, device=dev)
        p = torch.empty(n, d, dtype=torch.float32, device=dev)
        ly = self._layer()
        with torch.cuda.device(dev):
            _ffi.check(_ffi.lib().tq_quantize_keys(
                rows.data_ptr(), _ffi.dtype_tag(x.dtype), n, stride, C.byref(ly), packed.data_ptr(), signs.data_ptr(),
                norms.data_ptr(), rnorms.data_ptr(), y.data_ptr(), p.data_ptr(), 0, _ffi.stream_ptr(dev)),
                "tq_quantize_keys")
        lead = x.shape[:-1]
        code = ProdQuantized(mse_indices=packed.reshape(*lead, -1), qjl_signs=signs.reshape(*lead, -1),
                             residual_norms=rnorms.reshape(lead), norms=norms.reshape(lead), mse_bits=mb)
        return code, y.reshape(*lead, d), p.reshape(*lead, d)

    def dequantize(self, q: ProdQuantized) -> torch.Tensor:
        idx = _ffi.require_gpu(q.mse_indices, "mse_indices").contiguous()
        signs = q.qjl_signs.contiguous()
        norms = q.norms.contiguous()
        rnorms = q.residual_norms.contiguous().float()
        lead = norms.shape
        n = norms.numel()
        out = torch.empty(n, self.dim, dtype=torch.float32, device=idx.device)
        ly = self._layer()
        with torch.cuda.device(idx.device):
            _ffi.check(_ffi.lib().tq_dequant_keys(
                idx.data_ptr(), signs.data_ptr(), norms.data_ptr(), _ffi.dtype_tag(norms.dtype), rnorms.data_ptr(), n,
                C.byref(ly), out.data_ptr(), _ffi.stream_ptr(idx.device)), "tq_dequant_keys")
        return out.reshape(*lead, self.dim)

    def attention_score(self, query: torch.Tensor, quantized_key: ProdQuantized) -> torch.Tensor:
        """query (..., n_q, d), keys (..., n_k, ...) -> raw logits (..., n_q, n_k), fp32,
        without the 1/sqrt(d) factor."""
        _ffi.require_gpu(query, "query")
        d = self.dim
        lead = torch.broadcast_shapes(query.shape[:-2], quantized_key.norms.shape[:-1])
        n_q, n_k = query.shape[-2], quantized_key.norms.shape[-1]
        q = query.expand(*lead, n_q, d).contiguous()
        idx = quantized_key.mse_indices.expand(*lead, n_k, quantized_key.mse_indices.shape[-1]).contiguous()
        signs = quantized_key.qjl_signs.expand(*lead, n_k, quantized_key.qjl_signs.shape[-1]).contiguous()
        norms = quantized_key.norms.expand(*lead, n_k).contiguous()
        rnorms = quantized_key.residual_norms.expand(*lead, n_k).contiguous().float()
        batch = int(math.prod(lead)) if len(lead) else 1
        scores = torch.empty(*lead, n_q, n_k, dtype=torch.float32, device=q.device)
        work = torch.empty(2 * batch * n_q * d, dtype=torch.float32, device=q.device)
        ly = self._layer()
        with torch.cuda.device(q.device):
            _ffi.check(_ffi.lib().tq_score(
                q.data_ptr(), _ffi.dtype_tag(q.dtype), batch, n_q, idx.data_ptr(), signs.data_ptr(), norms.data_ptr(),
                _ffi.dtype_tag(norms.dtype), rnorms.data_ptr(), n_k, C.byref(ly), scores.data_ptr(), work.data_ptr(),
                _ffi.stream_ptr(q.device)), "tq_score")
        return scores

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.dequantize(self.quantize(x))
