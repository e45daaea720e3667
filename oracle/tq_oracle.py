"""CPU oracle for the TurboQuant KV-cache hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU with torch/numpy, the algorithm the reference
implements for key quantisation (rotation -> Lloyd-Max bucketise -> bit-pack ->
QJL residual sketch), value group quantisation, the asymmetric score estimator
and the de-quantise-everything decode attention.  It exists to check the HIP
kernels; nothing in the shipped package may import it.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  Pinning status (what proves each function right):

* ``lloyd_max_codebook``      : the nine codebook JSONs the reference ships
                                (known answers) + the b=1 closed form.
* ``pack_indices`` / ``unpack_indices`` / ``pack_signs`` / ``unpack_signs`` :
                                closed form ``sum idx_j << (eff*j)`` checked by
                                brute force over every byte value + round trip.
* ``bucketize``               : brute-force count of thresholds below y.
* ``rotation_matrix`` / ``qjl_matrix`` : library routines (seeded randn + QR);
                                orthogonality and sign-convention invariants.
* ``mse_quantize`` .. ``attention_score``, ``quantize_values`` ..,
  ``hybrid_attention``        : golden vectors written by the reference itself
                                (``tests/golden/*.npz``) plus algebraic
                                identities (dense matmul on small inputs,
                                |v - deq| <= scale/2, softmax/SDPA equivalence).
* ``RingModel`` / ``CaptureModel`` : bookkeeping invariants and the golden
                                token-routing trace.

All tensors are torch CPU tensors.  Arithmetic follows the dtypes torch would
produce on the reference's code path (bf16 inputs keep bf16 norms and bf16
per-op rounding in the value quantiser; everything after ``.float()`` is fp32).
"""

from __future__ import annotations

import math
from typing import Dict, List, NamedTuple, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F
from scipy import integrate, special

# --------------------------------------------------------------------------
# codebook  (reference: turboquant/codebook.py:21-143)
# --------------------------------------------------------------------------


def sphere_coord_pdf(x, d: int):
    """Density of one coordinate of a uniform point on S^{d-1}
    (reference codebook.py:21-36): C_d * (1-x^2)^((d-3)/2) with x clipped
    1e-15 away from +-1, evaluated through logs."""
    if d <= 2:
        raise ValueError(f"Dimension d={d} too small, need d >= 3")
    x = np.clip(np.asarray(x, dtype=np.float64), -1 + 1e-15, 1 - 1e-15)
    log_c = special.gammaln(d / 2.0) - 0.5 * np.log(np.pi) - special.gammaln((d - 1) / 2.0)
    return np.exp(log_c + ((d - 3) / 2.0) * np.log(1 - x ** 2))


def _pdf_scalar(t: float, d: int) -> float:
    return sphere_coord_pdf(np.array([t]), d)[0]


def _cell_mean(lo: float, hi: float, d: int) -> float:
    # reference codebook.py:39-46 -- ratio of two default-tolerance quad calls
    num, _ = integrate.quad(lambda t: t * _pdf_scalar(t, d), lo, hi)
    den, _ = integrate.quad(lambda t: _pdf_scalar(t, d), lo, hi)
    if den < 1e-30:
        return (lo + hi) / 2.0
    return num / den


def _edges_of(cent: np.ndarray) -> np.ndarray:
    n = len(cent)
    e = np.zeros(n + 1)
    e[0], e[-1] = -1.0, 1.0
    for i in range(n - 1):
        e[i + 1] = (cent[i] + cent[i + 1]) / 2.0
    return e


def _distortion(cent: np.ndarray, d: int) -> float:
    # reference codebook.py:49-65
    e = _edges_of(cent)
    total = 0.0
    for i in range(len(cent)):
        c = cent[i]
        v, _ = integrate.quad(lambda t: (t - c) ** 2 * _pdf_scalar(t, d), e[i], e[i + 1])
        total += v
    return total


def lloyd_max_codebook(d: int, bits: int, max_iter: int = 200, tol: float = 1e-12) -> Dict:
    """Early-stopped Lloyd-Max iteration (reference codebook.py:68-143).

    Initial centroids sit at the quantile mid-points of a 10 000-point
    rectangle-rule CDF; each sweep recomputes mid-point edges, conditional
    means and the distortion; it stops when the distortion moves by < tol."""
    k = 2 ** bits
    grid = np.linspace(-1 + 1e-10, 1 - 1e-10, 10000)
    cdf = np.cumsum(sphere_coord_pdf(grid, d)) * (grid[1] - grid[0])
    cdf /= cdf[-1]
    q_edges = np.linspace(0, 1, k + 1)
    cent = np.zeros(k)
    for i in range(k):
        mid = (q_edges[i] + q_edges[i + 1]) / 2.0
        pos = min(int(np.searchsorted(cdf, mid)), len(grid) - 1)
        cent[i] = grid[pos]

    last = float("inf")
    cost = float("nan")
    for _ in range(max_iter):
        e = _edges_of(cent)
        nxt = np.zeros(k)
        for i in range(k):
            nxt[i] = _cell_mean(e[i], e[i + 1], d)
        cost = _distortion(nxt, d)
        cent = nxt
        if abs(last - cost) < tol:
            break
        last = cost

    e = _edges_of(cent)
    return {
        "centroids": cent.tolist(),
        "boundaries": e.tolist(),
        "mse_per_coord": float(cost),
        "mse_total": float(cost * d),
        "d": d,
        "bits": bits,
    }


def codebook_tensors(cb: Dict, dtype=torch.float32) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(centroids, boundaries, interior thresholds) as the reference builds them
    (codebook.py:176-181, quantizer.py:121-127)."""
    cent = torch.tensor(cb["centroids"], dtype=dtype)
    edges = torch.tensor(cb["boundaries"], dtype=dtype)
    return cent, edges, edges[1:-1].contiguous()


# --------------------------------------------------------------------------
# rotation / sketch matrices  (reference: turboquant/rotation.py:17-66)
# --------------------------------------------------------------------------


def rotation_matrix(d: int, seed: int = 42) -> torch.Tensor:
    """Haar orthogonal Pi: QR of a seeded CPU Gaussian, columns re-signed by
    sign(diag R) (rotation.py:17-40)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    gauss = torch.randn(d, d, generator=g, dtype=torch.float32)
    q, r = torch.linalg.qr(gauss)
    return q * torch.sign(torch.diag(r)).unsqueeze(0)


def qjl_matrix(d: int, seed: int = 12345) -> torch.Tensor:
    """Gaussian sketch matrix S, d x d (rotation.py:43-56)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return torch.randn(d, d, generator=g, dtype=torch.float32)


# --------------------------------------------------------------------------
# packing  (reference: turboquant/quantizer.py:38-90, 214-229)
# --------------------------------------------------------------------------


def packing_params(bits: int) -> Tuple[int, int]:
    """(effective bits per stored index, indices per byte); 3-bit indices are
    stored as nibbles, >4 bits as raw bytes (quantizer.py:51-59)."""
    if bits == 1:
        return 1, 8
    if bits == 2:
        return 2, 4
    if bits <= 4:
        return 4, 2
    return 8, 1


def pack_indices(idx: torch.Tensor, bits: int) -> torch.Tensor:
    eff, per = packing_params(bits)
    if per == 1:
        return idx.to(torch.uint8)
    a = idx.to(torch.int64).numpy()
    d = a.shape[-1]
    pad = (-d) % per
    if pad:
        a = np.concatenate([a, np.zeros(a.shape[:-1] + (pad,), dtype=a.dtype)], axis=-1)
    a = a.reshape(a.shape[:-1] + (-1, per))
    out = np.zeros(a.shape[:-1], dtype=np.int64)
    for j in range(per):
        out |= (a[..., j] & 0xFF) << (eff * j)
    return torch.from_numpy((out & 0xFF).astype(np.uint8))


def unpack_indices(packed: torch.Tensor, bits: int, d: int) -> torch.Tensor:
    eff, per = packing_params(bits)
    if per == 1:
        return packed.long()
    a = packed.numpy().astype(np.int64)
    parts = [(a >> (eff * j)) & ((1 << eff) - 1) for j in range(per)]
    out = np.stack(parts, axis=-1).reshape(a.shape[:-1] + (-1,))
    return torch.from_numpy(out[..., :d].copy())


def pack_signs(projected: torch.Tensor) -> torch.Tensor:
    """bit j of byte k = (projected[8k+j] > 0), strict (quantizer.py:214-222)."""
    b = (projected > 0).numpy().astype(np.int64)
    d = b.shape[-1]
    pad = (-d) % 8
    if pad:
        b = np.concatenate([b, np.zeros(b.shape[:-1] + (pad,), dtype=b.dtype)], axis=-1)
    b = b.reshape(b.shape[:-1] + (-1, 8))
    out = np.zeros(b.shape[:-1], dtype=np.int64)
    for j in range(8):
        out |= b[..., j] << j
    return torch.from_numpy(out.astype(np.uint8))


def unpack_signs(packed: torch.Tensor, d: int) -> torch.Tensor:
    """-> fp32 tensor of -1/+1, length d (quantizer.py:224-229)."""
    a = packed.numpy().astype(np.int64)
    bits = np.stack([(a >> j) & 1 for j in range(8)], axis=-1).reshape(a.shape[:-1] + (-1,))
    return torch.from_numpy((2.0 * bits[..., :d] - 1.0).astype(np.float32))


def bucketize(y: torch.Tensor, thresholds: torch.Tensor) -> torch.Tensor:
    """idx = number of thresholds t for which `y <= t` is false: thresholds
    strictly below y, a tie falling in the lower bucket, and a NaN landing in
    the top bucket (lower-bound search of torch.searchsorted, quantizer.py:144)."""
    return (~(y.unsqueeze(-1) <= thresholds)).sum(dim=-1)


# --------------------------------------------------------------------------
# key quantiser  (reference: turboquant/quantizer.py:129-165, 231-302)
# --------------------------------------------------------------------------


class KeyCode(NamedTuple):
    mse_indices: torch.Tensor     # uint8 (..., d*eff/8)
    qjl_signs: torch.Tensor       # uint8 (..., ceil(d/8))
    residual_norms: torch.Tensor  # fp32 (...)
    norms: torch.Tensor           # input dtype (...)
    mse_bits: int
    y: torch.Tensor               # fp32 rotated unit vectors  (debug / parity input)
    p: torch.Tensor               # fp32 projected residual    (debug / parity input)


class KeyParams(NamedTuple):
    Pi: torch.Tensor
    S: torch.Tensor
    centroids: torch.Tensor
    thresholds: torch.Tensor
    mse_bits: int

    @property
    def d(self) -> int:
        return self.Pi.shape[0]

    @property
    def qjl_scale(self) -> float:
        return math.sqrt(math.pi / 2.0) / self.Pi.shape[0]


def make_key_params(d: int, key_bits: int, codebook: Dict, seed: int = 42) -> KeyParams:
    """Pi from `seed`, S from `seed + 1000`, (key_bits-1)-bit codebook
    (quantizer.py:186-212)."""
    assert key_bits >= 2
    cent, _, thr = codebook_tensors(codebook)
    return KeyParams(rotation_matrix(d, seed), qjl_matrix(d, seed + 1000), cent, thr, key_bits - 1)


def mse_quantize(x: torch.Tensor, prm: KeyParams):
    """Alg. 1 forward (quantizer.py:129-149).  Norm and normalisation happen in
    the input dtype; the rotation in fp32."""
    norms = x.norm(dim=-1)
    unit = x / (norms.unsqueeze(-1) + 1e-10)
    y = torch.matmul(unit.float(), prm.Pi.T)
    idx = bucketize(y, prm.thresholds)
    return pack_indices(idx, prm.mse_bits), norms, y, idx


def mse_dequantize(packed: torch.Tensor, norms: torch.Tensor, prm: KeyParams) -> torch.Tensor:
    """centroids[idx] @ Pi, rescaled by the stored norm (quantizer.py:151-165)."""
    idx = unpack_indices(packed, prm.mse_bits, prm.d)
    return torch.matmul(prm.centroids[idx], prm.Pi) * norms.unsqueeze(-1)


def prod_quantize(x: torch.Tensor, prm: KeyParams) -> KeyCode:
    """Alg. 2 forward (quantizer.py:231-257): MSE stage, residual in the
    ORIGINAL space, its norm, sign sketch of S r."""
    packed, norms, y, _ = mse_quantize(x, prm)
    x_hat = mse_dequantize(packed, norms, prm)
    resid = x - x_hat
    rnorm = resid.norm(dim=-1)
    p = torch.matmul(resid.float(), prm.S.T)
    return KeyCode(packed, pack_signs(p), rnorm, norms, prm.mse_bits, y, p)


def prod_dequantize(code, prm: KeyParams) -> torch.Tensor:
    """x_mse + (signs @ S) * qjl_scale * ||r|| (quantizer.py:259-272)."""
    x_mse = mse_dequantize(code.mse_indices, code.norms, prm)
    sg = unpack_signs(code.qjl_signs, prm.d)
    x_qjl = torch.matmul(sg, prm.S) * (prm.qjl_scale * code.residual_norms.unsqueeze(-1))
    return x_mse + x_qjl


def attention_score(query: torch.Tensor, code, prm: KeyParams) -> torch.Tensor:
    """Raw logits q.k_mse + (q S^T).signs * qjl_scale * ||r||, no 1/sqrt(d)
    (quantizer.py:274-302).  query (..., n_q, d) -> (..., n_q, n_k)."""
    k_mse = mse_dequantize(code.mse_indices, code.norms, prm)
    s_mse = torch.matmul(query.float(), k_mse.float().transpose(-2, -1))
    q_sk = torch.matmul(query.float(), prm.S.T)
    sg = unpack_signs(code.qjl_signs, prm.d)
    s_qjl = torch.matmul(q_sk, sg.transpose(-2, -1))
    s_qjl = s_qjl * (prm.qjl_scale * code.residual_norms.unsqueeze(-2))
    return s_mse + s_qjl.to(s_mse.dtype)


def fused_score(query: torch.Tensor, code, prm: KeyParams) -> torch.Tensor:
    """The rotated-query form of the same estimator
    (triton_kernels.py:49-53,138): n * sum_j (q Pi^T)_j c[idx_j]
    + qjl_scale * rho * sum_j (q S^T)_j sigma_j, accumulated in float64 so it
    can referee between fp32 formulations."""
    q64 = query.double()
    q_rot = q64 @ prm.Pi.double().T
    q_sk = q64 @ prm.S.double().T
    idx = unpack_indices(code.mse_indices, prm.mse_bits, prm.d)
    c = prm.centroids.double()[idx]
    sg = unpack_signs(code.qjl_signs, prm.d).double()
    mse = (q_rot @ c.transpose(-2, -1)) * code.norms.double().unsqueeze(-2)
    qjl = (q_sk @ sg.transpose(-2, -1)) * (prm.qjl_scale * code.residual_norms.double().unsqueeze(-2))
    return mse + qjl


# --------------------------------------------------------------------------
# value group quantiser  (reference: turboquant/kv_cache.py:28-116)
# --------------------------------------------------------------------------


class ValueCode(NamedTuple):
    data: torch.Tensor     # uint8 (..., T, d*bits/8)
    scales: torch.Tensor   # input dtype (..., T, d/gs)
    zeros: torch.Tensor    # input dtype (..., T, d/gs)
    bits: int


def quantize_values(v: torch.Tensor, bits: int = 2, group_size: int = 32) -> ValueCode:
    """Asymmetric min/max group quantiser; every op rounds to the input dtype
    because torch computes it there (kv_cache.py:45-98)."""
    d = v.shape[-1]
    assert d % group_size == 0
    g = v.reshape(*v.shape[:-1], d // group_size, group_size)
    lo = g.min(dim=-1, keepdim=True).values
    hi = g.max(dim=-1, keepdim=True).values
    levels = 2 ** bits - 1
    scale = ((hi - lo) / levels).clamp(min=1e-10)
    code = ((g - lo) / scale).round().clamp(0, levels).to(torch.uint8)
    flat = code.reshape(*v.shape[:-1], d).numpy().astype(np.uint8)
    if bits == 2:
        q = flat.reshape(flat.shape[:-1] + (d // 4, 4))
        flat = q[..., 0] | (q[..., 1] << 2) | (q[..., 2] << 4) | (q[..., 3] << 6)
    elif bits == 4:
        q = flat.reshape(flat.shape[:-1] + (d // 2, 2))
        flat = q[..., 0] | (q[..., 1] << 4)
    return ValueCode(torch.from_numpy(np.ascontiguousarray(flat)), scale.squeeze(-1), lo.squeeze(-1), bits)


def unpack_values(data: torch.Tensor, bits: int) -> torch.Tensor:
    """uint8 codes, one per element (kv_cache.py:28-42)."""
    a = data.numpy()
    if bits == 2:
        parts = [(a >> s) & 0x3 for s in (0, 2, 4, 6)]
    elif bits == 4:
        parts = [(a >> s) & 0xF for s in (0, 4)]
    else:
        return data
    out = np.stack(parts, axis=-1).reshape(a.shape[:-1] + (-1,))
    return torch.from_numpy(out.astype(np.uint8))


def dequantize_values(code, group_size: int = 32) -> torch.Tensor:
    """fp32(code) * scale + zero, promoted by torch to fp32 (kv_cache.py:101-116)."""
    raw = unpack_values(code.data, code.bits).float()
    d = raw.shape[-1]
    raw = raw.reshape(*raw.shape[:-1], d // group_size, group_size)
    out = raw * code.scales.unsqueeze(-1) + code.zeros.unsqueeze(-1)
    return out.reshape(*out.shape[:-2], d)


# --------------------------------------------------------------------------
# decode attention  (reference: turboquant/score.py:29-173)
# --------------------------------------------------------------------------

MIN_HISTORY = 16  # score.py:26


def dense_gqa_attention(query: torch.Tensor, keys: torch.Tensor, values: torch.Tensor,
                        num_kv_heads: int, scale: float) -> torch.Tensor:
    """fp32 softmax(scale q k^T) v with KV head h serving query heads
    h*G .. h*G+G-1, no mask, result cast to the query dtype (score.py:138-173).
    query (T,Hq,d); keys/values (Hkv,N,d)."""
    t, hq, d = query.shape
    grp = hq // num_kv_heads
    if hq != num_kv_heads * grp:
        raise ValueError(f"Incompatible GQA shapes: Q={hq}, H_kv={num_kv_heads}")
    q = query.float().reshape(t, num_kv_heads, grp, d).permute(1, 2, 0, 3)   # (H,G,T,d)
    k = keys.float()
    v = values.float()
    logits = torch.matmul(q, k.unsqueeze(1).transpose(-2, -1)) * scale      # (H,G,T,N)
    w = F.softmax(logits, dim=-1)
    out = torch.matmul(w, v.unsqueeze(1))                                    # (H,G,T,d)
    return out.permute(2, 0, 1, 3).reshape(t, hq, d).to(query.dtype)


def hybrid_attention(query: torch.Tensor, key_code, value_code, n_hist: int, prm: KeyParams,
                     num_kv_heads: int, recent_k: Optional[torch.Tensor], recent_v: Optional[torch.Tensor],
                     scale: Optional[float] = None, value_group_size: int = 32) -> torch.Tensor:
    """compute_hybrid_attention (score.py:29-135): de-quantise the whole
    history, append the exact recent tokens, run dense attention.  History is
    ignored below 16 tokens; with nothing to attend to the result is zeros.
    key_code / value_code hold (Hkv, N, ...) tensors; recent_* are (R,Hkv,d)."""
    t, hq, d = query.shape
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    has_hist = key_code is not None and n_hist >= MIN_HISTORY
    has_recent = recent_k is not None and recent_k.shape[0] > 0
    if not has_hist and not has_recent:
        return torch.zeros(t, hq, d, dtype=query.dtype)
    parts_k: List[torch.Tensor] = []
    parts_v: List[torch.Tensor] = []
    if has_hist:
        parts_k.append(prod_dequantize(key_code, prm).float())
        parts_v.append(dequantize_values(value_code, value_group_size).float())
    if has_recent:
        parts_k.append(recent_k.transpose(0, 1).float())
        parts_v.append(recent_v.transpose(0, 1).float())
    return dense_gqa_attention(query, torch.cat(parts_k, dim=1), torch.cat(parts_v, dim=1), num_kv_heads, scale)


# --------------------------------------------------------------------------
# write-side policy  (reference: turboquant/capture.py:75-131, 170-240)
# --------------------------------------------------------------------------


class RingModel:
    """List-based model of the exact-token ring (capture.py:21-131): holds at
    most `capacity` token ids; a write that finds the ring full first drains
    everything that is in it."""

    def __init__(self, capacity: int):
        self.capacity = capacity
        self.items: List[int] = []
        self.total_written = 0

    def write(self, tokens: List[int]) -> Optional[List[int]]:
        spilled: List[int] = []
        for tok in tokens:
            if len(self.items) >= self.capacity:
                spilled.extend(self.items)
                self.items = []
            self.items.append(tok)
        self.total_written += len(tokens)
        return spilled or None

    def drain(self) -> Optional[List[int]]:
        if not self.items:
            return None
        out, self.items = self.items, []
        return out


class CaptureModel:
    """Token routing of KVCaptureEngine (capture.py:134-240): prefill compresses
    all but the last `capacity` tokens and DISCARDS whatever the ring spills
    while taking the tail (capture.py:176,180); decode spills go to the store."""

    def __init__(self, capacity: int = 128):
        self.ring = RingModel(capacity)
        self.chunks: List[List[int]] = []

    def ingest_prefill(self, tokens: List[int]):
        cap = self.ring.capacity
        if len(tokens) <= cap:
            self.ring.write(tokens)
        else:
            self.chunks.append(tokens[:len(tokens) - cap])
            self.ring.write(tokens[len(tokens) - cap:])

    def ingest_decode(self, tokens: List[int]):
        spilled = self.ring.write(tokens)
        if spilled is not None:
            self.chunks.append(spilled)

    def flush(self):
        got = self.ring.drain()
        if got is not None:
            self.chunks.append(got)

    @property
    def compressed(self) -> List[int]:
        return [t for c in self.chunks for t in c]
