"""ctypes binding of libtq_hip.so (declarations: include/tq_hip.h).

The library is loaded on first use.  There is no fallback: if the shared object
is missing or a tensor is not on a GPU the call raises.
"""

from __future__ import annotations

import ctypes as C
import math
import os
from typing import Optional

import torch

TQ_F32, TQ_F16, TQ_BF16 = 0, 1, 2
TQ_PAGE_TOKENS = 16
TQ_MAX_TERMS = 15
ABI_VERSION = 2

# TQ_HIP_LIBRARY overrides the in-tree library (e.g. to compare two builds)
_LIB_PATH = os.environ.get("TQ_HIP_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtq_hip.so")
_lib: Optional[C.CDLL] = None

_ERR = {-1: "TQ_EINVAL (a size, stride or enum is out of range)",
        -2: "TQ_EUNSUPPORTED (no kernel for this shape / bit-width)",
        -3: "TQ_ENULL (a required pointer is NULL)",
        -4: "TQ_ETOOBIG (the call needs more scratch than the library's static area holds; use the workspace form)"}


class TqLayer(C.Structure):
    _fields_ = [
        ("d", C.c_int32), ("mse_bits", C.c_int32),
        ("Pi", C.c_void_p), ("PiT", C.c_void_p), ("S", C.c_void_p), ("ST", C.c_void_p),
        ("centroids", C.c_void_p), ("thresholds", C.c_void_p),
        ("qjl_scale", C.c_float),
        ("Pi_split", C.c_void_p), ("PiT_split", C.c_void_p), ("S_split", C.c_void_p), ("ST_split", C.c_void_p),
        ("Pi_colsum", C.c_void_p), ("S_colsum", C.c_void_p), ("S_rownorm_max", C.c_float),
        ("PiT_fp6", C.c_void_p), ("PiT_fp6_scale", C.c_void_p),
        ("n_terms", C.c_int32),
        ("term_mask", C.c_int32 * TQ_MAX_TERMS),
        ("term_coef", C.c_float * TQ_MAX_TERMS),
        ("term_const", C.c_float),
    ]


class TqPageLayout(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "d", "mse_bits", "value_bits", "group_size", "dtype", "key_lane_major",
        "off_keys", "off_meta", "off_vdata", "off_vscale", "off_vzero", "page_bytes")]


_vp, _i, _i64, _f = C.c_void_p, C.c_int, C.c_int64, C.c_float
_SIGNATURES = {
    "tq_version": (C.c_int, []),
    "tq_layer_fill_terms": (C.c_int, [C.POINTER(TqLayer), C.POINTER(C.c_float)]),
    "tq_page_layout_init": (C.c_int, [C.POINTER(TqPageLayout), _i, _i, _i, _i, _i]),
    "tq_bucketize_pack": (C.c_int, [_vp, _i64, _i, _vp, _i, _vp, _vp]),
    "tq_sign_pack": (C.c_int, [_vp, _i64, _i, _vp, _vp]),
    "tq_quantize_keys": (C.c_int, [_vp, _i, _i64, _i64, C.POINTER(TqLayer), _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "tq_quantize_values": (C.c_int, [_vp, _i, _i64, _i64, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "tq_dequant_keys": (C.c_int, [_vp, _vp, _vp, _i, _vp, _i64, C.POINTER(TqLayer), _vp, _vp]),
    "tq_dequant_values": (C.c_int, [_vp, _vp, _vp, _i, _i64, _i, _i, _i, _vp, _vp]),
    "tq_score": (C.c_int, [_vp, _i, _i64, _i64, _vp, _vp, _vp, _i, _vp, _i64, C.POINTER(TqLayer), _vp, _vp, _vp]),
    "tq_rotate_query": (C.c_int, [_vp, _i, _i64, C.POINTER(TqLayer), _vp, _vp, _vp]),
    "tq_append_kv_paged": (C.c_int, [_vp, _vp, _i, _i, _i, _i, _i64, _i64, _i64, _vp, _vp, _i,
                                     C.POINTER(TqLayer), C.POINTER(TqPageLayout), _vp, _i64, _vp]),
    "tq_append_kv_ragged": (C.c_int, [_vp, _vp, _i, _i, _i, _i, _i64, _i64, _vp, _vp, _vp, _vp, _i,
                                      C.POINTER(TqLayer), C.POINTER(TqPageLayout), _vp, _i64, _vp]),
    "tq_append_kv_from_blocks": (C.c_int, [_vp, _vp, _i, _i, _i, _i, _i64, _i64, _i64, _vp, _i, _vp, _vp, _vp, _i,
                                           C.POINTER(TqLayer), C.POINTER(TqPageLayout), _vp, _i64, _vp]),
    "tq_pool_export": (C.c_int, [_vp, _i64, _i, _vp, _i, C.POINTER(TqPageLayout), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "tq_decode_page_kernel": (C.c_int, [C.POINTER(TqLayer), C.POINTER(TqPageLayout)]),
    "tq_decode_workspace_bytes": (C.c_size_t, [_i, _i, _i, _i]),
    "tq_decode_attn_paged": (C.c_int, [_vp, _i, _i, _i, _i, _vp, _i64, _vp, _i, _vp, _f, C.POINTER(TqLayer),
                                       C.POINTER(TqPageLayout), _vp, _vp, _i, _i64, _i64, _i64, _vp, _vp, _vp, _i, _vp]),
    "tq_decode_attn_paged_stages": (C.c_int, [_vp, _i, _i, _i, _i, _vp, _i64, _vp, _i, _vp, _f, C.POINTER(TqLayer),
                                              C.POINTER(TqPageLayout), _vp, _vp, _i, _i64, _i64, _i64, _vp, _vp, _vp, _i,
                                              _i, _vp]),
    "tq_decode_attn_paged_ring": (C.c_int, [_vp, _i, _i, _i, _i, _vp, _i64, _vp, _i, _vp, _f, C.POINTER(TqLayer),
                                            C.POINTER(TqPageLayout), _vp, _vp, _i64, _i64, _i64, _i, _vp, _vp, _i, _vp]),
    "tq_decode_attn_paged_noalloc": (C.c_int, [_vp, _i, _i, _i, _i, _vp, _i64, _vp, _i, _vp, _f, C.POINTER(TqLayer),
                                               C.POINTER(TqPageLayout), _vp, _vp, _i, _i64, _i64, _i64, _vp, _vp, _i, _vp]),
    "tq_decode_noalloc_bytes": (C.c_size_t, [_i, _i, _i, _i, C.POINTER(TqLayer)]),
    "tq_noalloc_init": (C.c_int, []),
    "tq_decode_merge": (C.c_int, [_vp, _i64, _i, _i, _i, _vp, _vp]),
    "tq_time_next_page_kernel": (None, [_vp, _vp]),
    "tq_time_next_key_kernel": (None, [_vp, _vp]),
    "tq_set_option": (C.c_int, [C.c_char_p, _i64]),
    "tq_stream_read": (C.c_int, [_vp, C.c_size_t, _i, _i, _vp, _vp]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def library_path() -> str:
    return _LIB_PATH


def lib() -> C.CDLL:
    """Load libtq_hip.so (once) and attach the prototypes."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python -m turboquant_amd.build` "
                "(there is no CPU or PyTorch fallback for the TurboQuant kernels)")
        handle = C.CDLL(_LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        got = handle.tq_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"libtq_hip.so has ABI version {got}, the bindings expect {ABI_VERSION}")
        _lib = handle
    return _lib


def check(rc: int, what: str):
    if rc == 0:
        return
    if rc < 0:
        raise ValueError(f"{what}: {_ERR.get(rc, rc)}")
    raise RuntimeError(f"{what}: HIP error {rc}")


def dtype_tag(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return TQ_F32
    if dt == torch.float16:
        return TQ_F16
    if dt == torch.bfloat16:
        return TQ_BF16
    raise TypeError(f"TurboQuant kernels take float32, float16 or bfloat16 tensors, not {dt}")


def require_gpu(t: torch.Tensor, name: str) -> torch.Tensor:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} lives on {t.device}: the TurboQuant kernels run on the GPU only and have no CPU path")
    return t


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device) -> int:
    """hipStream_t of torch's current stream on `device` (the raw accessor when this torch has it: no Stream object)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class on_device:
    """`with on_device(dev):` - makes `dev` the current device for the library call inside, and costs nothing
    when it already is (the usual case: one process per GPU)."""
    __slots__ = ("dev", "ctx")

    def __init__(self, dev):
        self.dev, self.ctx = dev, None

    def __enter__(self):
        if self.dev.index is None or torch.cuda.current_device() != self.dev.index:
            self.ctx = torch.cuda.device(self.dev)
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def walsh_terms(centroids_host: torch.Tensor, mse_bits: int, layer: TqLayer):
    arr = (C.c_float * (1 << mse_bits))(*[float(v) for v in centroids_host.tolist()])
    layer.mse_bits = mse_bits
    check(lib().tq_layer_fill_terms(C.byref(layer), arr), "tq_layer_fill_terms")


def make_layer(d: int, mse_bits: int, Pi: torch.Tensor, PiT: torch.Tensor, centroids: torch.Tensor,
               thresholds: torch.Tensor, S: Optional[torch.Tensor] = None, ST: Optional[torch.Tensor] = None,
               centroids_host: Optional[torch.Tensor] = None, splits=None, query_consts=None) -> TqLayer:
    """Describe a layer's constants to the library.  The tensors must stay alive
    while the struct is in use; they must be fp32, contiguous and on one GPU."""
    for name, t in (("Pi", Pi), ("PiT", PiT), ("centroids", centroids), ("thresholds", thresholds), ("S", S), ("ST", ST)):
        if t is None:
            continue
        require_gpu(t, name)
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise TypeError(f"{name} must be a contiguous float32 tensor")
    ly = TqLayer()
    ly.d, ly.mse_bits = d, mse_bits
    ly.Pi, ly.PiT = Pi.data_ptr(), PiT.data_ptr()
    ly.S = None if S is None else S.data_ptr()
    ly.ST = None if ST is None else ST.data_ptr()
    ly.centroids, ly.thresholds = centroids.data_ptr(), thresholds.data_ptr()
    ly.qjl_scale = math.sqrt(math.pi / 2.0) / d
    if splits is not None:
        pi_s, pit_s, s_s, st_s = splits[:4]
        if len(splits) > 4 and splits[4] is not None:
            ly.PiT_fp6, ly.PiT_fp6_scale = splits[4][0].data_ptr(), splits[4][1].data_ptr()
        ly.Pi_split = None if pi_s is None else pi_s.data_ptr()
        ly.PiT_split = None if pit_s is None else pit_s.data_ptr()
        ly.S_split = None if s_s is None else s_s.data_ptr()
        ly.ST_split = None if st_s is None else st_s.data_ptr()
    if query_consts is not None:
        pi_cs, s_cs, s_max = query_consts
        ly.Pi_colsum, ly.S_colsum, ly.S_rownorm_max = pi_cs.data_ptr(), s_cs.data_ptr(), float(s_max)
    walsh_terms(centroids_host if centroids_host is not None else centroids.detach().cpu(), mse_bits, ly)
    return ly


def split_bf16x3(m: torch.Tensor) -> torch.Tensor:
    """fp32 (d, d) matrix -> int16 tensor of bf16 bit patterns of three terms that sum
    to the matrix exactly (each term rounds the running remainder), in the operand order
    of the matrix-core quantise kernel: [term][row // 16][col // 32][(col % 32) // 8]
    [row % 16][col % 8], i.e. the 64 lanes' 16-byte MFMA operands of one (row tile,
    32-column slice) are contiguous.  d must be a multiple of 32."""
    rest = m.float()
    d = rest.shape[0]
    if rest.dim() != 2 or rest.shape[1] != d or d % 32:
        raise ValueError("split_bf16x3 needs a square matrix whose size is a multiple of 32")
    parts = []
    for _ in range(3):
        term = rest.to(torch.bfloat16)
        parts.append(term)
        rest = rest - term.float()
    t = torch.stack(parts).view(3, d // 16, 16, d // 32, 4, 8)      # term, row tile, n, kblk, kb, j
    return t.permute(0, 1, 3, 4, 2, 5).contiguous().view(torch.int16)


FP6_TERMS = 5


def split_fp6x5(m: torch.Tensor):
    """fp32 (d, d) matrix (row = output coordinate, column = contraction index), d a multiple of 128 -> the
    operands of the block-scaled fp6 x fp4 MFMA (16x16x128) whose other operand is a bit-plane word turned
    into fp4 codes in place: (codes, scales).

    The 32 coordinates of plane word w reach the MFMA at contraction index 32 w + 8 (c % 4) + c // 4
    (c = coordinate inside the word) with the fp4 values 0.5, 1, 2, 0.5 for c % 4 = 0, 1, 2, 3, so the
    matrix is permuted the same way and divided by those factors.  Each row's 32 values of a block are
    written as v = 2^E * sum_t digit_t * 2^(-2 - 5 t) with 2^E >= max |v| and FP6_TERMS fp6 (e2m3) digits
    (each rounds what the digits before it left, to nearest even; good to 2^-23 of the block maximum).

    codes  int32 [d // 16][d // 128][FP6_TERMS][64 lanes][6]: lane (row % 16, block b) holds its 32 six-bit
           codes, contraction index s of the block at bits 6 s .. 6 s + 5 of the lane's 192 bits;
    scales int32 [d // 16][d // 128][64 lanes][2]: the E8M0 codes 127 + E - 2 - 5 t of the lane's (row,
           block), terms 0..3 in the bytes of the first word, term 4 in the lowest byte of the second."""
    import numpy as np
    a = m.detach().double().cpu().numpy()
    d = a.shape[0]
    if a.ndim != 2 or a.shape[1] != d or d % 128:
        raise ValueError("split_fp6x5 needs a square matrix whose size is a multiple of 128")
    s_idx = np.arange(32)
    coord = 4 * (s_idx % 8) + s_idx // 8                       # coordinate inside the word at contraction index s
    factor = np.array([0.5, 1.0, 2.0, 0.5])[coord % 4]
    blocks = a.reshape(d, d // 32, 32)[:, :, coord] / factor    # [row][block][s]
    mx = np.abs(blocks).max(-1)
    e = np.where(mx > 0, np.ceil(np.log2(np.maximum(mx, 1e-300))), -60.0)
    e = np.where(np.abs(blocks).max(-1) > 2.0 ** e, e + 1, e).astype(np.int64)       # guard against log2 rounding
    x = 4.0 * blocks / (2.0 ** e)[..., None]
    codes = np.zeros((FP6_TERMS,) + blocks.shape, dtype=np.uint64)
    for t in range(FP6_TERMS):
        mag = np.minimum(np.abs(x), 7.5)
        inv = np.where(mag < 2.0, 8.0, np.where(mag < 4.0, 4.0, 2.0))
        r = np.rint(mag * inv) / inv
        ex = np.where(r < 1.0, 0, np.where(r < 2.0, 1, np.where(r < 4.0, 2, 3)))
        unit = np.where(ex <= 1, 8.0, np.where(ex == 2, 4.0, 2.0))
        man = (r * unit).astype(np.int64) - np.where(ex == 0, 0, 8)
        neg = (x < 0) & (r != 0)
        codes[t] = (neg.astype(np.uint64) << np.uint64(5)) | (ex.astype(np.uint64) << np.uint64(3)) | man.astype(np.uint64)
        x = 32.0 * (x - np.where(x < 0, -r, r))
    # 32 six-bit codes -> 192 bits -> 6 little-endian dwords
    bits = np.zeros((FP6_TERMS,) + blocks.shape[:2] + (6,), dtype=np.uint64)
    for s_ in range(32):
        lo = 6 * s_
        w, sh = lo // 32, lo % 32
        bits[..., w] |= (codes[..., s_] << np.uint64(sh)) & np.uint64(0xFFFFFFFF)
        if sh > 26:
            bits[..., w + 1] |= codes[..., s_] >> np.uint64(32 - sh)
    # [t][row][block][6] -> [row tile][chunk of 128][t][lane = (row % 16) + 16 (block % 4)][6]
    bits = bits.reshape(FP6_TERMS, d // 16, 16, d // 128, 4, 6).transpose(1, 3, 0, 4, 2, 5)
    packed = np.ascontiguousarray(bits).reshape(d // 16, d // 128, FP6_TERMS, 64, 6).astype(np.uint32)
    sc = 127 + e[..., None] - 2 - 5 * np.arange(FP6_TERMS)                             # [row][block][t]
    if sc.min() < 0 or sc.max() > 254:
        raise ValueError("matrix values out of the range of the block scales")
    sc = sc.astype(np.uint32)
    words = np.stack([sc[..., 0] | (sc[..., 1] << 8) | (sc[..., 2] << 16) | (sc[..., 3] << 24), sc[..., 4]], axis=-1)
    words = words.reshape(d // 16, 16, d // 128, 4, 2).transpose(0, 2, 3, 1, 4)
    scales = np.ascontiguousarray(words).reshape(d // 16, d // 128, 64, 2).astype(np.uint32)
    dev = m.device
    return (torch.from_numpy(packed.view(np.int32)).to(dev), torch.from_numpy(scales.view(np.int32)).to(dev))


def make_page_layout(d: int, mse_bits: int, value_bits: int, group_size: int, dtype: torch.dtype) -> TqPageLayout:
    L = TqPageLayout()
    check(lib().tq_page_layout_init(C.byref(L), d, mse_bits, value_bits, group_size, dtype_tag(dtype)),
          "tq_page_layout_init")
    return L
