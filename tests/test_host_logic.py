"""CPU: host-side logic of the package (no kernel launches): the C-ABI library
loads and exports what include/tq_hip.h declares, argument checking, page
geometry, codebook files, ring / capture policy against the reference's trace,
and the loud failure on CPU tensors."""

import ctypes as C
import json
import os
import re

import numpy as np
import pytest
import torch

import turboquant_amd
from turboquant_amd import _ffi
from turboquant_amd.capture import KVCaptureEngine, RingBuffer
from turboquant_amd.codebook import compute_lloyd_max_codebook, get_codebook, get_codebook_tensors
from turboquant_amd.quantizer import TurboQuantMSE, TurboQuantProd, _pack_indices, _unpack_indices
from turboquant_amd.kv_cache import ValueQuantized, quantize_values, unpack_values

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "tq_hip.h")).read()
    declared = set(re.findall(r"\b(tq_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = _ffi.lib()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in tq_hip.h but not exported"
    assert declared == set(_ffi.EXPORTED_SYMBOLS)
    assert lib.tq_version() == _ffi.ABI_VERSION


@pytest.mark.parametrize("d", [128, 256])
def test_split_matrices_sum_exactly_and_follow_the_documented_operand_order(d):
    """The three bf16 terms of a split matrix add up to the fp32 matrix bit for bit, and element
    (row, col) of term t sits where include/tq_hip.h says the matrix-core kernels read it."""
    g = torch.Generator().manual_seed(d)
    m = torch.randn(d, d, generator=g) * torch.logspace(-6, 2, d)[None, :]
    raw = _ffi.split_bf16x3(m)
    assert raw.dtype == torch.int16 and raw.numel() == 3 * d * d
    flat = raw.reshape(-1).view(torch.bfloat16).float()
    t, r, c = torch.meshgrid(torch.arange(3), torch.arange(d), torch.arange(d), indexing="ij")
    pos = ((((t * (d // 16) + r // 16) * (d // 32) + c // 32) * 4 + (c % 32) // 8) * 16 + r % 16) * 8 + c % 8
    assert torch.equal(torch.sort(pos.reshape(-1)).values, torch.arange(3 * d * d))       # a permutation
    terms = flat[pos]                                                                       # (3, d, d) row-major
    want = m.clone()
    for k in range(3):                       # each term is the bf16 rounding of what the terms before it left
        assert torch.equal(terms[k], want.to(torch.bfloat16).float())
        want = want - terms[k]
    assert torch.equal(terms[0] + terms[1] + terms[2], m)
    with pytest.raises(ValueError):
        _ffi.split_bf16x3(torch.zeros(48, 48))


def test_argument_errors_are_reported_before_any_launch():
    lib = _ffi.lib()
    assert lib.tq_bucketize_pack(None, 4, 128, None, 2, None, None) == -3
    assert lib.tq_sign_pack(None, 4, 128, None, None) == -3
    ly = _ffi.TqLayer()
    ly.d, ly.mse_bits = 100, 2                       # not a multiple of 64
    assert lib.tq_quantize_keys(1, 0, 4, 128, C.byref(ly), 1, 1, 1, 1, None, None, 0, None) == -2
    assert lib.tq_quantize_values(1, 0, 4, 128, 128, 48, 2, 1, 1, 1, None) == -1     # 128 % 48 != 0
    assert lib.tq_quantize_values(1, 0, 4, 128, 128, 32, 3, 1, 1, 1, None) == -2     # 3-bit values
    assert lib.tq_decode_workspace_bytes(0, 8, 128, 4) == 0
    with pytest.raises(ValueError):
        _ffi.check(-1, "x")
    with pytest.raises(RuntimeError):
        _ffi.check(700, "x")
    with pytest.raises(TypeError):
        _ffi.dtype_tag(torch.float64)


@pytest.mark.parametrize("d,mb,vb,gs,dt,per_token", [
    (128, 2, 4, 32, torch.bfloat16, 32 + 16 + 4 + 4 + 64 + 16),      # 136 B: fp32 norm and residual norm
    (256, 2, 2, 32, torch.bfloat16, 64 + 32 + 4 + 4 + 64 + 32),      # 200 B
    (128, 2, 2, 32, torch.float16, 32 + 16 + 4 + 4 + 32 + 16),
    (128, 3, 4, 64, torch.float32, 48 + 16 + 4 + 4 + 64 + 16),
    (64, 2, 2, 32, torch.bfloat16, 16 + 8 + 4 + 4 + 16 + 8),
])
def test_page_layout_geometry(d, mb, vb, gs, dt, per_token):
    L = _ffi.make_page_layout(d, mb, vb, gs, dt)
    assert L.off_keys == 0 and L.key_lane_major == (1 if d % 128 == 0 or d == 64 else 0)
    offs = [L.off_keys, L.off_meta, L.off_vdata, L.off_vscale, L.off_vzero]
    assert offs == sorted(offs) and all(o % 16 == 0 for o in offs)
    used = L.off_vzero + (d // gs) * 16 * (4 if dt == torch.float32 else 2)
    assert used == 16 * per_token
    assert L.page_bytes % 128 == 0 and used <= L.page_bytes < used + 128
    with pytest.raises(ValueError):
        _ffi.make_page_layout(100, 2, 2, 32, torch.bfloat16)
    with pytest.raises(ValueError):
        _ffi.make_page_layout(128, 2, 3, 32, torch.bfloat16)


@pytest.mark.parametrize("d,mb", [(128, 1), (128, 2), (128, 3), (128, 4), (64, 2), (256, 2), (576, 3)])
def test_walsh_terms_reconstruct_the_codebook(d, mb):
    cb = get_codebook(d, mb)
    cent = torch.tensor(cb["centroids"], dtype=torch.float32)
    ly = _ffi.TqLayer()
    _ffi.walsh_terms(cent, mb, ly)
    assert 1 <= ly.n_terms <= 2 ** mb - 1
    # a symmetric codebook is an odd function of the +-1 index bits: only odd-size subsets survive
    assert ly.n_terms == 2 ** (mb - 1)
    for idx in range(2 ** mb):
        val = ly.term_const + sum(ly.term_coef[t] * (bin(idx & ly.term_mask[t]).count("1") & 1)
                                  for t in range(ly.n_terms))
        assert val == pytest.approx(float(cent[idx]), abs=2e-7)
    # an asymmetric codebook keeps every subset
    skew = torch.arange(2 ** mb, dtype=torch.float32) ** 2
    _ffi.walsh_terms(skew, mb, ly)
    for idx in range(2 ** mb):
        val = ly.term_const + sum(ly.term_coef[t] * (bin(idx & ly.term_mask[t]).count("1") & 1)
                                  for t in range(ly.n_terms))
        assert val == pytest.approx(float(skew[idx]), abs=1e-4)


def test_shipped_codebooks_equal_reference_files(golden):
    for d, b in [(64, 1), (64, 2), (64, 3), (64, 4), (128, 1), (128, 2), (128, 3), (128, 4), (576, 3),
                 (256, 1), (256, 2), (256, 3)]:
        ref, got = golden.codebook(d, b), get_codebook(d, b)
        assert got["d"] == d and got["bits"] == b
        assert set(got) == {"centroids", "boundaries", "mse_per_coord", "mse_total", "d", "bits"}
        assert np.allclose(got["centroids"], ref["centroids"], rtol=0, atol=1e-15)
        # the fp32 tensors handed to the kernels are identical
        c, e = get_codebook_tensors(d, b, "cpu")
        assert torch.equal(c, torch.tensor(ref["centroids"], dtype=torch.float32))
        # ... and so are the thresholds, the middle one included: two of the reference's tables hold
        # -4e-17 / -3e-18 there instead of 0, which decides the bucket of a coordinate that is exactly 0
        # (every coordinate of an all-zero vector), so the shipped tables carry the published values
        assert torch.equal(e, torch.tensor(ref["boundaries"], dtype=torch.float32)), (d, b)


def test_rotation_and_sketch_matrices_equal_the_reference_ones(golden):
    """generate_rotation_matrix / generate_qjl_matrix (rotation.py:17-56) against the matrices the
    reference produced for config 1 (seed 42, sketch seed 42 + 1000) and for the other golden cases.
    torch.randn from a seeded CPU generator is bit-stable, so S must match bit for bit; Pi goes
    through LAPACK's QR, whose summation order depends on the BLAS thread count (differences of 1e-6
    between 1 and 8 threads were observed), hence 2e-6."""
    from turboquant_amd.rotation import generate_qjl_matrix, generate_rotation_matrix
    z = golden.npz("config1_full")
    S = generate_qjl_matrix(128, "cpu", seed=42 + 1000)
    assert S.dtype == torch.float32 and torch.equal(S, torch.from_numpy(z["S"]))
    Pi = generate_rotation_matrix(128, "cpu", seed=42)
    ref = torch.from_numpy(z["Pi"])
    assert Pi.shape == ref.shape and (Pi - ref).abs().max() <= 2e-6
    assert (Pi @ Pi.T - torch.eye(128)).abs().max() < 1e-5
    # a wrong sign convention, a transposed factor or a different seed rule would be off by O(1)
    assert (Pi.T - ref).abs().max() > 0.1
    for file, case in golden.key_case_list():
        kc = golden.npz(file)
        d, bits, seed = [int(v) for v in kc[case + ".meta"]]
        if golden.has(file, case + ".S"):
            assert torch.equal(generate_qjl_matrix(d, "cpu", seed=seed + 1000), torch.from_numpy(kc[case + ".S"])), case
        assert (generate_rotation_matrix(d, "cpu", seed=seed) - torch.from_numpy(kc[case + ".Pi"])).abs().max() <= 2e-6, case
    # the quantiser objects draw their matrices through the same two functions, seeds as quantizer.py:107,208
    tq = TurboQuantProd(128, bits=3, device="cpu", seed=42)
    assert torch.equal(tq.S, torch.from_numpy(z["S"]))
    assert (tq.mse_quantizer.Pi - ref).abs().max() <= 2e-6


def test_codebook_solver_known_answer(golden):
    got = compute_lloyd_max_codebook(128, 2)
    ref = golden.codebook(128, 2)
    assert got["centroids"] == pytest.approx(ref["centroids"], abs=1e-15)
    assert got["mse_total"] == pytest.approx(0.11600007032012699, abs=1e-13)
    with pytest.raises(ValueError):
        compute_lloyd_max_codebook(2, 1)


def test_pack_helpers_match_reference_vectors(golden):
    z = golden.npz("packing")
    for bits in (1, 2, 3, 4, 5):
        for d in (128, 13):
            idx = torch.from_numpy(z[f"idx_b{bits}_d{d}"])
            pk = _pack_indices(idx, bits)
            assert pk.dtype == torch.uint8 and np.array_equal(pk.numpy(), z[f"packed_b{bits}_d{d}"])
            assert np.array_equal(_unpack_indices(pk, bits, d).numpy(), z[f"unpacked_b{bits}_d{d}"])
    vq = ValueQuantized(torch.tensor([[0b11100100, 0b00011011]], dtype=torch.uint8), None, None, 2)
    assert unpack_values(vq).tolist() == [[0, 1, 2, 3, 3, 2, 1, 0]]
    vq = ValueQuantized(torch.tensor([[0xA5]], dtype=torch.uint8), None, None, 4)
    assert unpack_values(vq).tolist() == [[5, 10]]


def test_public_surface():
    assert turboquant_amd.__version__ == "0.2.0"
    for name in ("compute_lloyd_max_codebook", "get_codebook", "TurboQuantMSE", "TurboQuantProd", "TurboQuantKVCache",
                 "RingBuffer", "KVCaptureEngine", "CompressedKVStore", "compute_hybrid_attention"):
        assert hasattr(turboquant_amd, name)
    tq = TurboQuantProd(128, bits=3, device=torch.device("cpu"))
    assert set(dict(tq.named_buffers())) >= {"S", "mse_quantizer.Pi", "mse_quantizer.centroids",
                                             "mse_quantizer.boundaries", "mse_quantizer.decision_boundaries"}
    assert set(tq.state_dict()) == {"S", "mse_quantizer.Pi", "mse_quantizer.centroids", "mse_quantizer.boundaries",
                                    "mse_quantizer.decision_boundaries"}
    assert tq.mse_quantizer.bits == 2 and tq.mse_quantizer.n_clusters == 4
    with pytest.raises(AssertionError):
        TurboQuantProd(128, bits=1, device=torch.device("cpu"))


def test_no_cpu_fallback():
    tq = TurboQuantProd(128, bits=3, device=torch.device("cpu"))
    x = torch.randn(4, 128)
    with pytest.raises(RuntimeError, match="GPU only"):
        tq.quantize(x)
    with pytest.raises(RuntimeError, match="GPU only"):
        tq.mse_quantizer.quantize(x)
    with pytest.raises(RuntimeError, match="GPU only"):
        quantize_values(x, 2, 32)


class _TagStore:
    def __init__(self, heads, dim):
        self.num_kv_heads, self.head_dim, self.device = heads, dim, torch.device("cpu")
        self.chunks = []

    @property
    def num_tokens(self):
        return sum(len(c) for c in self.chunks)

    def append_chunk(self, key, value):
        assert torch.equal(key, value)
        self.chunks.append([int(t) for t in key[:, 0, 0].float().tolist()])

    def reset(self):
        self.chunks = []


def test_capture_engine_routes_tokens_like_the_reference(golden):
    for tr in golden.json("capture_trace.json"):
        if tr.get("double_prefill"):
            st = _TagStore(1, 4)
            eng = KVCaptureEngine(st, ring_capacity=4, device="cpu", dtype=torch.float32)
            a = torch.arange(3.0).view(-1, 1, 1).expand(3, 1, 4)
            eng.ingest_prefill(a, a, 3)
            eng.ingest_prefill(a + 10, a + 10, 3)
        else:
            st = _TagStore(2, 8)
            eng = KVCaptureEngine(st, ring_capacity=tr["capacity"], device="cpu", dtype=torch.float32)
            tok = 0
            if tr["prefill"]:
                k = torch.arange(float(tr["prefill"])).view(-1, 1, 1).expand(tr["prefill"], 2, 8)
                eng.ingest_prefill(k, k, tr["prefill"])
                tok = tr["prefill"]
            for _ in range(tr["decodes"]):
                k = torch.full((1, 2, 8), float(tok))
                eng.ingest_decode(k, k, 1)
                tok += 1
            if tr["flush"]:
                eng.flush()
            assert eng.total_compressed_tokens == tr["total_compressed"]
            assert eng.total_buffered_tokens == tr["total_buffered"]
            assert eng.total_tokens == tr["total_compressed"] + tr["total_buffered"]
            assert eng.ring.total_written == tr["ring_total_written"]
        peek = eng.ring.peek()
        ring = [] if peek is None else [int(t) for t in peek[0][:, 0, 0].tolist()]
        assert st.chunks == tr["chunks"]
        assert ring == tr["ring"]


def test_ring_buffer_contract():
    rb = RingBuffer(4, 2, 8, "cpu", torch.float32)
    assert rb.size == 0 and not rb.is_full and rb.peek() is None and rb.drain() is None
    k = torch.arange(6.0).view(-1, 1, 1).expand(6, 2, 8)
    spill = rb.write(k, k, 6)
    assert spill is not None and spill[0][:, 0, 0].tolist() == [0, 1, 2, 3]
    assert rb.size == 2 and rb.total_written == 6
    assert rb.peek()[0][:, 0, 0].tolist() == [4, 5]
    got = rb.drain()
    assert got[0][:, 0, 0].tolist() == [4, 5] and rb.size == 0
    rb.reset()
    assert rb.total_written == 0


def test_paged_cache_ingest_gathers_blocks_in_table_order():
    st = _TagStore(1, 4)
    eng = KVCaptureEngine(st, ring_capacity=4, device="cpu", dtype=torch.float32)
    cache = torch.zeros(2, 5, 4, 1, 4)
    table = torch.tensor([3, 0, 4])
    for logical, phys in enumerate(table.tolist()):
        for s in range(4):
            cache[:, phys, s] = logical * 4 + s
    eng.ingest_prefill_from_paged_cache(cache, 10, table, 4)
    assert st.chunks == [[0, 1, 2, 3, 4, 5]]
    assert eng.ring.peek()[0][:, 0, 0].tolist() == [6, 7, 8, 9]


def test_fp6_digits_of_the_rotation_decode_back_to_it():
    """_ffi.split_fp6x5: the five fp6 (e2m3) digits and block scales of Pi^T, in the lane order of the block-scaled
    MFMA, decode back to the matrix within 2^-22 of each (row, 32-coordinate block)'s largest value (the permuted
    contraction index and the 0.5 / 1 / 2 / 0.5 position factors of the fp4 bit operand included)."""
    from turboquant_amd import _ffi
    from turboquant_amd.rotation import generate_rotation_matrix
    d = 128
    m = generate_rotation_matrix(d, "cpu", seed=42).T.contiguous()
    codes, scales = _ffi.split_fp6x5(m)
    assert tuple(codes.shape) == (d // 16, 1, 5, 64, 6) and tuple(scales.shape) == (d // 16, 1, 64, 2)
    c = codes.numpy().view(np.uint32).astype(np.uint64)
    sc = scales.numpy().view(np.uint32)
    s_idx = np.arange(32)
    coord = 4 * (s_idx % 8) + s_idx // 8
    factor = np.array([0.5, 1.0, 2.0, 0.5])[coord % 4]
    rec = np.zeros((d, d))
    for t in range(5):
        word = sc[:, 0, :, 0] if t < 4 else sc[:, 0, :, 1]                   # [tile][lane]
        e8 = ((word >> (8 * (t % 4))) & 0xFF).astype(np.int64) - 127
        for s_ in range(32):
            lo = 6 * s_
            w, sh = lo // 32, lo % 32
            code = (c[:, 0, t, :, w] >> np.uint64(sh)) & np.uint64(63)
            if sh > 26:
                code |= (c[:, 0, t, :, w + 1] << np.uint64(32 - sh)) & np.uint64(63)
            code = code.astype(np.int64)
            ex, man = (code >> 3) & 3, code & 7
            mag = np.where(ex == 0, man / 8.0, (1 + man / 8.0) * 2.0 ** (ex - 1))
            val = np.where(code & 32, -mag, mag) * 2.0 ** e8 * factor[s_]    # [tile][lane]
            for lane in range(64):
                rec[16 * np.arange(d // 16) + (lane & 15), 32 * (lane >> 4) + coord[s_]] += val[:, lane]
    ref = m.double().numpy()
    blockmax = np.abs(ref).reshape(d, d // 32, 32).max(-1).repeat(32, axis=1)
    assert np.all(np.abs(rec - ref) <= 2.0 ** -22 * 2.0 * blockmax)


def test_quotient_of_bf16_numbers_rounds_like_its_product_with_a_reciprocal():
    """The value quantiser (kv_cache.py:53-99 divides bf16 numbers and rounds to bf16) replaces a / s by
    a * r, r an fp32 reciprocal of s good to one ulp.  Both operands have at most 8 significant bits, so the
    quotient is never a rounding tie of bf16 and never closer than 2^-17 (relative) to one, far more than the
    product's error: the two round to the same bf16 number.  Exhaustive over all pairs of significands, the
    exponent offsets the quantiser can meet, and the three reciprocals nearest to 1 / s."""
    def bf16_bits(f):
        u = f.view(np.uint32).astype(np.uint64)
        return ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint32)
    ms = np.arange(128, 256, dtype=np.float32)[:, None, None]
    ma = np.arange(128, 256, dtype=np.float32)[None, :, None]
    a = ma * np.exp2(np.arange(-30, 9, dtype=np.float32))[None, None, :]
    ref = bf16_bits((a / ms).astype(np.float32))
    r0 = (np.float32(1.0) / ms).astype(np.float32)
    for step in (-1, 0, 1):
        r = (r0.view(np.int32) + step).view(np.float32)
        got = bf16_bits((a * r).astype(np.float32))
        assert np.array_equal(got, np.broadcast_to(ref, got.shape)), step


def test_bench_refuses_more_than_one_gpu_and_its_shape_table_is_well_formed():
    """bench.py measures one GPU: --gpus 2 exits with a message instead of running; the shapes of its table mode
    are ones the entry points accept (query heads a multiple of KV heads, head sizes a multiple of 64 up to 768,
    key bits 2 - 5, value bits 2 / 4 / 8) and the byte count per token and head follows the page layout."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode == 2 and "one GPU" in res.stderr and res.stdout.strip() == ""
    sys.path.insert(0, root)
    import bench
    assert len(set(bench.SHAPE_TABLE)) == len(bench.SHAPE_TABLE)
    for (B, N, Hq, Hkv, d, kb, vb) in bench.SHAPE_TABLE:
        assert B > 0 and N > 0 and Hq % Hkv == 0 and d % 64 == 0 and 64 <= d <= 768
        assert 2 <= kb <= 5 and vb in (2, 4, 8)
    # 3-bit keys (2-bit indices), 2-bit values in groups of 32 at head_dim 256: 64 + 32 + 2 + 2 + 64 + 32 bytes
    assert bench.algorithmic_bytes_per_token_head(256, 2, 2, 32) == 196
    assert bench.algorithmic_bytes_per_token_head(128, 2, 4, 32) == 132
