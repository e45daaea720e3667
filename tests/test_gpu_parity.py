"""GPU: the HIP kernels, called through the C ABI, against the pinned oracle and
the reference's golden vectors.

Gates (from the north star): packed bytes bit-exact when the kernel is fed the
reference's rotated / projected fp32 tensors; scores within 1e-3 relative to the
score scale, |delta| <= 1e-3 * rms(scores), on identical packed bytes;
attention outputs cosine >= 0.9999 on an identical packed store.  End-to-end
quantisation (own rotation on the GPU) differs from a CPU BLAS only by fp32
summation order; its index / sign flip rates are bounded here at 1e-4.
"""

import math

import numpy as np
import pytest
import torch

from oracle import tq_oracle as O
from tests.helpers import (bit_mismatch, byte_mismatch, cosine, install_matrices, key_code, params_of, value_code)

pytestmark = pytest.mark.gpu

SCORE_TOL = 1e-3          # x rms(scores)
COS_GATE = 0.9999
FLIP_RATE = 1e-4


def _import():
    import ctypes as C
    from turboquant_amd import _ffi
    return C, _ffi


def _progress(msg):
    print(f"[gpu-parity] {msg}", flush=True)


# ------------------------------------------------------------------ packing entry points
def test_bucketize_and_sign_pack_bit_exact_on_reference_tensors(gpu, golden):
    C, ffi = _import()
    lib = ffi.lib()
    z = golden.npz("config1_full")
    jobs = [("config1", torch.from_numpy(z["y_head"]), torch.from_numpy(z["p_head"]), torch.from_numpy(z["thresholds"]),
             2, z["mse_indices"][:256], z["qjl_signs"][:256])]
    for file, case in golden.key_case_list():
        kc = golden.npz(file)
        d, bits, _ = [int(v) for v in kc[case + ".meta"]]
        y = torch.from_numpy(kc[case + ".y"]).reshape(-1, d)
        p = torch.from_numpy(kc[case + ".p"]).reshape(-1, d)
        jobs.append((case, y, p, torch.from_numpy(kc[case + ".thresholds"]), bits - 1,
                     kc[case + ".mse_indices"].reshape(y.shape[0], -1), kc[case + ".qjl_signs"].reshape(y.shape[0], -1)))
    for name, y, p, thr, mb, want_idx, want_sgn in jobs:
        _progress(f"pack {name} mb={mb} shape={tuple(y.shape)}")
        n, d = y.shape
        yd, pd, td = y.to(gpu).contiguous(), p.to(gpu).contiguous(), thr.to(gpu).contiguous()
        idx = torch.zeros(n, want_idx.shape[1], dtype=torch.uint8, device=gpu)
        sgn = torch.zeros(n, want_sgn.shape[1], dtype=torch.uint8, device=gpu)
        ffi.check(lib.tq_bucketize_pack(yd.data_ptr(), n, d, td.data_ptr(), mb, idx.data_ptr(), None), "bucketize")
        ffi.check(lib.tq_sign_pack(pd.data_ptr(), n, d, sgn.data_ptr(), None), "sign_pack")
        torch.cuda.synchronize()
        assert np.array_equal(idx.cpu().numpy(), want_idx), name
        assert np.array_equal(sgn.cpu().numpy(), want_sgn), name


def test_pack_ragged_dim_and_special_values(gpu):
    C, ffi = _import()
    lib = ffi.lib()
    g = torch.Generator().manual_seed(9)
    for mb, d in [(1, 13), (2, 13), (3, 77), (4, 5), (2, 128)]:
        thr = torch.sort(torch.randn(2 ** mb - 1, generator=g) * 0.1).values
        y = torch.randn(9, d, generator=g) * 0.1
        y[0, 0], y[0, 1], y[0, 2] = float("nan"), float("inf"), -float("inf")
        m = min(d, thr.numel())
        y[1, :m] = thr[:m]                            # exact ties go to the lower bucket
        want = O.pack_indices(O.bucketize(y, thr), mb)
        idx = torch.zeros_like(want, device=gpu)
        yd, td = y.to(gpu), thr.to(gpu)              # named, so the buffers outlive the launch
        ffi.check(lib.tq_bucketize_pack(yd.data_ptr(), 9, d, td.data_ptr(), mb, idx.data_ptr(), None), "b")
        p = torch.randn(9, d, generator=g)
        p[0, :4] = torch.tensor([0.0, -0.0, float("nan"), 1e-40])
        wsg = O.pack_signs(p)
        sgn = torch.zeros_like(wsg, device=gpu)
        pd = p.to(gpu)
        ffi.check(lib.tq_sign_pack(pd.data_ptr(), 9, d, sgn.data_ptr(), None), "s")
        torch.cuda.synchronize()
        assert torch.equal(idx.cpu(), want), (mb, d)
        assert torch.equal(sgn.cpu(), wsg), (mb, d)
    # empty input is a no-op
    ffi.check(lib.tq_sign_pack(pd.data_ptr(), 0, 8, sgn.data_ptr(), None), "empty")


# ------------------------------------------------------------------ key quantiser, flat layout
def _quantizer_for(prm, key_bits, gpu):
    from turboquant_amd.quantizer import TurboQuantProd
    tq = TurboQuantProd(prm.Pi.shape[0], bits=key_bits, device=gpu)
    return install_matrices(tq, prm)


def test_key_quantiser_end_to_end_vs_reference_vectors(gpu, golden):
    for file, case in golden.key_case_list():
        kc = golden.npz(file)
        d, bits, _ = [int(v) for v in kc[case + ".meta"]]
        if bits - 1 > 4:
            continue
        _progress(f"quantize_keys {case}")
        prm = golden.key_params(file, case)
        tq = _quantizer_for(prm, bits, gpu)
        x = golden.tensor(file, case + ".x")
        code, y, p = tq.quantize_traced(x.to(gpu))
        torch.cuda.synchronize()
        n_coord = x.numel()
        want_idx = torch.from_numpy(kc[case + ".mse_indices"])
        want_sgn = torch.from_numpy(kc[case + ".qjl_signs"])
        assert code.mse_indices.shape == want_idx.shape and code.mse_indices.dtype == torch.uint8
        assert code.qjl_signs.shape == want_sgn.shape
        assert code.norms.dtype == x.dtype and code.residual_norms.dtype == torch.float32
        idx_flips = byte_mismatch(code.mse_indices, want_idx)
        sgn_flips = bit_mismatch(code.qjl_signs, want_sgn)
        _progress(f"   index bytes differing {idx_flips}, sign bits differing {sgn_flips} of {n_coord}")
        assert idx_flips <= max(1, FLIP_RATE * n_coord), case
        assert sgn_flips <= max(2, FLIP_RATE * n_coord), case
        ref_norm = golden.tensor(file, case + ".norms").float()
        got_norm = code.norms.float().cpu()
        ulp = 2.0 ** -7 if x.dtype == torch.bfloat16 else (2.0 ** -10 if x.dtype == torch.float16 else 2.0 ** -22)
        assert torch.all((got_norm - ref_norm).abs() <= ulp * ref_norm.abs() + 1e-30), case
        if x.dtype != torch.float32:           # 16-bit norms: rounding hides the fp32 summation order
            assert (got_norm != ref_norm).float().mean() < 0.02, case
        ref_rn = torch.from_numpy(kc[case + ".residual_norms"])
        assert torch.allclose(code.residual_norms.cpu(), ref_rn, rtol=2e-5, atol=1e-6), case
        yr = torch.from_numpy(kc[case + ".y"])
        ok = ~torch.isnan(yr)
        assert (y.cpu()[ok] - yr[ok]).abs().max() < 2e-6, case
        assert torch.equal(torch.isnan(y.cpu()), torch.isnan(yr)), case
        pr = torch.from_numpy(kc[case + ".p"])
        assert (p.cpu() - pr).abs().max() <= 1e-4 * pr.abs().max(), case
        # feeding the kernel's own y / p back through the pack entry points reproduces its bytes
        assert torch.equal(O.pack_indices(O.bucketize(y.cpu(), prm.thresholds), bits - 1), code.mse_indices.cpu())
        assert torch.equal(O.pack_signs(p.cpu()), code.qjl_signs.cpu())


def test_mse_only_quantiser_and_dequant(gpu, golden):
    case = "fp32_d128_b4"
    kc = golden.npz("key_cases")
    prm = golden.key_params("key_cases", case)
    tq = _quantizer_for(prm, 4, gpu)
    x = golden.tensor("key_cases", case + ".x").to(gpu)
    mq = tq.mse_quantizer.quantize(x)
    full = tq.quantize(x)
    assert torch.equal(mq.indices, full.mse_indices) and torch.equal(mq.norms, full.norms) and mq.bits == 3
    ref_code = key_code(torch.from_numpy(kc[case + ".mse_indices"]), torch.from_numpy(kc[case + ".qjl_signs"]),
                        torch.from_numpy(kc[case + ".residual_norms"]), golden.tensor("key_cases", case + ".norms"), 3)
    from turboquant_amd.quantizer import MSEQuantized, ProdQuantized
    deq = tq.mse_quantizer.dequantize(MSEQuantized(ref_code.mse_indices.to(gpu), ref_code.norms.to(gpu), 3)).cpu()
    want = O.mse_dequantize(ref_code.mse_indices, ref_code.norms, prm)
    assert (deq - want).abs().max() <= 2e-6 * want.abs().max()
    rt = tq.mse_quantizer(x).cpu()
    assert rt.shape == x.shape
    assert ((rt - x.cpu()).norm(dim=-1) / x.cpu().norm(dim=-1).clamp_min(1e-6))[1:].pow(2).mean() < 0.06   # mse_total(3b)=0.034


def test_prod_dequant_and_score_on_reference_bytes(gpu, golden):
    from turboquant_amd.quantizer import ProdQuantized
    for file, case in golden.key_case_list():
        kc = golden.npz(file)
        d, bits, _ = [int(v) for v in kc[case + ".meta"]]
        if bits - 1 > 4:
            continue
        _progress(f"dequant+score {case}")
        prm = golden.key_params(file, case)
        tq = _quantizer_for(prm, bits, gpu)
        code = ProdQuantized(torch.from_numpy(kc[case + ".mse_indices"]).to(gpu),
                             torch.from_numpy(kc[case + ".qjl_signs"]).to(gpu),
                             torch.from_numpy(kc[case + ".residual_norms"]).to(gpu),
                             golden.tensor(file, case + ".norms").to(gpu), bits - 1)
        deq = tq.dequantize(code).cpu()
        want = torch.from_numpy(kc[case + ".dequant"])
        assert (deq - want).abs().max() <= 4e-6 * want.abs().max(), case
        q = golden.tensor(file, case + ".q").to(gpu)
        sc = tq.attention_score(q, code).cpu()
        ref = torch.from_numpy(kc[case + ".scores"])
        assert sc.shape == ref.shape and sc.dtype == torch.float32
        rms = ref.pow(2).mean().sqrt()
        assert (sc - ref).abs().max() <= SCORE_TOL * rms, case
        assert (sc - ref).abs().max() <= 2e-5 * rms, case      # fp32 kernels sit far inside the gate


@pytest.mark.parametrize("d,key_bits,n,dtype", [(128, 3, 1000, torch.bfloat16), (128, 2, 64, torch.float32),
                                               (128, 4, 77, torch.float16), (128, 5, 129, torch.bfloat16),
                                               (256, 3, 333, torch.bfloat16), (256, 5, 31, torch.float32)])
def test_matrix_core_dequantiser_vs_double_precision_and_vector_kernel(gpu, d, key_bits, n, dtype):
    """head_dim 128 / 256 de-quantise on the matrix cores.  Random codes (every code and sign value
    occurs), ragged vector counts, all index widths: the result must sit within fp32 product-sum
    accuracy of the float64 value of quantizer.py:259-272, and agree with the vector-ALU kernel
    (taken when the output is not 16-byte aligned) to the same accuracy."""
    import ctypes as C
    from turboquant_amd import _ffi
    from turboquant_amd.quantizer import MSEQuantized, ProdQuantized, TurboQuantProd
    tq = TurboQuantProd(d, bits=key_bits, device=gpu)
    prm = params_of(tq)
    mb = key_bits - 1
    g = torch.Generator().manual_seed(7 * d + key_bits)
    idx = torch.randint(0, 1 << mb, (n, d), generator=g)
    packed = O.pack_indices(idx, mb)
    signs = torch.randint(0, 256, (n, d // 8), generator=g, dtype=torch.uint8)
    norms = (torch.rand(n, generator=g) * 8 + 0.05).to(dtype)
    rnorms = torch.rand(n, generator=g) * 3
    _progress(f"dequant d={d} bits={key_bits} n={n} {dtype}")
    code = ProdQuantized(packed.to(gpu), signs.to(gpu), rnorms.to(gpu), norms.to(gpu), mb)
    got = tq.dequantize(code).cpu().double()
    cent = prm.centroids.double()[idx]
    sg = O.unpack_signs(signs, d).double()
    want = (cent @ prm.Pi.double()) * norms.double()[:, None] + \
        (sg @ prm.S.double()) * (float(np.float32(prm.qjl_scale)) * rnorms.double())[:, None]
    scale = want.abs().max()
    assert (got - want).abs().max() <= 2e-6 * scale
    got_mse = tq.mse_quantizer.dequantize(MSEQuantized(packed.to(gpu), norms.to(gpu), mb)).cpu().double()
    want_mse = (cent @ prm.Pi.double()) * norms.double()[:, None]
    assert (got_mse - want_mse).abs().max() <= 2e-6 * want_mse.abs().max()
    # the same call with an output that is only 4-byte aligned runs the vector-ALU kernel
    buf = torch.empty(n * d + 1, dtype=torch.float32, device=gpu)
    out = buf[1:]
    ly = tq._layer()
    with torch.cuda.device(gpu):
        _ffi.check(_ffi.lib().tq_dequant_keys(code.mse_indices.data_ptr(), code.qjl_signs.data_ptr(),
                                              code.norms.data_ptr(), _ffi.dtype_tag(dtype),
                                              code.residual_norms.data_ptr(), n, C.byref(ly), out.data_ptr(),
                                              _ffi.stream_ptr(torch.device(gpu))), "tq_dequant_keys")
    valu = out.cpu().double().reshape(n, d)
    assert (valu - want).abs().max() <= 2e-6 * scale
    assert (valu - got).abs().max() <= 2e-6 * scale


@pytest.mark.parametrize("d,key_bits,n_q", [(128, 3, 4), (64, 2, 9), (256, 4, 3), (192, 5, 8)])
def test_score_word_and_byte_kernels_agree_bit_for_bit(gpu, d, key_bits, n_q):
    """tq_score reads a key's codes a word at a time when the index / sign rows are 4-byte aligned and a
    byte at a time otherwise; both sum over the coordinates in the same order, so the logits are equal."""
    import ctypes as C
    from turboquant_amd import _ffi
    from turboquant_amd.quantizer import TurboQuantProd
    tq = TurboQuantProd(d, bits=key_bits, device=gpu)
    g = torch.Generator(device=gpu).manual_seed(d + key_bits)
    n_k = 333
    code = tq.quantize(torch.randn(n_k, d, generator=g, device=gpu))
    q = torch.randn(n_q, d, generator=g, device=gpu)
    _progress(f"score kernels d={d} bits={key_bits} n_q={n_q}")
    aligned = tq.attention_score(q, code)
    # the same call on copies of the index and sign rows that start one byte into an allocation
    ib = torch.empty(code.mse_indices.numel() + 1, dtype=torch.uint8, device=gpu)
    sb = torch.empty(code.qjl_signs.numel() + 1, dtype=torch.uint8, device=gpu)
    ib[1:] = code.mse_indices.reshape(-1)
    sb[1:] = code.qjl_signs.reshape(-1)
    scores = torch.empty(n_q, n_k, dtype=torch.float32, device=gpu)
    work = torch.empty(2 * n_q * d, dtype=torch.float32, device=gpu)
    rn = code.residual_norms.float().contiguous()
    ly = tq._layer()
    with torch.cuda.device(gpu):
        _ffi.check(_ffi.lib().tq_score(q.data_ptr(), _ffi.dtype_tag(q.dtype), 1, n_q, ib[1:].data_ptr(),
                                       sb[1:].data_ptr(), code.norms.data_ptr(), _ffi.dtype_tag(code.norms.dtype),
                                       rn.data_ptr(), n_k, C.byref(ly), scores.data_ptr(), work.data_ptr(),
                                       _ffi.stream_ptr(torch.device(gpu))), "tq_score")
    assert torch.equal(scores, aligned)
    ref = O.attention_score(q.cpu(), O.KeyCode(code.mse_indices.cpu(), code.qjl_signs.cpu(), code.residual_norms.cpu(),
                                               code.norms.cpu(), key_bits - 1, None, None), params_of(tq))
    assert (aligned.cpu() - ref).abs().max() <= 2e-5 * ref.pow(2).mean().sqrt()


def test_config1_scores_on_reference_bytes_and_round_trip(gpu, golden):
    from turboquant_amd.quantizer import ProdQuantized
    z = golden.npz("config1_full")
    prm = O.KeyParams(torch.from_numpy(z["Pi"]), torch.from_numpy(z["S"]), torch.from_numpy(z["centroids"]),
                      torch.from_numpy(z["thresholds"]), 2)
    tq = _quantizer_for(prm, 3, gpu)
    code = ProdQuantized(torch.from_numpy(z["mse_indices"]).to(gpu), torch.from_numpy(z["qjl_signs"]).to(gpu),
                         torch.from_numpy(z["residual_norms"]).to(gpu), torch.from_numpy(z["norms"]).to(gpu), 2)
    Q = torch.from_numpy(z["Q"]).to(gpu)
    sc = tq.attention_score(Q, code).cpu()
    ref = torch.from_numpy(z["scores"])
    rms = float(ref.pow(2).mean().sqrt())
    err = float((sc - ref).abs().max())
    _progress(f"config1 scores: max|delta| {err:.3e} = {err / rms:.2e} x rms")
    assert sc.shape == (32, 4096)
    assert err <= SCORE_TOL * rms
    # full round trip on the regenerated config-1 keys: bytes differ from the reference's only by
    # fp32 summation order
    g = torch.Generator(device="cpu").manual_seed(0)
    K = torch.randn(4096, 128, generator=g, dtype=torch.float32)
    K = K / K.norm(dim=-1, keepdim=True)
    K = K * (0.5 + 1.5 * torch.rand(4096, generator=g)).unsqueeze(-1)
    got = tq.quantize(K.to(gpu))
    idx_flips = byte_mismatch(got.mse_indices, torch.from_numpy(z["mse_indices"]))
    sgn_flips = bit_mismatch(got.qjl_signs, torch.from_numpy(z["qjl_signs"]))
    _progress(f"config1 end-to-end: {idx_flips} index bytes, {sgn_flips} sign bits differ of 524288 coordinates")
    assert idx_flips <= 52 and sgn_flips <= 52
    assert torch.allclose(got.norms.cpu(), torch.from_numpy(z["norms"]), rtol=1e-6)
    assert torch.allclose(got.residual_norms.cpu(), torch.from_numpy(z["residual_norms"]), rtol=2e-5)
    sc2 = tq.attention_score(Q, got).cpu()
    # a flipped sign moves one score by a few percent of rms; everything else agrees to 1e-5
    assert ((sc2 - ref).abs() > 1e-4 * rms).float().mean() < 1e-3


def test_attention_score_batched_and_broadcast(gpu):
    from turboquant_amd.quantizer import TurboQuantProd
    tq = TurboQuantProd(128, bits=3, device=gpu)
    prm = params_of(tq)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 3, 70, 128, generator=g).bfloat16()
    q = torch.randn(2, 3, 5, 128, generator=g).bfloat16()
    code = tq.quantize(x.to(gpu))
    sc = tq.attention_score(q.to(gpu), code).cpu()
    host = key_code(code.mse_indices.cpu(), code.qjl_signs.cpu(), code.residual_norms.cpu(), code.norms.cpu(), 2)
    want = O.attention_score(q, host, prm)
    rms = want.pow(2).mean().sqrt()
    assert sc.shape == (2, 3, 5, 70)
    assert (sc - want).abs().max() <= 2e-5 * rms
    one_q = q[:1, :1]
    sc_b = tq.attention_score(one_q.to(gpu), code).cpu()           # query broadcast over the key batch dims
    assert torch.allclose(sc_b, O.attention_score(one_q, host, prm), atol=float(2e-5 * rms))


# ------------------------------------------------------------------ values
def test_value_quantiser_bit_exact_vs_reference_vectors(gpu, golden):
    from turboquant_amd.kv_cache import dequantize_values, quantize_values, ValueQuantized
    z = golden.npz("values")
    for case in golden.cases("values"):
        tag, b, g_ = case.split("_")
        bits, gs = int(b[1:]), int(g_[1:])
        v = golden.tensor("values", case + ".v")
        vq = quantize_values(v.to(gpu), bits=bits, group_size=gs)
        assert vq.bits == bits and vq.scales.dtype == v.dtype and vq.zeros.dtype == v.dtype
        assert np.array_equal(vq.data.cpu().numpy(), z[case + ".data"]), case
        assert torch.equal(vq.scales.cpu(), golden.tensor("values", case + ".scales")), case
        assert torch.equal(vq.zeros.cpu(), golden.tensor("values", case + ".zeros")), case
        deq = dequantize_values(vq, gs).cpu()
        assert np.array_equal(deq.numpy(), z[case + ".dequant"], equal_nan=True), case


def test_value_quantiser_strided_rows_and_nan(gpu):
    from turboquant_amd.kv_cache import quantize_values
    g = torch.Generator().manual_seed(2)
    big = torch.randn(37, 256, generator=g).bfloat16()
    view = big[:, :128]                                     # row stride 256, 128 used
    vq = quantize_values(view.to(gpu)[:, :], bits=4, group_size=32)
    want = O.quantize_values(view.contiguous(), 4, 32)
    assert torch.equal(vq.data.cpu(), want.data) and torch.equal(vq.scales.cpu(), want.scales)
    v = torch.randn(3, 64, generator=g)
    v[1, 5] = float("nan")
    vq = quantize_values(v.to(gpu), bits=2, group_size=32)
    want = O.quantize_values(v, 2, 32)
    assert torch.equal(torch.isnan(vq.scales.cpu()), torch.isnan(want.scales))
    assert torch.equal(vq.data.cpu()[[0, 2]], want.data[[0, 2]])


# ------------------------------------------------------------------ paged store
def _make_pool(gpu, d, key_bits, vb, H, n_pages, dtype=torch.bfloat16, seed=42, gs=32):
    from turboquant_amd.paged import PagedKVPool
    from turboquant_amd.quantizer import TurboQuantProd
    tq = TurboQuantProd(d, bits=key_bits, device=gpu, seed=seed)
    return PagedKVPool(tq, H, n_pages, value_bits=vb, value_group_size=gs, dtype=dtype, device=gpu), tq


@pytest.mark.parametrize("d,key_bits,vb,dtype", [(128, 3, 4, torch.bfloat16), (256, 3, 2, torch.bfloat16),
                                                   (64, 2, 2, torch.float16), (128, 4, 4, torch.bfloat16),
                                                   (128, 5, 2, torch.float32)])
def test_paged_append_equals_flat_quantise(gpu, d, key_bits, vb, dtype):
    from turboquant_amd.kv_cache import quantize_values
    H, T = 2, 75
    pool, tq = _make_pool(gpu, d, key_bits, vb, H, 16, dtype)
    g = torch.Generator().manual_seed(d + key_bits)
    k = torch.randn(1, T, H, d, generator=g).to(dtype).to(gpu)
    v = torch.randn(1, T, H, d, generator=g).to(dtype).to(gpu)
    table = torch.randperm(16, generator=g).to(torch.int32).to(gpu)[None, :]     # scattered physical pages
    # three appends with ragged boundaries: 0..20, 20..21, 21..75
    for a, b in ((0, 20), (20, 21), (21, 75)):
        pool.append(k[:, a:b], v[:, a:b], table, torch.tensor([a], dtype=torch.int32, device=gpu))
    idx, sgn, norms, rnorms, vdata, vsc, vz = pool.export_flat(table[0], T)
    ref = tq.quantize(k[0].transpose(0, 1))                 # (H, T, d)
    refv = quantize_values(v[0].transpose(0, 1), bits=vb, group_size=32)
    torch.cuda.synchronize()
    assert torch.equal(idx, ref.mse_indices) and torch.equal(sgn, ref.qjl_signs)
    assert torch.equal(norms, ref.norms) and torch.equal(rnorms, ref.residual_norms)
    assert torch.equal(vdata, refv.data) and torch.equal(vsc, refv.scales) and torch.equal(vz, refv.zeros)
    # and the same tokens appended in one go give the same pages
    pool2, _ = _make_pool(gpu, d, key_bits, vb, H, 16, dtype)
    pool2.append(k, v, table)
    n_pg = (T + 15) // 16
    used = table[0, :n_pg].long()
    assert torch.equal(pool.data[used[:-1]], pool2.data[used[:-1]])


@pytest.mark.parametrize("d,key_bits,vb,dtype,B,H", [(128, 3, 4, torch.bfloat16, 32, 8), (256, 3, 2, torch.bfloat16, 5, 2),
                                                       (64, 2, 2, torch.float16, 40, 4), (128, 4, 4, torch.float32, 7, 8)])
def test_single_token_append_with_a_workgroup_per_tile(gpu, d, key_bits, vb, dtype, B, H):
    """The page write of a decode step: a token per sequence at ragged positions.  Few 16-vector tiles get a
    workgroup each that computes its tile only (option "append_small", the default); the pages must equal,
    byte for byte, those of the kernel whose workgroups compute groups of tiles (option 0)."""
    from turboquant_amd import _ffi
    pages = 8
    g = torch.Generator().manual_seed(11 * d + B)
    k = torch.randn(B, 1, H, d, generator=g).to(dtype).to(gpu)
    v = torch.randn(B, 1, H, d, generator=g).to(dtype).to(gpu)
    table = torch.randperm(B * pages, generator=g).to(torch.int32).view(B, pages).to(gpu)
    pos = torch.randint(0, pages * 16, (B,), generator=g).to(torch.int32).to(gpu)
    got = {}
    try:
        for mode in (0, -1, 3):                      # 3: only appends of up to three tiles take the small kernel
            _ffi.check(_ffi.lib().tq_set_option(b"append_small", mode), "tq_set_option")
            pool, _ = _make_pool(gpu, d, key_bits, vb, H, B * pages, dtype)
            pool.data.fill_(0x3C)
            _progress(f"single-token append d={d} {dtype} B={B} append_small={mode}")
            pool.append(k, v, table, pos)
            torch.cuda.synchronize()
            got[mode] = pool.data.clone()
    finally:
        _ffi.check(_ffi.lib().tq_set_option(b"append_small", -1), "tq_set_option")
    assert torch.equal(got[0], got[-1]) and torch.equal(got[0], got[3])
    assert not torch.all(got[0] == 0x3C)


def test_paged_append_random_chunks_equal_flat_quantise(gpu):
    # seeded sweep: several sequences appended in ragged chunks (any start slot inside a page, chunk
    # lengths across page boundaries, batched calls with per-sequence start positions); the exported
    # pages must equal the flat quantisers' output bit for bit
    import random
    from turboquant_amd.kv_cache import quantize_values
    rnd = random.Random(77)
    for case in range(8):
        d = rnd.choice([64, 128, 256])
        key_bits = rnd.choice([2, 3, 4]) if d != 256 else rnd.choice([2, 3])
        vb = rnd.choice([2, 4])
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        H, B = rnd.choice([1, 2, 4]), rnd.choice([1, 2, 3])
        total = rnd.choice([16, 31, 64, 100, 177])
        cuts = sorted(set([0, total] + [rnd.randrange(1, total) for _ in range(rnd.choice([0, 1, 2]))]))
        pages = (total + 15) // 16
        pool, tq = _make_pool(gpu, d, key_bits, vb, H, B * pages + 2, dtype, seed=5 + case)
        g = torch.Generator().manual_seed(300 + case)
        k = torch.randn(B, total, H, d, generator=g).to(dtype).to(gpu)
        v = torch.randn(B, total, H, d, generator=g).to(dtype).to(gpu)
        table = torch.randperm(B * pages + 2, generator=g)[: B * pages].to(torch.int32).reshape(B, pages).to(gpu)
        _progress(f"append case {case}: d={d} kb={key_bits} vb={vb} {dtype} H={H} B={B} cuts={cuts}")
        for a0, a1 in zip(cuts[:-1], cuts[1:]):
            pool.append(k[:, a0:a1], v[:, a0:a1], table, torch.full((B,), a0, dtype=torch.int32, device=gpu))
        for b in range(B):
            idx, sgn, norms, rnorms, vdata, vsc, vz = pool.export_flat(table[b], total)
            ref = tq.quantize(k[b].transpose(0, 1))
            refv = quantize_values(v[b].transpose(0, 1), bits=vb, group_size=32)
            torch.cuda.synchronize()
            assert torch.equal(idx, ref.mse_indices) and torch.equal(sgn, ref.qjl_signs), (case, b)
            assert torch.equal(norms, ref.norms) and torch.equal(rnorms, ref.residual_norms), (case, b)
            assert torch.equal(vdata, refv.data) and torch.equal(vsc, refv.scales) and torch.equal(vz, refv.zeros), (case, b)


def test_large_append_runs_values_beside_keys_and_stays_ordered(gpu):
    # an append of >= 4096 tiles forks the value kernel onto a side stream and joins it back: the
    # pages must equal those of two small appends (plain path), and a reader queued on the caller's
    # stream right after the call must see finished pages
    H, T, d = 8, 8192, 128
    g = torch.Generator().manual_seed(21)
    k = torch.randn(1, T, H, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(1, T, H, d, generator=g).bfloat16().to(gpu)
    table = torch.randperm(T // 16, generator=g).to(torch.int32).to(gpu)[None, :]
    big, _ = _make_pool(gpu, d, 3, 2, H, T // 16)
    small, _ = _make_pool(gpu, d, 3, 2, H, T // 16)
    for _ in range(3):                               # repeated so that a missing join would show as a race
        big.data.zero_()
        big.append(k, v, table)
        seen = big.data.clone()                      # queued behind the append on the same stream
    half = T // 2
    small.append(k[:, :half], v[:, :half], table)
    small.append(k[:, half:], v[:, half:], table, torch.tensor([half], dtype=torch.int32, device=gpu))
    torch.cuda.synchronize()
    used = table[0].long()
    assert torch.equal(seen[used], small.data[used])
    assert torch.equal(big.data[used], small.data[used])


def _store_from_oracle_view(pool, table_row, n_tok):
    idx, sgn, norms, rnorms, vdata, vsc, vz = [t.cpu() for t in pool.export_flat(table_row, n_tok)]
    return key_code(idx, sgn, rnorms, norms, pool.quantizer.bits - 1), value_code(vdata, vsc, vz, pool.value_bits)


def _decode_case(gpu, d, key_bits, vb, B, Hq, Hkv, lens, recent, seed, n_split=None, dtype=torch.bfloat16,
                 shape_kq=None, recent_pad=0, return_out=False):
    g = torch.Generator().manual_seed(seed)
    max_len = max(max(lens), 1)
    pages_per_seq = (max_len + 15) // 16
    n_pages = B * pages_per_seq + 3
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, n_pages, dtype, seed=42 + 7 * (seed % 5))
    perm = torch.randperm(n_pages, generator=g)[: B * pages_per_seq].to(torch.int32)
    table = perm.reshape(B, pages_per_seq).to(gpu)
    k = torch.randn(B, max_len, Hkv, d, generator=g).to(dtype)
    v = torch.randn(B, max_len, Hkv, d, generator=g).to(dtype)
    q = torch.randn(B, Hq, d, generator=g).to(dtype)
    if shape_kq is not None:
        k, q = shape_kq(k.float(), q.float())
        k, q = k.to(dtype), q.to(dtype)
    pool.append(k.to(gpu), v.to(gpu), table)
    rk = rv = rl = None
    if recent:
        rk = torch.randn(B, max(recent), Hkv, d, generator=g).to(dtype)
        rv = torch.randn(B, max(recent), Hkv, d, generator=g).to(dtype)
        rl = torch.tensor(recent, dtype=torch.int32)
    seq = torch.tensor(lens, dtype=torch.int32)
    rk_dev, rv_dev = (None, None) if rk is None else (rk.to(gpu), rv.to(gpu))
    if rk is not None and recent_pad:
        # rows inside a wider buffer, starting `recent_pad` elements in: strided, and not word-aligned when odd
        wide = [torch.zeros(B, max(recent), Hkv, d + 2 * recent_pad, dtype=dtype, device=gpu) for _ in range(2)]
        wide[0][..., recent_pad:recent_pad + d] = rk_dev
        wide[1][..., recent_pad:recent_pad + d] = rv_dev
        rk_dev, rv_dev = wide[0][..., recent_pad:recent_pad + d], wide[1][..., recent_pad:recent_pad + d]
    out = pool.decode_attention(q.to(gpu), table, seq.to(gpu), recent_k=rk_dev, recent_v=rv_dev,
                                recent_len=None if rl is None else rl.to(gpu), n_split=n_split, max_len=max_len)
    torch.cuda.synchronize()
    prm = params_of(tq)
    worst = 1.0
    for b in range(B):
        kc = vc = None
        if lens[b]:
            kc, vc = _store_from_oracle_view(pool, table[b], lens[b])
        r = recent[b] if recent else 0
        # MIN_HISTORY is host policy; the kernel itself attends to any non-empty history
        want = O.hybrid_attention(q[b:b + 1], kc, vc, max(lens[b], O.MIN_HISTORY) if lens[b] else 0, prm, Hkv,
                                  rk[b, :r] if r else None, rv[b, :r] if r else None)
        got = out[b:b + 1].cpu()
        assert got.dtype == q.dtype
        if lens[b] == 0 and r == 0:
            assert torch.count_nonzero(got) == 0
            continue
        c = cosine(got, want)
        worst = min(worst, c)
        assert c >= COS_GATE, (b, c)
        assert (got.float() - want.float()).abs().max() <= 2 ** -7 * want.float().abs().max() + 1e-3, b
    return out.cpu() if return_out else worst


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv", [(128, 3, 4, 8, 2), (256, 3, 2, 16, 2), (128, 3, 2, 4, 4),
                                                   (64, 3, 4, 4, 1), (128, 4, 4, 8, 2), (128, 2, 2, 6, 2),
                                                   (256, 4, 2, 16, 2), (256, 4, 4, 8, 4), (256, 2, 4, 6, 2)])
def test_decode_attention_matches_oracle_on_the_same_store(gpu, d, key_bits, vb, Hq, Hkv):
    _progress(f"decode d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv}")
    worst = _decode_case(gpu, d, key_bits, vb, 3, Hq, Hkv, [200, 37, 512], None, seed=d + vb)
    _progress(f"   worst cosine {worst:.7f}")


@pytest.mark.parametrize("trend", ["rising", "falling", "all_low", "spiky"])
def test_decode_softmax_over_wide_score_ranges(gpu, trend):
    # logits that climb or fall by hundreds over the context, sit far below zero everywhere, or jump
    # at a few tokens: the running reference of the softmax has to follow without overflow, underflow
    # or loss of the small weights that matter
    d, Hkv, Hq = 256, 2, 16

    def shape_kq(k, q):
        B, N, H, _ = k.shape
        u = torch.nn.functional.normalize(torch.ones(d), dim=0)
        ramp = torch.linspace(-1.0, 1.0, N)[None, :, None, None]
        if trend == "rising":
            k = k + 60.0 * ramp * u
        elif trend == "falling":
            k = k - 60.0 * ramp * u
        elif trend == "all_low":
            k = k - 80.0 * u
        else:
            spikes = torch.zeros(N)
            spikes[[3, N // 3, N // 2 + 1, N - 2]] = torch.tensor([20.0, 45.0, 70.0, 95.0])
            k = k + spikes[None, :, None, None] * u
        q = q + 40.0 * u                       # sm_scale * q.k swings by about +-150 along the ramp
        return k, q

    worst = _decode_case(gpu, d, 3, 2, 2, Hq, Hkv, [1500, 333], None, seed=11, shape_kq=shape_kq)
    _progress(f"softmax range {trend}: worst cosine {worst:.7f}")
    worst = _decode_case(gpu, 128, 3, 4, 2, 8, 2, [700, 64], [5, 0], seed=12, n_split=3,
                         shape_kq=lambda k, q: (shape_kq_128(k, trend), q + 30.0 * torch.nn.functional.normalize(torch.ones(128), dim=0)))
    _progress(f"softmax range {trend} (d=128, tail): worst cosine {worst:.7f}")


def shape_kq_128(k, trend):
    N = k.shape[1]
    u = torch.nn.functional.normalize(torch.ones(128), dim=0)
    ramp = torch.linspace(-1.0, 1.0, N)[None, :, None, None]
    if trend == "rising":
        return k + 50.0 * ramp * u
    if trend == "falling":
        return k - 50.0 * ramp * u
    if trend == "all_low":
        return k - 70.0 * u
    spikes = torch.zeros(N)
    spikes[[1, N // 2, N - 1]] = torch.tensor([30.0, 60.0, 90.0])
    return k + spikes[None, :, None, None] * u


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,dtype", [(128, 3, 4, 8, 2, torch.float16), (128, 3, 2, 32, 2, torch.bfloat16),
                                                         (64, 3, 4, 12, 1, torch.float16), (128, 4, 4, 4, 2, torch.float32),
                                                         (256, 3, 2, 16, 2, torch.float16), (128, 4, 2, 6, 2, torch.float16),
                                                         (256, 4, 4, 8, 8, torch.float16), (128, 2, 4, 7, 1, torch.float16),
                                                         (128, 3, 4, 12, 1, torch.bfloat16), (256, 3, 2, 18, 2, torch.bfloat16),
                                                         (128, 3, 2, 11, 1, torch.bfloat16), (128, 4, 4, 32, 2, torch.float16),
                                                         (576, 3, 2, 16, 1, torch.bfloat16), (768, 2, 4, 4, 2, torch.float32),
                                                         (192, 3, 4, 6, 2, torch.float16), (64, 5, 2, 10, 2, torch.bfloat16),
                                                         (128, 3, 4, 22, 2, torch.bfloat16), (256, 3, 2, 26, 2, torch.bfloat16),
                                                         (64, 3, 4, 9, 1, torch.float16), (128, 3, 4, 15, 1, torch.bfloat16),
                                                         (128, 3, 8, 20, 2, torch.bfloat16)])
def test_decode_attention_general_kernel_shapes(gpu, d, key_bits, vb, Hq, Hkv, dtype):
    # fp16 pools (matrix-core kernel with the fp16 zero-point product), more than 8 query heads per KV head
    # (served as ceil(G / 8) groups of at most 8 that read the same pages: 16 = 8 + 8, 12 = 6 + 6, and unequal ones
    # where G does not divide: 9 = 5 + 4, 11 = 6 + 5, 13 = 7 + 6, 15 = 8 + 7), and shapes without a matrix-core
    # kernel (fp32 pools, head sizes other than 64 / 128 / 256, 5-bit keys at head_dim 64), which take the general page
    # kernel:
    # all must meet the same gate
    _progress(f"general decode d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} {dtype}")
    worst = _decode_case(gpu, d, key_bits, vb, 2, Hq, Hkv, [300, 77], [0, 9], seed=500 + d + Hq, dtype=dtype)
    _progress(f"   worst cosine {worst:.7f}")


def test_decode_attention_random_shapes(gpu):
    # seeded sweep over head dims, bit widths, GQA ratios, batch sizes, ragged lengths (block and page
    # boundaries included), split counts and exact tails
    import random
    rnd = random.Random(1234)
    boundary = [0, 1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257]
    for case in range(14):
        d = rnd.choice([64, 128, 128, 256, 256])
        key_bits = rnd.choice([2, 3, 3, 4]) if d != 256 else rnd.choice([2, 3])
        vb = rnd.choice([2, 4])
        Hkv = rnd.choice([1, 2, 3])
        G = rnd.choice([1, 2, 4, 8])
        B = rnd.choice([1, 2, 4])
        lens = [rnd.choice(boundary + [rnd.randrange(300, 900)]) for _ in range(B)]
        recent = [rnd.choice([0, 0, 1, 7, 33]) for _ in range(B)] if rnd.random() < 0.4 else None
        n_split = rnd.choice([None, 1, 2, 5, 16])
        _progress(f"random case {case}: d={d} kb={key_bits} vb={vb} Hkv={Hkv} G={G} lens={lens} recent={recent} split={n_split}")
        worst = _decode_case(gpu, d, key_bits, vb, B, Hkv * G, Hkv, lens, recent, seed=100 + case, n_split=n_split)
        _progress(f"   worst cosine {worst:.7f}")


def test_decode_attention_ragged_empty_and_hybrid_tail(gpu):
    # empty sequence, history shorter than a page, page-aligned history, ragged exact tails
    worst = _decode_case(gpu, 128, 3, 4, 5, 8, 2, [0, 5, 16, 33, 1000], [0, 3, 128, 0, 77], seed=77)
    _progress(f"ragged+tail worst cosine {worst:.7f}")
    worst = _decode_case(gpu, 128, 3, 2, 2, 8, 8, [0, 0], [40, 1], seed=78)          # exact tokens only
    worst = _decode_case(gpu, 128, 3, 2, 2, 4, 2, [0, 64], None, seed=79)            # one row has nothing at all


@pytest.mark.parametrize("d,dtype,Hq,Hkv,recent,pad", [
    (256, torch.bfloat16, 16, 2, [300, 129, 1], 0),       # three chunks of 128 rows, ragged
    (256, torch.bfloat16, 16, 2, [128, 77, 0], 1),        # rows not word-aligned: row-staged kernel
    (128, torch.float16, 8, 8, [200, 256, 13], 2),        # strided rows, still word-aligned; one head per KV head
    (128, torch.bfloat16, 8, 2, [150, 128, 1], 8),        # 16-byte aligned rows in a wider buffer, two chunks' worth
    (256, torch.bfloat16, 16, 2, [128, 40, 0], 6),        # word-aligned but not 16-byte aligned: 4-byte loads
    (64, torch.float16, 6, 2, [520, 3, 64], 0),           # two chunks at the smallest head size, 3 heads per group
    (128, torch.float32, 8, 2, [130, 64, 5], 0),          # fp32 rows
    (576, torch.float32, 4, 1, [40, 17, 33], 0),          # fp32 rows wider than the workgroup: two columns per thread
    (768, torch.bfloat16, 4, 2, [70, 32, 1], 0),
])
def test_exact_tail_shapes(gpu, d, dtype, Hq, Hkv, recent, pad):
    """The exact recent tokens (score.py:99-111) at the tail kernels' corners: several chunks, rows that are
    strided or not word-aligned, every element type, head sizes from 64 to 768."""
    _progress(f"exact tail d={d} {dtype} Hq={Hq} Hkv={Hkv} recent={recent} pad={pad}")
    worst = _decode_case(gpu, d, 3, 2, 3, Hq, Hkv, [100, 0, 33], recent, seed=300 + d + pad, dtype=dtype, recent_pad=pad)
    _progress(f"  worst cosine {worst:.7f}")


def test_hybrid_step_of_many_sequences_at_head_dim_256(gpu):
    """Twenty sequences at head_dim 256 with 128 exact tokens each: the exact tail's tiles fill a compute unit's
    LDS, the grid is larger than the card, and the tail and the query preparation run as two launches instead of
    one (score.py:99-173 against the oracle, ragged histories and tails, few and many splits)."""
    B = 20
    lens = [64 * (b % 5) + 17 * b for b in range(B)]
    recent = [128 if b % 3 else 7 * b % 128 for b in range(B)]
    for n_split in (2, 9):
        _progress(f"many sequences d=256 n_split={n_split}")
        worst = _decode_case(gpu, 256, 3, 2, B, 16, 2, lens, recent, seed=4242, n_split=n_split)
        _progress(f"  worst cosine {worst:.7f}")


def test_hybrid_step_of_many_sequences_with_the_preparation_on_the_matrix_cores(gpu):
    """A hybrid step whose query preparation alone is more workgroups than the card holds at once (here 80 sequences
    x 32 query heads at head_dim 128, bf16): the exact tail and the preparation run as a launch each, the latter on the
    matrix cores, instead of sharing the launch of the vector-ALU preparation (score.py:99-173 against the oracle,
    ragged histories and tails; and against the shared launch, which sums the rotation in another order)."""
    from turboquant_amd import _ffi
    B = 80
    lens = [48 * (b % 7) + 5 * b for b in range(B)]
    recent = [128 if b % 3 else (11 * b) % 128 for b in range(B)]
    outs = []
    try:
        for on in (1, 0):
            _ffi.check(_ffi.lib().tq_set_option(b"prep_mfma", on), "tq_set_option")
            _progress(f"many sequences d=128 prep_mfma={on}")
            outs.append(_decode_case(gpu, 128, 3, 4, B, 32, 8, lens, recent, seed=977, n_split=1, return_out=True))
    finally:
        _ffi.check(_ffi.lib().tq_set_option(b"prep_mfma", 1), "tq_set_option")
    assert float((outs[0].float() - outs[1].float()).abs().max()) <= 2.0 ** -7 * float(outs[1].float().abs().max()) + 1e-6


@pytest.mark.parametrize("d,dtype,Hq,Hkv,recent,n_split,pad", [
    (256, torch.bfloat16, 16, 2, [128, 3, 0], 12, 0),      # four workgroups per head group; shares of 32, of 0 / 1 tokens, of none
    (128, torch.float16, 8, 1, [300, 77, 1], 9, 8),        # several load rounds per share, rows inside a wider buffer
    (128, torch.float32, 4, 4, [64, 33, 2], 16, 0),        # 64 rows: two workgroups
    (64, torch.bfloat16, 3, 1, [130, 5, 129], 11, 6),      # 4-byte loads
    (576, torch.float32, 4, 1, [40, 17, 33], 10, 0),       # a head size of the general page kernel
])
def test_exact_tail_shared_by_several_workgroups(gpu, d, dtype, Hq, Hkv, recent, n_split, pad):
    """A hybrid step (score.py:99-173) with more than eight context splits and few (sequence, KV head) pairs gives
    the exact tokens of a group of query heads to 2 or 4 workgroups, a share of the tokens and a partial each
    (option "tail_chunks"): against the oracle, and against the one-workgroup tail to rounding."""
    from turboquant_amd import _ffi

    def _set_option(name, value):
        _ffi.check(_ffi.lib().tq_set_option(name.encode(), int(value)), "tq_set_option")

    _progress(f"shared exact tail d={d} {dtype} Hq={Hq} Hkv={Hkv} recent={recent} n_split={n_split} pad={pad}")
    outs = []
    try:
        for on in (1, 0):
            _set_option("tail_chunks", on)
            outs.append(_decode_case(gpu, d, 3, 2, 3, Hq, Hkv, [400, 0, 33], recent, seed=500 + d + pad, dtype=dtype,
                                     recent_pad=pad, n_split=n_split, return_out=True))
    finally:
        _set_option("tail_chunks", 1)
    eps = 2.0 ** -20 if dtype == torch.float32 else 2.0 ** -8
    assert float((outs[0].float() - outs[1].float()).abs().max()) <= eps * float(outs[1].float().abs().max()) + 1e-6


@pytest.mark.parametrize("d,key_bits,vb,dtype", [(128, 3, 4, torch.bfloat16), (256, 3, 2, torch.bfloat16),
                                                   (64, 2, 2, torch.float16), (128, 4, 4, torch.float32)])
def test_append_from_blocks_equals_gather_then_append(gpu, d, key_bits, vb, dtype):
    """tq_append_kv_from_blocks reads the tokens in place from a paged exact cache; the pool it fills must be
    byte-identical to gathering every sequence's tokens with torch indexing and appending them
    (capture.py:187-217), for ragged run lengths and runs that start inside a page."""
    from turboquant_amd.paged import PagedKVPool
    g = torch.Generator().manual_seed(3 * d + vb)
    H, B, n_blocks, per_seq = 2, 3, 40, 12
    kc = torch.randn(n_blocks, 16, H, d, generator=g).to(dtype).to(gpu)
    vc = torch.randn(n_blocks, 16, H, d, generator=g).to(dtype).to(gpu)
    src = torch.randperm(n_blocks, generator=g)[: B * per_seq].view(B, per_seq).to(torch.int32).to(gpu)
    dst = torch.randperm(B * per_seq, generator=g).view(B, per_seq).to(torch.int32).to(gpu)
    for start, run in (([0, 0, 0], [70, 16, 133]), ([16, 5, 37], [100, 1, 90])):
        _progress(f"append_from_blocks d={d} {dtype} start={start} run={run}")
        pa, tq = _make_pool(gpu, d, key_bits, vb, H, B * per_seq, dtype=dtype)
        pb = PagedKVPool(tq, H, B * per_seq, value_bits=vb, dtype=dtype, device=gpu)
        sp = torch.tensor(start, dtype=torch.int32)
        pa.append_from_blocks(kc, vc, src, dst, torch.tensor(run, dtype=torch.int32), start_pos=sp)
        for b in range(B):
            pos = torch.arange(start[b], start[b] + run[b], device=gpu)
            blk = src[b].long()[pos // 16]
            k = kc[blk, pos % 16][None]                       # (1, run, H, d)
            v = vc[blk, pos % 16][None]
            pb.append(k, v, dst[b:b + 1], start_pos=sp[b:b + 1])
        assert torch.equal(pa.data, pb.data)


def test_capture_engine_ingests_a_paged_cache_in_place(gpu):
    """KVCaptureEngine.ingest_prefill_from_paged_cache (capture.py:187-217) with 16-token blocks quantises the
    part to compress straight out of the paged cache; store and ring must equal the gather-then-ingest path."""
    from turboquant_amd.capture import KVCaptureEngine
    from turboquant_amd.store import CompressedKVStore
    g = torch.Generator().manual_seed(17)
    H, d, n_tok, n_blocks = 2, 128, 300, 32
    cache = torch.randn(2, n_blocks, 16, H, d, generator=g).bfloat16().to(gpu)
    table = torch.randperm(n_blocks, generator=g)[:19].to(torch.int32)
    engines = []
    for _ in range(2):
        store = CompressedKVStore(head_dim=d, num_kv_heads=H, key_bits=3, value_bits=2, device=gpu)
        engines.append(KVCaptureEngine(store=store, ring_capacity=128, device=gpu))
    engines[0].ingest_prefill_from_paged_cache(cache, n_tok, table, 16)
    phys = table.long().to(gpu)
    k = cache[0].index_select(0, phys).reshape(-1, H, d)[:n_tok]
    v = cache[1].index_select(0, phys).reshape(-1, H, d)[:n_tok]
    engines[1].ingest_prefill(k, v, n_tok)
    assert engines[0].store.num_tokens == engines[1].store.num_tokens == n_tok - 128
    fa, fb = engines[0].store.get_flat_cache(), engines[1].store.get_flat_cache()
    for a, b in zip(tuple(fa.prod_q)[:4] + tuple(fa.value_q)[:3], tuple(fb.prod_q)[:4] + tuple(fb.value_q)[:3]):
        assert torch.equal(a, b)
    for a, b in zip(engines[0].ring.peek(), engines[1].ring.peek()):
        assert torch.equal(a, b)
    assert engines[0].total_tokens == n_tok


def test_pool_export_word_and_byte_kernels_agree(gpu):
    """tq_pool_export writes the flat tensors a word at a time; outputs that are not 4-byte aligned take the
    byte-wise kernel.  Both must give the same bytes (ragged token count, permuted pages, every value width)."""
    import ctypes as C
    from turboquant_amd import _ffi
    for d, key_bits, vb in [(128, 3, 2), (256, 4, 4), (64, 2, 2), (128, 5, 4)]:
        g = torch.Generator().manual_seed(d + vb)
        H, n_tok = 2, 75
        pool, tq = _make_pool(gpu, d, key_bits, vb, H, 8)
        table = torch.randperm(8, generator=g).to(torch.int32)[None].to(gpu)
        k = torch.randn(1, n_tok, H, d, generator=g).bfloat16().to(gpu)
        v = torch.randn(1, n_tok, H, d, generator=g).bfloat16().to(gpu)
        pool.append(k, v, table)
        _progress(f"export kernels d={d} key_bits={key_bits} vb={vb}")
        idx, sgn, norms, rn, vd, vs, vz = pool.export_flat(table[0], n_tok)
        bufs = [torch.zeros(t.numel() + 1, dtype=torch.uint8, device=gpu) for t in (idx, sgn, vd)]
        norms2, rn2, vs2, vz2 = [torch.zeros_like(t) for t in (norms, rn, vs, vz)]
        with torch.cuda.device(gpu):
            _ffi.check(_ffi.lib().tq_pool_export(
                pool.data.data_ptr(), pool.num_pages, H, table[0].contiguous().data_ptr(), n_tok, C.byref(pool.layout),
                bufs[0][1:].data_ptr(), bufs[1][1:].data_ptr(), norms2.data_ptr(), rn2.data_ptr(), bufs[2][1:].data_ptr(),
                vs2.data_ptr(), vz2.data_ptr(), _ffi.stream_ptr(torch.device(gpu))), "tq_pool_export")
        for got, want in zip(bufs, (idx, sgn, vd)):
            assert torch.equal(got[1:], want.reshape(-1))
        for got, want in ((norms2, norms), (rn2, rn), (vs2, vs), (vz2, vz)):
            assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))


def test_decode_split_invariance_and_page_permutation(gpu):
    from turboquant_amd.paged import PagedKVPool
    g = torch.Generator().manual_seed(5)
    d, Hkv, Hq, B, N = 128, 2, 8, 2, 1500
    pool, tq = _make_pool(gpu, d, 3, 4, Hkv, 2 * 94 + 1)
    k = torch.randn(B, N, Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, N, Hkv, d, generator=g).bfloat16().to(gpu)
    q = torch.randn(B, Hq, d, generator=g).bfloat16().to(gpu)
    t1 = torch.arange(2 * 94, dtype=torch.int32).reshape(2, 94).to(gpu)
    pool.append(k, v, t1)
    seq = torch.tensor([N, N - 7], dtype=torch.int32, device=gpu)
    outs = [pool.decode_attention(q, t1, seq, n_split=s, max_len=N).float() for s in (1, 3, 32, 94)]
    for o in outs[1:]:
        assert (o - outs[0]).abs().max() <= 2 ** -7 * outs[0].abs().max()
    # the same tokens behind a permuted page table give bit-identical results
    pool2 = PagedKVPool(tq, Hkv, 2 * 94 + 1, value_bits=4, dtype=torch.bfloat16, device=gpu)
    t2 = torch.randperm(2 * 94, generator=g).to(torch.int32).reshape(2, 94).to(gpu)
    pool2.append(k, v, t2)
    o2 = pool2.decode_attention(q, t2, seq, n_split=3, max_len=N).float()
    assert torch.equal(o2, outs[1])


def test_decode_one_million_token_context_against_dense_attention_on_the_dequantised_cache(gpu):
    """The largest context of the size table: one sequence of 2^20 tokens (65,536 pages, appended in four
    chunks at growing start positions).  Size-independent checks: the result does not depend on the split
    count, and it equals dense fp32 attention over the de-quantised keys and values (score.py:117-173),
    which the flat entry points produce from the exported pages."""
    from turboquant_amd.kv_cache import ValueQuantized, dequantize_values
    from turboquant_amd.quantizer import ProdQuantized
    g = torch.Generator(device=gpu).manual_seed(21)
    d, Hkv, Hq, N = 128, 1, 4, 1 << 20
    pool, tq = _make_pool(gpu, d, 3, 2, Hkv, N // 16)
    table = torch.randperm(N // 16, generator=g, device=gpu).to(torch.int32)[None]
    chunk = N // 4
    for c in range(4):
        _progress(f"1M context: append chunk {c}")
        k = torch.randn(1, chunk, Hkv, d, generator=g, device=gpu).bfloat16()
        v = torch.randn(1, chunk, Hkv, d, generator=g, device=gpu).bfloat16()
        pool.append(k, v, table, start_pos=torch.tensor([c * chunk], dtype=torch.int32))
    q = (torch.randn(1, Hq, d, generator=g, device=gpu) * 3).bfloat16()
    seq = torch.tensor([N - 5], dtype=torch.int32, device=gpu)
    outs = [pool.decode_attention(q, table, seq, n_split=s, max_len=N).float() for s in (64, 512, 7)]
    for o in outs[1:]:
        assert (o - outs[0]).abs().max() <= 2 ** -7 * outs[0].abs().max()
    n = N - 5
    idx, sgn, norms, rn, vd, vs, vz = pool.export_flat(table[0], n)
    khat = tq.dequantize(ProdQuantized(idx[0], sgn[0], rn[0], norms[0], 2))             # (n, d) fp32
    vhat = dequantize_values(ValueQuantized(vd[0], vs[0], vz[0], 2), 32).float()         # (n, d)
    logits = (q[0].float() @ khat.T) / math.sqrt(d)                                      # (Hq, n)
    want = torch.softmax(logits, dim=-1) @ vhat
    cos = cosine(outs[0][0].cpu(), want.cpu())
    _progress(f"1M context: cosine vs dense attention on the de-quantised cache {cos:.7f}")
    assert cos >= 0.9999


def test_decode_step_replays_from_a_captured_graph(gpu):
    """A serving loop captures its decode step once and replays it.  One step = advance the lengths, append one
    token per sequence, fused decode attention; the library allocates nothing and never synchronises, so the
    step can be captured.  Every replay (inputs refilled in place, eager work and synchronisation between the
    replays) must equal the same step run eagerly on a twin pool."""
    g = torch.Generator(device=gpu).manual_seed(13)
    d, Hkv, Hq, B, N0, cap = 128, 2, 8, 3, 200, 256
    pools = [_make_pool(gpu, d, 3, 4, Hkv, B * (cap // 16))[0] for _ in range(2)]
    table = torch.randperm(B * (cap // 16), generator=g, device=gpu).to(torch.int32).view(B, -1)
    k0 = torch.randn(B, N0, Hkv, d, generator=g, device=gpu).bfloat16()
    v0 = torch.randn(B, N0, Hkv, d, generator=g, device=gpu).bfloat16()
    for p in pools:
        p.append(k0, v0, table)
    seqs = [torch.tensor([N0, N0 - 37, N0 - 150], dtype=torch.int32, device=gpu) for _ in range(2)]
    k1, v1 = torch.zeros(B, 1, Hkv, d, dtype=torch.bfloat16, device=gpu), torch.zeros(B, 1, Hkv, d, dtype=torch.bfloat16, device=gpu)
    q = torch.zeros(B, Hq, d, dtype=torch.bfloat16, device=gpu)
    outs = [torch.zeros_like(q) for _ in range(2)]
    ws = [p.workspace(B, Hq, 4) for p in pools]

    def step(i):
        seqs[i].add_(1)
        pools[i].append(k1, v1, table, start_pos=seqs[i] - 1)
        pools[i].decode_attention(q, table, seqs[i], n_split=4, workspace=ws[i], out=outs[i], max_len=cap)

    def refill():
        k1.copy_(torch.randn(k1.shape, generator=g, device=gpu).bfloat16())
        v1.copy_(torch.randn(v1.shape, generator=g, device=gpu).bfloat16())
        q.copy_(torch.randn(q.shape, generator=g, device=gpu).bfloat16())

    refill()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up outside the capture (launch attributes, allocator)
        step(0)
    torch.cuda.current_stream().wait_stream(side)
    step(1)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(0)
    step(1)                                            # the capture itself does not run the step: ...
    graph.replay()                                     # ... this replay is step 2 of pool 0
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(seqs[0], seqs[1])
    for r in range(4):
        refill()
        _progress(f"graph replay {r}")
        graph.replay()
        step(1)
        torch.cuda.synchronize()
        assert torch.equal(seqs[0], seqs[1])
        assert torch.equal(outs[0], outs[1]), r
    assert torch.equal(pools[0].data, pools[1].data)


def test_page_kernel_timing_hook_times_one_dispatch_and_changes_nothing(gpu):
    # tq_time_next_page_kernel attaches an event pair to the next page-kernel dispatch of this thread:
    # the elapsed time is positive and below the bracketing stream markers', the hook disarms itself,
    # and the result is bit-identical to an untimed call
    from turboquant_amd import _ffi
    g = torch.Generator().manual_seed(9)
    d, Hkv, Hq, N = 256, 2, 16, 4096
    pool, _ = _make_pool(gpu, d, 3, 2, Hkv, N // 16)
    k = torch.randn(1, N, Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(1, N, Hkv, d, generator=g).bfloat16().to(gpu)
    t = torch.arange(N // 16, dtype=torch.int32)[None].to(gpu)
    pool.append(k, v, t)
    q = torch.randn(1, Hq, d, generator=g).bfloat16().to(gpu)
    seq = torch.tensor([N], dtype=torch.int32, device=gpu)
    ref = pool.decode_attention(q, t, seq, max_len=N).clone()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    for e in ev:
        e.record()                                   # creates the underlying events
    torch.cuda.synchronize()
    ev[0].record()
    _ffi.lib().tq_time_next_page_kernel(ev[1].cuda_event, ev[2].cuda_event)
    out = pool.decode_attention(q, t, seq, max_len=N).clone()
    ev[3].record()
    torch.cuda.synchronize()
    inner, outer = ev[1].elapsed_time(ev[2]), ev[0].elapsed_time(ev[3])
    _progress(f"page kernel {inner * 1e3:.1f} us inside a {outer * 1e3:.1f} us call")
    assert 0.0 < inner < outer
    assert torch.equal(out, ref)
    again = pool.decode_attention(q, t, seq, max_len=N)          # hook disarmed: plain launch
    torch.cuda.synchronize()
    assert torch.equal(again, ref)


def test_decode_constant_values_and_convexity(gpu):
    # softmax weights are a convex combination: constant V comes back exactly (up to value
    # quantisation of a constant group, which is exact) and outputs stay inside [min v, max v]
    g = torch.Generator().manual_seed(6)
    d, Hkv, Hq, N = 128, 1, 4, 300
    pool, _ = _make_pool(gpu, d, 3, 2, Hkv, 20)
    k = torch.randn(1, N, Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.full((1, N, Hkv, d), 0.75).bfloat16().to(gpu)
    t = torch.arange(19, dtype=torch.int32)[None].to(gpu)
    pool.append(k, v, t)
    q = torch.randn(1, Hq, d, generator=g).bfloat16().to(gpu)
    out = pool.decode_attention(q, t, torch.tensor([N], dtype=torch.int32, device=gpu), max_len=N)
    assert torch.all(out.float() == 0.75)


# ------------------------------------------------------------------ store / capture / score API (reference call shapes)
def test_store_flat_cache_matches_reference_golden(gpu, golden):
    from turboquant_amd.score import compute_hybrid_attention
    from turboquant_amd.store import CompressedKVStore
    z = golden.npz("hybrid")
    for case in golden.cases("hybrid"):
        H, G, d, n_hist, n_recent, vb = [int(x) for x in z[case + ".meta"]]
        _progress(f"hybrid {case}")
        store = CompressedKVStore(d, H, key_bits=3, value_bits=vb, value_group_size=32, device=gpu, layer_idx=3)
        cent, _, thr = O.codebook_tensors(golden.codebook(d, 2))
        prm = O.KeyParams(torch.from_numpy(z[case + ".Pi"]), torch.from_numpy(z[case + ".S"]), cent, thr, 2)
        install_matrices(store.quantizer, prm)
        q = golden.tensor("hybrid", case + ".q").to(gpu)
        if n_hist:
            k = golden.tensor("hybrid", case + ".k").to(gpu)
            v = golden.tensor("hybrid", case + ".v").to(gpu)
            store.append_chunk(k[: n_hist // 2], v[: n_hist // 2])
            store.append_chunk(k[n_hist // 2:], v[n_hist // 2:])
            assert store.num_tokens == n_hist and store.num_chunks == 2
            flat = store.get_flat_cache()
            assert flat.num_tokens == n_hist and flat is store.get_flat_cache()
            n_coord = n_hist * H * d
            assert flat.prod_q.mse_indices.shape == z[case + ".mse_indices"].shape
            assert byte_mismatch(flat.prod_q.mse_indices, torch.from_numpy(z[case + ".mse_indices"])) <= max(1, FLIP_RATE * n_coord)
            assert bit_mismatch(flat.prod_q.qjl_signs, torch.from_numpy(z[case + ".qjl_signs"])) <= max(2, FLIP_RATE * n_coord)
            assert torch.equal(flat.value_q.data.cpu(), torch.from_numpy(z[case + ".v_data"]))
            assert torch.equal(flat.value_q.scales.cpu(), golden.tensor("hybrid", case + ".v_scales"))
            assert torch.equal(flat.value_q.zeros.cpu(), golden.tensor("hybrid", case + ".v_zeros"))
            assert store.memory_bytes() == int(z[case + ".memory_bytes"])
        else:
            assert store.get_flat_cache() is None
        rk = golden.tensor("hybrid", case + ".recent_k").to(gpu) if n_recent else None
        rv = golden.tensor("hybrid", case + ".recent_v").to(gpu) if n_recent else None
        out = compute_hybrid_attention(q, store, rk, rv, num_query_heads=H * G).cpu()
        ref = golden.tensor("hybrid", case + ".out")
        assert out.shape == ref.shape and out.dtype == ref.dtype
        c = cosine(out, ref)
        _progress(f"   cosine vs reference output {c:.7f}")
        assert c >= COS_GATE, case
    # nothing stored, nothing recent: zeros (score.py:59-63); GQA mismatch raises
    store = CompressedKVStore(128, 2, device=gpu)
    q = torch.randn(1, 4, 128, device=gpu, dtype=torch.bfloat16)
    assert torch.count_nonzero(compute_hybrid_attention(q, store, None, None, 4)) == 0
    with pytest.raises(ValueError):
        compute_hybrid_attention(torch.randn(1, 5, 128, device=gpu, dtype=torch.bfloat16), store,
                                 torch.randn(3, 2, 128, device=gpu, dtype=torch.bfloat16),
                                 torch.randn(3, 2, 128, device=gpu, dtype=torch.bfloat16), 5)


def test_capture_engine_end_to_end_on_gpu(gpu):
    from turboquant_amd.capture import KVCaptureEngine
    from turboquant_amd.score import compute_hybrid_attention
    from turboquant_amd.store import CompressedKVStore
    g = torch.Generator().manual_seed(8)
    H, G, d = 2, 4, 128
    store = CompressedKVStore(d, H, key_bits=3, value_bits=4, device=gpu, layer_idx=1)
    eng = KVCaptureEngine(store, ring_capacity=32, device=gpu)
    k = torch.randn(500, H, d, generator=g).bfloat16()
    v = torch.randn(500, H, d, generator=g).bfloat16()
    eng.ingest_prefill(k[:300].to(gpu), v[:300].to(gpu), 300)
    for t in range(300, 500):
        eng.ingest_decode(k[t:t + 1].to(gpu), v[t:t + 1].to(gpu), 1)
    assert eng.total_tokens == 500 and eng.total_buffered_tokens == 500 - store.num_tokens
    assert store.num_tokens == 268 + 32 * 7 and store.num_chunks == 8
    q = torch.randn(2, H * G, d, generator=g).bfloat16()
    rk, rv = eng.ring.peek()
    out = compute_hybrid_attention(q.to(gpu), store, rk, rv, num_query_heads=H * G).cpu()
    flat = store.get_flat_cache()
    kc = key_code(flat.prod_q.mse_indices.cpu(), flat.prod_q.qjl_signs.cpu(), flat.prod_q.residual_norms.cpu(),
                  flat.prod_q.norms.cpu(), 2)
    vc = value_code(flat.value_q.data.cpu(), flat.value_q.scales.cpu(), flat.value_q.zeros.cpu(), 4)
    want = O.hybrid_attention(q, kc, vc, store.num_tokens, params_of(store.quantizer), H, rk.cpu(), rv.cpu())
    assert cosine(out, want) >= COS_GATE
    eng.reset()
    assert eng.total_tokens == 0 and store.get_flat_cache() is None


def test_kv_cache_object_against_reference_golden(gpu, golden):
    from turboquant_amd.kv_cache import TurboQuantKVCache
    z = golden.npz("kv_cache_object")
    cache = TurboQuantKVCache(128, key_bits=3, value_bits=2, buffer_size=16, device=gpu, dtype=torch.float32, layer_idx=1)
    cent, _, thr = O.codebook_tensors(golden.codebook(128, 2))
    install_matrices(cache.key_quantizer, O.KeyParams(torch.from_numpy(z["Pi"]), torch.from_numpy(z["S"]), cent, thr, 2))
    cache.prefill(torch.from_numpy(z["k"]).to(gpu), torch.from_numpy(z["v"]).to(gpu))
    for i in range(5):
        cache.append(torch.from_numpy(z[f"append_k{i}"]).to(gpu), torch.from_numpy(z[f"append_v{i}"]).to(gpu))
    assert cache.get_seq_length() == int(z["seq_len"])
    sc = cache.attention_scores(torch.from_numpy(z["q"]).to(gpu)).cpu()
    ref = torch.from_numpy(z["scores"])
    assert sc.shape == ref.shape
    # a flipped sign bit moves single entries; everything else agrees tightly
    assert ((sc - ref).abs() > 1e-4).float().mean() < 0.01
    out = cache.attend(torch.softmax(sc.to(gpu), dim=-1)).cpu()
    assert cosine(out, torch.from_numpy(z["out"])) >= COS_GATE
    mem = cache.memory_bytes()
    assert [mem[n] for n in ("quantized_keys", "quantized_values", "buffer", "total")] == z["memory"].tolist()


def test_stream_read_probe_runs_and_rejects_bad_arguments(gpu):
    # the read-only probe behind the bench's "fraction of streaming-read bandwidth": argument checks and a
    # launch that completes (it writes nothing, so there is no output to compare)
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    buf = torch.ones(1 << 22, dtype=torch.uint8, device=gpu)
    st = torch.cuda.current_stream().cuda_stream
    for flight in (1, 4, 8):
        assert lib.tq_stream_read(buf.data_ptr(), buf.numel(), 4, flight, None, st) == 0
    assert lib.tq_stream_read(buf.data_ptr(), 16 * 1000 + 16, 2, 4, None, st) == 0      # tail shorter than a round
    assert lib.tq_stream_read(buf.data_ptr(), 0, 4, 4, None, st) == 0
    torch.cuda.synchronize()
    assert lib.tq_stream_read(None, 16, 4, 4, None, st) < 0
    assert lib.tq_stream_read(buf.data_ptr() + 4, 16, 4, 4, None, st) < 0
    assert lib.tq_stream_read(buf.data_ptr(), 24, 4, 4, None, st) < 0
    assert lib.tq_stream_read(buf.data_ptr(), 16, 4, 3, None, st) < 0
    assert lib.tq_stream_read(buf.data_ptr(), 16, 0, 4, None, st) < 0


@pytest.mark.parametrize("d,dtype,Hq,Hkv,ring,n_split", [(128, torch.bfloat16, 16, 4, 128, None), (256, torch.bfloat16, 16, 2, 128, None),
                                                           (64, torch.float16, 8, 2, 200, None), (128, torch.float32, 4, 2, 48, None),
                                                           (256, torch.bfloat16, 16, 2, 128, 12),       # many splits: the exact tokens
                                                           (128, torch.float16, 4, 1, 100, 9),          # are shared by 2 / 4 workgroups
                                                           (576, torch.bfloat16, 8, 1, 128, None),      # wide heads: the exact tail in the
                                                           (512, torch.bfloat16, 16, 2, 100, 5)])       # launch of the matrix-core rotation
def test_ring_entry_reads_the_exact_cache_in_place(gpu, d, dtype, Hq, Hkv, ring, n_split):
    """tq_decode_attn_paged_ring takes the exact recent tokens (score.py:99-111) straight from a paged exact
    cache through the block table; it must equal, bit for bit, gathering those rows with torch indexing and
    passing them as recent_k / recent_v with the history lengths reduced by their count."""
    g = torch.Generator().manual_seed(5 * d + ring)
    lens = [0, 7, ring, ring + 1, 333, 16 * 40]
    B, per_seq = len(lens), 40
    n_blocks = B * per_seq + 5
    pool, _ = _make_pool(gpu, d, 3, 2, Hkv, n_blocks, dtype)
    perm = torch.randperm(n_blocks, generator=g)[: B * per_seq].view(B, per_seq).to(torch.int32)
    used = (torch.tensor(lens)[:, None] + 15) // 16 > torch.arange(per_seq)[None]
    table = torch.where(used, perm, torch.zeros_like(perm)).to(gpu)        # unused entries padded with block 0
    cache = torch.zeros(2, n_blocks, 16, Hkv, d, dtype=dtype, device=gpu)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype).to(gpu)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype).to(gpu)
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    for b, n in enumerate(lens):
        if n == 0:
            continue
        pos = torch.arange(n, device=gpu)
        blk = table[b].long()[pos // 16]
        cache[0, blk, pos % 16] = k[b, :n]
        cache[1, blk, pos % 16] = v[b, :n]
        pool.append(k[b:b + 1, :n], v[b:b + 1, :n], table[b:b + 1])
    q = torch.randn(B, Hq, d, generator=g).to(dtype).to(gpu)
    _progress(f"ring entry d={d} {dtype} ring={ring} lens={lens}")
    got = pool.decode_attention_ring(q, table, seq, cache[0], cache[1], ring, n_split=n_split, max_len=max(lens)).clone()
    # the same step with the rows gathered on the host side
    tail = torch.clamp(seq.long(), max=ring)
    pos = (seq.long() - tail)[:, None] + torch.arange(ring, device=gpu)[None]
    pos = torch.minimum(pos, (seq.long() - 1).clamp_min(0)[:, None])
    slot = torch.gather(table.long(), 1, pos // 16) * 16 + pos % 16
    rk = cache[0].reshape(-1, Hkv, d)[slot]
    rv = cache[1].reshape(-1, Hkv, d)[slot]
    want = pool.decode_attention(q, table, (seq.long() - tail).to(torch.int32), recent_k=rk, recent_v=rv,
                                 recent_len=tail.to(torch.int32), n_split=n_split, max_len=max(lens))
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert torch.count_nonzero(got[0]) == 0                         # the empty sequence
    # and against the oracle on one sequence that has both parts
    b = 4
    kc, vc = _store_from_oracle_view(pool, table[b], lens[b] - ring)
    ref = O.hybrid_attention(q[b:b + 1].cpu(), kc, vc, max(lens[b] - ring, O.MIN_HISTORY), params_of(pool.quantizer), Hkv,
                             k[b, lens[b] - ring:lens[b]].cpu(), v[b, lens[b] - ring:lens[b]].cpu())
    assert cosine(got[b:b + 1].cpu(), ref) >= COS_GATE


def test_config2_full_size_prefill_quantise(gpu):
    """The prefill-quantise workload at its full size (32768 tokens x 8 KV heads, head size 128, four outlier
    channels x20 per tensor and head, bf16; 3-bit keys, 2-bit values in groups of 32, 2048 pages per head):
    a sample of tokens against the oracle, and over all tokens what does not depend on the size - chunked
    appends give the same pages, every value is within half a step of its code, the key estimator
    (quantizer.py:274-302) is unbiased, the MSE stage's distortion is the codebook's."""
    from turboquant_amd.codebook import get_codebook
    from turboquant_amd.quantizer import MSEQuantized, ProdQuantized
    H, T, d = 8, 32768, 128
    g = torch.Generator().manual_seed(1)
    K = torch.randn(1, H, T, d, generator=g)
    V = torch.randn(1, H, T, d, generator=g)
    for X in (K, V):
        for h in range(H):
            X[0, h][:, torch.randperm(d, generator=g)[:4]] *= 20.0
    k = K[0].transpose(0, 1)[None].bfloat16().contiguous()             # (1, T, H, d)
    v = V[0].transpose(0, 1)[None].bfloat16().contiguous()
    table = torch.randperm(T // 16, generator=g).to(torch.int32)[None].to(gpu)
    pool, tq = _make_pool(gpu, d, 3, 2, H, T // 16)
    _progress("config 2 full size: one append of 32768 tokens x 8 heads")
    kd, vd = k.to(gpu), v.to(gpu)
    pool.append(kd, vd, table)
    idx, sgn, norms, rnorms, vdata, vsc, vz = pool.export_flat(table[0], T)
    torch.cuda.synchronize()
    # (1) the same tokens in four chunks with ragged boundaries
    pool2, _ = _make_pool(gpu, d, 3, 2, H, T // 16)
    for a, b in ((0, 5000), (5000, 5001), (5001, 20000), (20000, T)):
        pool2.append(kd[:, a:b], vd[:, a:b], table, torch.tensor([a], dtype=torch.int32, device=gpu))
    torch.cuda.synchronize()
    assert torch.equal(pool.data, pool2.data)
    # (2) 1024 sampled tokens against the oracle
    prm = params_of(tq)
    pick = torch.randperm(T, generator=g)[:1024].sort().values
    ks = k[0, pick].transpose(0, 1).contiguous()                        # (H, 1024, d)
    vs = v[0, pick].transpose(0, 1).contiguous()
    want = O.prod_quantize(ks, prm)
    n_coord = ks.numel()
    pk = pick.to(gpu)
    idx_flips = byte_mismatch(idx[:, pk].cpu(), want.mse_indices)
    sgn_flips = bit_mismatch(sgn[:, pk].cpu(), want.qjl_signs)
    _progress(f"   sample: index bytes differing {idx_flips}, sign bits differing {sgn_flips} of {n_coord}")
    assert idx_flips <= max(1, FLIP_RATE * n_coord)
    assert sgn_flips <= max(2, FLIP_RATE * n_coord)
    got_norm, ref_norm = norms[:, pk].float().cpu(), want.norms.float()
    assert torch.all((got_norm - ref_norm).abs() <= 2.0 ** -7 * ref_norm.abs())
    assert torch.allclose(rnorms[:, pk].cpu(), want.residual_norms, rtol=2e-5, atol=1e-6)
    wv = O.quantize_values(vs, 2, 32)
    assert torch.equal(vdata[:, pk].cpu(), wv.data)
    assert torch.equal(vsc[:, pk].cpu(), wv.scales) and torch.equal(vz[:, pk].cpu(), wv.zeros)
    # (3) every value within half a quantisation step (plus the bf16 rounding of the per-op arithmetic)
    vt = vd[0].transpose(0, 1).float()                                  # (H, T, d)
    codes = torch.stack([(vdata >> s) & 3 for s in (0, 2, 4, 6)], dim=-1).reshape(H, T, d).float()
    sc = vsc.float().repeat_interleave(32, dim=-1)
    zr = vz.float().repeat_interleave(32, dim=-1)
    err = (codes * sc + zr - vt).abs()
    assert torch.all(err <= 0.5 * sc + 2.0 ** -6 * (vt.abs() + zr.abs() + sc) + 1e-6)
    # (4) MSE stage: relative distortion of the de-quantised unit vectors = the codebook's (within 5 %)
    kt = kd[0].transpose(0, 1).float()
    mse_hat = tq.mse_quantizer.dequantize(MSEQuantized(idx, norms, 2))
    rel = ((mse_hat - kt) ** 2).sum(-1) / (kt ** 2).sum(-1)
    theory = float(get_codebook(d, 2)["mse_total"])
    _progress(f"   relative MSE distortion {rel.mean().item():.5f}, codebook {theory:.5f}")
    assert abs(rel.mean().item() - theory) <= 0.05 * theory
    # (5) the inner-product estimator is unbiased: the slope of estimate on truth over all tokens is 1
    q = torch.randn(H, 4, d, generator=g).to(gpu)
    code = ProdQuantized(idx, sgn, rnorms, norms, 2)
    est = tq.attention_score(q, code)                                   # (H, 4, T)
    true = torch.einsum("hqd,htd->hqt", q, kt)
    slope = (est * true).sum() / (true * true).sum()
    _progress(f"   estimator slope {slope.item():.5f}")
    assert abs(slope.item() - 1.0) < 0.01


def test_config3_full_size_decode_against_the_oracle(gpu):
    """The GQA decode workload at its full size (16 sequences x 8192 tokens, 32 query / 8 KV heads of 128,
    3-bit keys, 4-bit values in groups of 32, physical pages a random permutation): every sequence against
    the oracle on the same store (score.py:84-173), and the split count must not matter."""
    _progress("config 3 full size: 16 x 8192, 32 / 8 heads of 128")
    worst = _decode_case(gpu, 128, 3, 4, 16, 32, 8, [8192] * 16, None, seed=2)
    _progress(f"   worst cosine over 16 sequences {worst:.7f}")
    worst = _decode_case(gpu, 128, 3, 4, 4, 32, 8, [8192, 8191, 4097, 8192], [128, 0, 5, 64], seed=3, n_split=7)
    _progress(f"   ragged, hybrid, 7 splits: worst cosine {worst:.7f}")


@pytest.mark.parametrize("d,key_bits,vb,dtype", [(128, 3, 4, torch.bfloat16), (256, 3, 2, torch.bfloat16),
                                                   (64, 2, 2, torch.float16)])
def test_append_ragged_equals_one_append_per_sequence(gpu, d, key_bits, vb, dtype):
    """tq_append_kv_ragged writes a step's ragged rows (several sequences, each continuing at its own
    position, store.py:73-90 per sequence) in one call; the pages must equal, byte for byte, one
    tq_append_kv_paged call per sequence."""
    g = torch.Generator().manual_seed(7 * d + vb)
    H, per_seq = 2, 12
    runs = [37, 0, 1, 150, 16, 5]
    starts = [0, 20, 33, 7, 16, 170]
    B, n_pages = len(runs), len(runs) * per_seq
    rows = sum(runs) + 9                                               # a few rows that belong to nobody
    k = torch.randn(rows, H, d, generator=g).to(dtype).to(gpu)
    v = torch.randn(rows, H, d, generator=g).to(dtype).to(gpu)
    table = torch.randperm(n_pages, generator=g).view(B, per_seq).to(torch.int32).to(gpu)
    row0 = [3]                                                         # the first run does not start at row 0
    for r in runs[:-1]:
        row0.append(row0[-1] + r)
    _progress(f"append_ragged d={d} {dtype} runs={runs} starts={starts}")
    pa, _ = _make_pool(gpu, d, key_bits, vb, H, n_pages, dtype)
    pb, _ = _make_pool(gpu, d, key_bits, vb, H, n_pages, dtype)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    pa.append_ragged(k, v, i32(row0), i32(runs), i32(starts), table, max_run=max(runs))
    for b in range(B):
        if runs[b]:
            pb.append(k[None, row0[b]:row0[b] + runs[b]], v[None, row0[b]:row0[b] + runs[b]], table[b:b + 1],
                      start_pos=i32([starts[b]]))
    torch.cuda.synchronize()
    assert torch.equal(pa.data, pb.data)
