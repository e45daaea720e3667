"""CPU: the oracle against the reference's golden vectors, known answers and
what the mathematics fixes.  These tests pin the oracle; the GPU tests then
compare the HIP kernels with the pinned oracle."""

import itertools
import math

import numpy as np
import pytest
import torch

from oracle import tq_oracle as O
from tests.helpers import key_code, value_code, cosine

SHIPPED = [(64, 1), (64, 2), (64, 3), (64, 4), (128, 1), (128, 2), (128, 3), (128, 4), (576, 3)]


# ---------------------------------------------------------------- codebooks
@pytest.mark.parametrize("d,bits", [(64, 1), (64, 2), (128, 1), (128, 2), (128, 3), (256, 1), (256, 2), (256, 3)])
def test_codebook_solver_reproduces_reference_files(golden, d, bits):
    ref = golden.codebook(d, bits)
    got = O.lloyd_max_codebook(d, bits)
    assert np.allclose(got["centroids"], ref["centroids"], rtol=0, atol=1e-15)
    assert np.allclose(got["boundaries"], ref["boundaries"], rtol=0, atol=1e-15)
    assert abs(got["mse_total"] - ref["mse_total"]) < 1e-14
    # what the kernels consume is the fp32 cast: that must be identical
    assert np.array_equal(np.float32(got["centroids"]), np.float32(ref["centroids"]))
    assert np.array_equal(np.float32(got["boundaries"]), np.float32(ref["boundaries"]))


@pytest.mark.parametrize("d", [64, 128, 256, 576])
def test_one_bit_codebook_closed_form(d):
    # b=1: c = E|x| = Gamma(d/2) / (sqrt(pi) Gamma((d+1)/2)), mse = 1/d - c^2
    from scipy.special import gammaln
    c = math.exp(gammaln(d / 2) - gammaln((d + 1) / 2)) / math.sqrt(math.pi)
    got = O.lloyd_max_codebook(d, 1)
    assert got["centroids"][0] == pytest.approx(-c, rel=1e-9)
    assert got["centroids"][1] == pytest.approx(c, rel=1e-9)
    assert got["mse_per_coord"] == pytest.approx(1.0 / d - c * c, rel=1e-7)


@pytest.mark.parametrize("d,bits", SHIPPED)
def test_shipped_codebook_invariants(golden, d, bits):
    cb = golden.codebook(d, bits)
    c, b = np.array(cb["centroids"]), np.array(cb["boundaries"])
    assert len(c) == 2 ** bits and len(b) == 2 ** bits + 1
    assert b[0] == -1.0 and b[-1] == 1.0
    assert np.all(np.diff(c) > 0)
    assert np.allclose(b[1:-1], (c[:-1] + c[1:]) / 2, atol=1e-16)
    assert np.allclose(c, -c[::-1], atol=1e-15)               # symmetric density
    assert cb["mse_total"] == pytest.approx(cb["mse_per_coord"] * d)


def test_pdf_integrates_to_one():
    from scipy import integrate
    for d in (64, 128, 256):
        mass, _ = integrate.quad(lambda t: O.sphere_coord_pdf(np.array([t]), d)[0], -1, 1)
        assert mass == pytest.approx(1.0, abs=1e-8)
        var, _ = integrate.quad(lambda t: t * t * O.sphere_coord_pdf(np.array([t]), d)[0], -1, 1)
        assert var == pytest.approx(1.0 / d, rel=1e-6)


# ---------------------------------------------------------------- packing
@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("d", [128, 13])
def test_pack_indices_golden(golden, bits, d):
    z = golden.npz("packing")
    idx = torch.from_numpy(z[f"idx_b{bits}_d{d}"])
    assert np.array_equal(O.pack_indices(idx, bits).numpy(), z[f"packed_b{bits}_d{d}"])
    assert np.array_equal(O.unpack_indices(torch.from_numpy(z[f"packed_b{bits}_d{d}"]), bits, d).numpy(),
                          z[f"unpacked_b{bits}_d{d}"])


def test_pack_indices_every_byte_value():
    # brute force over every byte: unpack(pack(x)) == x and pack follows sum idx_j << (eff*j)
    for bits in (1, 2, 3, 4):
        eff, per = O.packing_params(bits)
        combos = torch.tensor(list(itertools.product(range(2 ** bits), repeat=per))) if 2 ** (bits * per) <= 65536 \
            else torch.randint(0, 2 ** bits, (4096, per))
        packed = O.pack_indices(combos, bits)
        want = sum(combos[:, j].numpy().astype(np.int64) << (eff * j) for j in range(per))
        assert np.array_equal(packed[:, 0].numpy().astype(np.int64), want)
        assert torch.equal(O.unpack_indices(packed, bits, per), combos.long())


def test_sign_pack_golden_and_strictness(golden):
    z = golden.npz("packing")
    for d in (64, 13):
        assert np.array_equal(O.pack_signs(torch.from_numpy(z[f"proj_d{d}"])).numpy(), z[f"signs_d{d}"])
    assert np.array_equal(O.unpack_signs(torch.from_numpy(z["signs_d64"]), 64).numpy(), z["signs_unpacked_d64"])
    p = torch.tensor([[0.0, -0.0, 1e-30, -1e-30, float("nan"), 1.0, -1.0, float("inf")]])
    assert O.pack_signs(p).item() == (1 << 2) | (1 << 5) | (1 << 7)      # zero and NaN give bit 0


def test_bucketize_matches_searchsorted_and_brute_force():
    thr = torch.tensor([-0.3, -0.1, 0.0, 0.2])
    y = torch.tensor([-1.0, -0.3, -0.2999, -0.1, 0.0, 1e-9, 0.2, 0.5, float("nan"), float("inf"), -float("inf")])
    got = O.bucketize(y, thr)
    assert torch.equal(got, torch.searchsorted(thr, y))
    brute = torch.tensor([sum(1 for t in thr.tolist() if not (v <= t)) for v in y.tolist()])
    assert torch.equal(got, brute)


# ---------------------------------------------------------------- matrices
@pytest.mark.parametrize("d,seed", [(64, 42), (128, 42), (128, 63), (256, 42)])
def test_rotation_is_orthogonal_with_positive_r_diagonal(d, seed):
    Pi = O.rotation_matrix(d, seed)
    assert (Pi @ Pi.T - torch.eye(d)).abs().max() < 2e-6
    g = torch.Generator().manual_seed(seed)
    G = torch.randn(d, d, generator=g)
    R = Pi.T @ G                                   # G = Q R with Q = Pi  =>  R upper triangular, diag > 0
    assert torch.all(torch.diag(R) > 0)
    assert R.tril(-1).abs().max() < 1e-4
    S = O.qjl_matrix(d, seed + 1000)
    g2 = torch.Generator().manual_seed(seed + 1000)
    assert torch.equal(S, torch.randn(d, d, generator=g2))


# ---------------------------------------------------------------- key quantiser vs reference vectors
def test_key_cases_match_reference(golden):
    for file, case in golden.key_case_list():
        prm = golden.key_params(file, case)
        x = golden.tensor(file, case + ".x")
        q = golden.tensor(file, case + ".q")
        code = O.prod_quantize(x, prm)
        z = golden.npz(file)
        assert np.array_equal(code.mse_indices.numpy(), z[case + ".mse_indices"]), case
        assert np.array_equal(code.qjl_signs.numpy(), z[case + ".qjl_signs"]), case
        assert code.norms.dtype == x.dtype
        assert torch.equal(code.norms, golden.tensor(file, case + ".norms")), case
        assert np.array_equal(code.residual_norms.numpy(), z[case + ".residual_norms"]), case
        assert np.array_equal(code.y.numpy(), z[case + ".y"], equal_nan=True), case
        assert np.array_equal(code.p.numpy(), z[case + ".p"], equal_nan=True), case
        assert np.array_equal(O.prod_dequantize(code, prm).numpy(), z[case + ".dequant"]), case
        assert np.array_equal(O.attention_score(q, code, prm).numpy(), z[case + ".scores"]), case


def _config1_inputs():
    g = torch.Generator(device="cpu").manual_seed(0)
    K = torch.randn(4096, 128, generator=g, dtype=torch.float32)
    K = K / K.norm(dim=-1, keepdim=True)
    K = K * (0.5 + 1.5 * torch.rand(4096, generator=g)).unsqueeze(-1)
    Q = torch.randn(32, 128, generator=g, dtype=torch.float32)
    Q = Q / Q.norm(dim=-1, keepdim=True)
    Q = Q * (0.5 + 1.5 * torch.rand(32, generator=g)).unsqueeze(-1)
    return K, Q


def test_config1_round_trip_matches_reference(golden):
    z = golden.npz("config1_full")
    K, Q = _config1_inputs()
    assert np.array_equal(K[:256].numpy(), z["K_head"]) and np.array_equal(Q.numpy(), z["Q"])
    prm = O.KeyParams(torch.from_numpy(z["Pi"]), torch.from_numpy(z["S"]), torch.from_numpy(z["centroids"]),
                      torch.from_numpy(z["thresholds"]), 2)
    code = O.prod_quantize(K, prm)
    # same Pi, but another host's BLAS may order the fp32 sums differently: allow a handful of
    # near-threshold flips (0 on the machine that wrote the fixture)
    assert (code.mse_indices.numpy() != z["mse_indices"]).sum() <= 4
    assert (code.qjl_signs.numpy() != z["qjl_signs"]).sum() <= 8
    assert torch.equal(code.norms, torch.from_numpy(z["norms"])) or \
        (code.norms - torch.from_numpy(z["norms"])).abs().max() < 1e-6
    ref_code = key_code(torch.from_numpy(z["mse_indices"]), torch.from_numpy(z["qjl_signs"]),
                        torch.from_numpy(z["residual_norms"]), torch.from_numpy(z["norms"]), 2)
    scores = O.attention_score(Q, ref_code, prm)
    ref = torch.from_numpy(z["scores"])
    rms = ref.pow(2).mean().sqrt()
    assert (scores - ref).abs().max() <= 1e-5 * rms
    # packing of the reference's own rotated / projected tensors is bit exact
    assert np.array_equal(O.pack_indices(O.bucketize(torch.from_numpy(z["y_head"]), prm.thresholds), 2).numpy(),
                          z["mse_indices"][:256])
    assert np.array_equal(O.pack_signs(torch.from_numpy(z["p_head"])).numpy(), z["qjl_signs"][:256])


def test_score_identity_fused_form_equals_dequant_matmul(golden):
    # <q, x_mse + x_qjl> computed three ways: dense dequant + matmul, the reference's split
    # form, and the rotated-query form the kernels use (float64 referee)
    case = "bf16_d128_b3"
    prm = golden.key_params("key_cases", case)
    x = golden.tensor("key_cases", case + ".x")
    q = golden.tensor("key_cases", case + ".q")
    code = O.prod_quantize(x, prm)
    dense = torch.matmul(q.double(), O.prod_dequantize(code, prm).double().transpose(-2, -1))
    split = O.attention_score(q, code, prm).double()
    fused = O.fused_score(q, code, prm)
    scale = dense.pow(2).mean().sqrt()
    assert (split - dense).abs().max() < 1e-5 * scale
    assert (fused - dense).abs().max() < 1e-5 * scale


def test_estimator_statistics_match_readme_table():
    # unbiasedness (relative bias < 0.1 % in the README; here a looser Monte-Carlo bound),
    # residual norm ~ ||x|| sqrt(mse_total), qjl_scale = sqrt(pi/2)/d
    d = 128
    prm = O.make_key_params(d, 3, O.lloyd_max_codebook(d, 2))
    assert prm.qjl_scale == pytest.approx(math.sqrt(math.pi / 2) / d)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(4096, d, generator=g)
    q = torch.randn(64, d, generator=g)
    code = O.prod_quantize(x, prm)
    est = O.attention_score(q, code, prm)
    true = q @ x.T
    err = est - true
    assert abs(err.mean()) < 0.02 * true.abs().mean()
    ratio = (code.residual_norms / x.norm(dim=-1)).mean()
    assert ratio == pytest.approx(math.sqrt(0.11600007), rel=0.02)
    # MSE-only reconstruction distortion equals the codebook's mse_total
    xm = O.mse_dequantize(code.mse_indices, code.norms, prm)
    rel = ((x - xm).norm(dim=-1) / x.norm(dim=-1)).pow(2).mean()
    assert rel == pytest.approx(0.11600007, rel=0.03)


# ---------------------------------------------------------------- values
def test_value_quantiser_matches_reference(golden):
    for case in golden.cases("values"):
        tag, b, g = case.split("_")
        bits, gs = int(b[1:]), int(g[1:])
        v = golden.tensor("values", case + ".v")
        code = O.quantize_values(v, bits, gs)
        z = golden.npz("values")
        assert np.array_equal(code.data.numpy(), z[case + ".data"]), case
        assert torch.equal(code.scales, golden.tensor("values", case + ".scales")), case
        assert torch.equal(code.zeros, golden.tensor("values", case + ".zeros")), case
        assert code.scales.dtype == v.dtype
        assert np.array_equal(O.dequantize_values(code, gs).numpy(), z[case + ".dequant"], equal_nan=True), case


def test_value_quantiser_error_bound_and_brute_force():
    g = torch.Generator().manual_seed(3)
    v = torch.randn(5, 7, 64, generator=g)
    for bits in (2, 4, 8):
        code = O.quantize_values(v, bits, 32)
        deq = O.dequantize_values(code, 32)
        half = code.scales.unsqueeze(-1).expand(5, 7, 2, 32).reshape(5, 7, 64) / 2
        assert torch.all((v - deq).abs() <= half * (1 + 1e-5) + 1e-7)
        # brute force one group
        grp = v[0, 0, :32]
        lo, hi = grp.min(), grp.max()
        sc = max((hi - lo) / (2 ** bits - 1), torch.tensor(1e-10))
        want = torch.clamp(torch.round((grp - lo) / sc), 0, 2 ** bits - 1).to(torch.uint8)
        assert torch.equal(O.unpack_values(code.data, bits)[0, 0, :32], want)


# ---------------------------------------------------------------- attention
def test_hybrid_attention_matches_reference(golden):
    z = golden.npz("hybrid")
    for case in golden.cases("hybrid"):
        H, G, d, n_hist, n_recent, vb = [int(v) for v in z[case + ".meta"]]
        cb = golden.codebook(d, 2)
        cent, _, thr = O.codebook_tensors(cb)
        prm = O.KeyParams(torch.from_numpy(z[case + ".Pi"]), torch.from_numpy(z[case + ".S"]), cent, thr, 2)
        q = golden.tensor("hybrid", case + ".q")
        kc = vc = None
        if n_hist:
            k = golden.tensor("hybrid", case + ".k").transpose(0, 1)      # (H, N, d)
            v = golden.tensor("hybrid", case + ".v").transpose(0, 1)
            half = n_hist // 2
            parts = [O.prod_quantize(k[:, :half], prm), O.prod_quantize(k[:, half:], prm)]
            kc = key_code(torch.cat([p.mse_indices for p in parts], 1), torch.cat([p.qjl_signs for p in parts], 1),
                          torch.cat([p.residual_norms for p in parts], 1), torch.cat([p.norms for p in parts], 1), 2)
            assert np.array_equal(kc.mse_indices.numpy(), z[case + ".mse_indices"]), case
            assert np.array_equal(kc.qjl_signs.numpy(), z[case + ".qjl_signs"]), case
            vq = O.quantize_values(v, vb, 32)
            assert np.array_equal(vq.data.numpy(), z[case + ".v_data"]), case
            vc = vq
            per_tok = 32 + 16 + 2 + 2 + d * vb // 8 + 2 * 2 * (d // 32)
            assert int(z[case + ".memory_bytes"]) == n_hist * H * per_tok
        rk = golden.tensor("hybrid", case + ".recent_k") if n_recent else None
        rv = golden.tensor("hybrid", case + ".recent_v") if n_recent else None
        out = O.hybrid_attention(q, kc, vc, n_hist, prm, H, rk, rv)
        ref = golden.tensor("hybrid", case + ".out")
        assert out.dtype == ref.dtype
        assert (out.float() - ref.float()).abs().max() <= 2 ** -8 * ref.float().abs().max(), case
        assert cosine(out, ref) > 0.999999, case


def test_dense_attention_equals_sdpa():
    g = torch.Generator().manual_seed(5)
    q = torch.randn(3, 8, 64, generator=g)
    k = torch.randn(2, 50, 64, generator=g)
    v = torch.randn(2, 50, 64, generator=g)
    out = O.dense_gqa_attention(q, k, v, 2, 0.125)
    kk = k.repeat_interleave(4, dim=0)
    vv = v.repeat_interleave(4, dim=0)
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, scale=0.125).transpose(0, 1)
    assert (out - ref).abs().max() < 1e-5
    with pytest.raises(ValueError):
        O.dense_gqa_attention(torch.randn(1, 7, 64), k, v, 2, 0.125)


def test_kv_cache_object_golden(golden):
    # the stand-alone cache: scores = [estimator * scale ; exact buffer], attend = weights @ [deq ; buffer]
    z = golden.npz("kv_cache_object")
    d = 128
    cent, _, thr = O.codebook_tensors(golden.codebook(d, 2))
    prm = O.KeyParams(torch.from_numpy(z["Pi"]), torch.from_numpy(z["S"]), cent, thr, 2)
    k = torch.cat([torch.from_numpy(z["k"])] + [torch.from_numpy(z[f"append_k{i}"]) for i in range(5)], dim=-2)
    v = torch.cat([torch.from_numpy(z["v"])] + [torch.from_numpy(z[f"append_v{i}"]) for i in range(5)], dim=-2)
    n_q = 45 - 16                                      # buffer_size 16: everything older is compressed
    # the reference compressed 24 tokens at prefill and then one per append
    chunks = [(0, 24)] + [(24 + i, 25 + i) for i in range(5)]
    codes = [O.prod_quantize(k[..., a:b, :], prm) for a, b in chunks]
    kc = key_code(torch.cat([c.mse_indices for c in codes], -2), torch.cat([c.qjl_signs for c in codes], -2),
                  torch.cat([c.residual_norms for c in codes], -1), torch.cat([c.norms for c in codes], -1), 2)
    q = torch.from_numpy(z["q"])
    s = torch.cat([O.attention_score(q, kc, prm) / math.sqrt(d), (q @ k[..., n_q:, :].transpose(-2, -1)) / math.sqrt(d)], -1)
    assert (s - torch.from_numpy(z["scores"])).abs().max() < 1e-5
    assert int(z["seq_len"]) == 45


# ---------------------------------------------------------------- write-side policy
def test_capture_model_matches_reference_trace(golden):
    for tr in golden.json("capture_trace.json"):
        m = O.CaptureModel(tr["capacity"])
        if tr.get("double_prefill"):
            m.ingest_prefill([0, 1, 2])
            m.ingest_prefill([10, 11, 12])
        else:
            tok = 0
            if tr["prefill"]:
                m.ingest_prefill(list(range(tr["prefill"])))
                tok = tr["prefill"]
            for _ in range(tr["decodes"]):
                m.ingest_decode([tok])
                tok += 1
            if tr["flush"]:
                m.flush()
            assert len(m.compressed) == tr["total_compressed"]
            assert len(m.ring.items) == tr["total_buffered"]
            assert m.ring.total_written == tr["ring_total_written"]
        assert m.chunks == tr["chunks"]
        assert m.ring.items == tr["ring"]
