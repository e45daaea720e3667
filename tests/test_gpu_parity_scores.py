"""GPU: the scores the page-streaming kernels compute in flight, the long-context workload at its full
size, and the wide-head (576) quantiser - each through the C ABI against the pinned oracle.

The fused decode kernels never write a score; what they do write per (sequence, query head, split) is the
partial (running maximum m, sum l of exp(score - m), accumulator).  m + log l is the log-sum-exp of the
scores of the sequence's tokens, so a family of sequences that share one block table and have lengths
1, 2, 3, ... gives every token's score as a difference of neighbouring sums."""

import math

import numpy as np
import pytest
import torch

from oracle import tq_oracle as O
from tests.helpers import bit_mismatch, byte_mismatch, cosine, key_code, params_of, value_code
from tests.test_gpu_parity import COS_GATE, FLIP_RATE, SCORE_TOL, _decode_case, _make_pool, _progress, _store_from_oracle_view

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("d,key_bits,vb,G,dtype", [(128, 3, 4, 8, torch.bfloat16), (128, 2, 2, 8, torch.bfloat16),
                                                   (128, 4, 4, 8, torch.bfloat16), (256, 3, 2, 8, torch.bfloat16),
                                                   (256, 4, 2, 8, torch.bfloat16), (256, 2, 4, 5, torch.float16),
                                                   (128, 3, 2, 3, torch.float16), (64, 3, 2, 4, torch.bfloat16),
                                                   (128, 5, 4, 8, torch.bfloat16)])
def test_scores_inside_the_decode_kernels_meet_the_score_gate(gpu, d, key_bits, vb, G, dtype):
    """sm_scale * TurboQuantProd.attention_score (quantizer.py:274-302) as the page kernels compute it
    from the packed pages: matrix-core kernel (head_dim 128 / 256, up to 4-bit keys) and the general kernel
    (head_dim 64, 5-bit keys).  Gate: |delta| <= 1e-3 * rms(scores) on the same stored bytes."""
    Hkv, N = 2, 192
    Hq = Hkv * G
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, N // 16 + 2, dtype, seed=42 + 7 * key_bits)
    g = torch.Generator().manual_seed(1000 + d + key_bits)
    k = torch.randn(1, N, Hkv, d, generator=g).to(dtype)
    k = k * (0.25 + 1.5 * torch.rand(1, N, Hkv, 1, generator=g)).to(dtype)       # norms that differ per token
    v = torch.randn(1, N, Hkv, d, generator=g).to(dtype)
    q0 = torch.randn(Hq, d, generator=g).to(dtype)
    table = torch.randperm(N // 16 + 2, generator=g)[: N // 16].to(torch.int32).to(gpu)
    pool.append(k.to(gpu), v.to(gpu), table[None, :])
    # sequence b = the first b + 1 tokens of the same pages; scores with a spread of about 0.4, so that
    # no token is a negligible share of a sum it has to be recovered from
    sm_scale = 0.4 / math.sqrt(d)
    B = N
    q = q0[None].expand(B, Hq, d).contiguous().to(gpu)
    seq = torch.arange(1, B + 1, dtype=torch.int32, device=gpu)
    ws = pool.workspace(B, Hq, 1)
    _progress(f"in-kernel scores d={d} kb={key_bits} vb={vb} G={G} {dtype}")
    pool.decode_attention(q, table, seq, scale=sm_scale, n_split=1, workspace=ws, stages=3)
    torch.cuda.synchronize()
    parts = ws[: B * Hq * 2 * (d + 2)].view(B, Hq, 2, d + 2)[:, :, 0, :2].double().cpu()
    lse = parts[..., 0] + parts[..., 1].log()                                       # (B, Hq)
    rel = (lse - lse[-1:]).exp()                                                   # prefix sums / the total
    w = torch.cat([rel[:1], rel[1:] - rel[:-1]], dim=0)                            # share of token t
    assert torch.all(w > 0)
    got = (w.log() + lse[-1:]).transpose(0, 1)                                     # (Hq, N) scaled scores
    kc, _ = _store_from_oracle_view(pool, table, N)
    want = sm_scale * O.attention_score(q0.view(Hkv, G, d), kc, params_of(tq)).double().reshape(Hq, N)
    rms = want.pow(2).mean().sqrt()
    err = (got - want).abs().max()
    _progress(f"   max |delta| {err:.3e} = {err / rms:.2e} x rms(scores)")
    assert err <= SCORE_TOL * rms


def _student_t(shape, nu, gen):
    """z / sqrt(chi2_nu / nu) element-wise, chi2 as the sum of nu squared normals."""
    z = torch.randn(shape, generator=gen)
    c = torch.zeros(shape)
    for _ in range(nu):
        c.add_(torch.randn(shape, generator=gen).square_())
    return z.div_(c.div_(nu).sqrt_())


def test_config4_full_size_decode_against_the_oracle(gpu):
    """The long-context decode workload at its full size: 4 sequences x 131072 tokens, 16 query / 2 KV heads
    of 256, 3-bit keys, 2-bit values in groups of 32, bf16 Student-t (nu = 5) keys and values from a CPU
    generator seeded 3, physical pages a random permutation, default split count.  Every sequence against
    the oracle's de-quantise-everything attention on the same store (score.py:84-173)."""
    B, Hq, Hkv, d, N = 4, 16, 2, 256, 131072
    pages = N // 16
    pool, tq = _make_pool(gpu, d, 3, 2, Hkv, B * pages, torch.bfloat16, seed=42)
    g = torch.Generator().manual_seed(3)
    table = torch.randperm(B * pages, generator=g).to(torch.int32).view(B, pages).to(gpu)
    for b in range(B):
        _progress(f"config 4: sequence {b}: Student-t keys / values, quantise")
        k = _student_t((1, N, Hkv, d), 5, g).bfloat16().to(gpu)
        v = _student_t((1, N, Hkv, d), 5, g).bfloat16().to(gpu)
        pool.append(k, v, table[b:b + 1])
        del k, v
    q = torch.randn(B, Hq, d, generator=g).bfloat16()
    seq = torch.full((B,), N, dtype=torch.int32, device=gpu)
    out = pool.decode_attention(q.to(gpu), table, seq, max_len=N).cpu()
    torch.cuda.synchronize()
    prm = params_of(tq)
    for b in range(B):
        kc, vc = _store_from_oracle_view(pool, table[b], N)
        want = O.hybrid_attention(q[b:b + 1], kc, vc, N, prm, Hkv, None, None)
        c = cosine(out[b:b + 1], want)
        _progress(f"config 4: sequence {b} cosine {c:.8f}")
        assert c >= COS_GATE, (b, c)
        assert (out[b:b + 1].float() - want.float()).abs().max() <= 2 ** -7 * want.float().abs().max() + 1e-3, b


def test_config5_layer_at_full_size_against_the_oracle(gpu):
    """One attention layer of the 32-layer serving step at its full size: batch 32 x 32768 context tokens, 32
    query / 8 KV heads of 128, 3-bit keys, 4-bit values in groups of 32 (the shape every layer of the
    backend decode-step benchmark runs), pages a random permutation, default split count, sequences of
    unequal length.  Every sequence against the oracle's de-quantise-everything attention on the same store
    (score.py:84-173)."""
    B, Hq, Hkv, d, N = 32, 32, 8, 128, 32768
    pages = N // 16
    pool, tq = _make_pool(gpu, d, 3, 4, Hkv, B * pages, torch.bfloat16, seed=42 + 7 * 5)
    g = torch.Generator().manual_seed(5)
    table = torch.randperm(B * pages, generator=g).to(torch.int32).view(B, pages).to(gpu)
    gg = torch.Generator(device=gpu).manual_seed(5)         # keys and values straight on the card (1 GB of them)
    for b0 in range(0, B, 4):
        _progress(f"config 5 layer: sequences {b0}..{b0 + 3}: quantise")
        k = torch.randn(4, N, Hkv, d, generator=gg, device=gpu).bfloat16()
        v = torch.randn(4, N, Hkv, d, generator=gg, device=gpu).bfloat16()
        pool.append(k, v, table[b0:b0 + 4])
        del k, v
    q = torch.randn(B, Hq, d, generator=g).bfloat16()
    lens = torch.randint(N // 2, N + 1, (B,), generator=g).to(torch.int32)
    lens[0], lens[B - 1] = N, N // 2 + 3
    out = pool.decode_attention(q.to(gpu), table, lens.to(gpu), max_len=N).cpu()
    torch.cuda.synchronize()
    prm = params_of(tq)
    worst = 1.0
    for b in range(B):
        n = int(lens[b])
        kc, vc = _store_from_oracle_view(pool, table[b], n)
        want = O.hybrid_attention(q[b:b + 1], kc, vc, n, prm, Hkv, None, None)
        c = cosine(out[b:b + 1], want)
        worst = min(worst, c)
        assert c >= COS_GATE, (b, c)
    _progress(f"config 5 layer: all {B} sequences, worst cosine {worst:.8f} (1 - cos = {1 - worst:.2e})")


@pytest.mark.parametrize("d,key_bits,dtype", [(576, 4, torch.bfloat16), (576, 3, torch.float32), (192, 4, torch.float16)])
def test_wide_head_quantiser_against_the_oracle(gpu, d, key_bits, dtype):
    """Head sizes without a matrix-core quantiser (the fp32 vector-ALU kernel): 576 with 4-bit keys is the shape
    the reference ships a codebook for (codebook_d576_b3.json; integration/vllm.py:378-379 sizes a layer from
    kv_lora_rank).  Bytes against the oracle on the same Pi / S (quantizer.py:231-257): a coordinate that
    sits on a threshold may flip with the fp32 summation order, bounded at 1e-4 per coordinate; norms and
    residual norms to rounding; all-zero vectors byte for byte."""
    from turboquant_amd.quantizer import TurboQuantProd
    tq = TurboQuantProd(d, bits=key_bits, device=gpu, seed=49)
    prm = params_of(tq)
    g = torch.Generator().manual_seed(d + key_bits)
    n = 300
    x = torch.randn(n, d, generator=g)
    x[:, torch.randperm(d, generator=g)[:4]] *= 20.0
    x[7] = 0.0
    x[n - 1] = 0.0
    x = x.to(dtype)
    _progress(f"wide quantiser d={d} kb={key_bits} {dtype}")
    code = tq.quantize(x.to(gpu))
    torch.cuda.synchronize()
    want = O.prod_quantize(x, prm)
    n_coord = x.numel()
    idx_flips = byte_mismatch(code.mse_indices, want.mse_indices)
    sgn_flips = bit_mismatch(code.qjl_signs, want.qjl_signs)
    _progress(f"   index bytes differing {idx_flips}, sign bits differing {sgn_flips} of {n_coord}")
    assert idx_flips <= max(1, FLIP_RATE * n_coord) and sgn_flips <= max(2, FLIP_RATE * n_coord)
    for row in (7, n - 1):
        assert torch.equal(code.mse_indices[row].cpu(), want.mse_indices[row])
        assert torch.equal(code.qjl_signs[row].cpu(), want.qjl_signs[row])
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else (2.0 ** -10 if dtype == torch.float16 else 2.0 ** -22)
    assert torch.all((code.norms.float().cpu() - want.norms.float()).abs() <= ulp * want.norms.float().abs() + 1e-30)
    assert torch.allclose(code.residual_norms.cpu(), want.residual_norms, rtol=3e-5, atol=1e-6)
    # the paged sink of the same kernel writes the same codes
    pool, _ = _make_pool(gpu, d, key_bits, 2, 1, n // 16 + 2, dtype if dtype != torch.float32 else torch.float32, seed=49)
    table = torch.arange(n // 16 + 1, dtype=torch.int32, device=gpu)[None, :]
    pool.append(x.to(gpu)[None, :, None, :], x.to(gpu)[None, :, None, :], table)
    idx, sgn, norms, rnorms, _, _, _ = pool.export_flat(table[0], n)
    torch.cuda.synchronize()
    assert torch.equal(idx[0], code.mse_indices) and torch.equal(sgn[0], code.qjl_signs)
    assert torch.equal(norms[0], code.norms) and torch.equal(rnorms[0], code.residual_norms)


@pytest.mark.parametrize("d,key_bits", [(128, 5), (576, 4)])
def test_all_zero_vectors_land_in_the_reference_bucket(gpu, golden, d, key_bits):
    """Two of the reference's tables (codebook_d128_b4.json, codebook_d576_b3.json) hold a tiny negative
    middle threshold instead of 0, so a coordinate that is exactly 0 - every coordinate of an all-zero key,
    e.g. a padding row - belongs to the bucket above the middle (searchsorted, quantizer.py:144).  Flat and
    paged quantisers must pack exactly those bytes."""
    from turboquant_amd.quantizer import TurboQuantProd
    mb = key_bits - 1
    ref_thr = torch.tensor(golden.codebook(d, mb)["boundaries"][1:-1], dtype=torch.float32)
    assert ref_thr[len(ref_thr) // 2] < 0
    for dtype in (torch.bfloat16, torch.float32):
        tq = TurboQuantProd(d, bits=key_bits, device=gpu)
        assert torch.equal(tq.mse_quantizer.decision_boundaries.cpu(), ref_thr)
        x = torch.zeros(20, d, dtype=dtype)
        code = tq.quantize(x.to(gpu))
        want = O.prod_quantize(x, params_of(tq))
        assert int(want.mse_indices[0, 0]) == (1 << (mb - 1)) * 0x11           # both nibbles: upper middle bucket
        assert torch.equal(code.mse_indices.cpu(), want.mse_indices)
        assert torch.equal(code.qjl_signs.cpu(), want.qjl_signs)
        assert torch.count_nonzero(code.norms) == 0 and torch.count_nonzero(code.residual_norms) == 0
        pool, _ = _make_pool(gpu, d, key_bits, 2, 1, 4, dtype)
        table = torch.arange(2, dtype=torch.int32, device=gpu)[None, :]
        pool.append(x.to(gpu)[None, :, None, :], x.to(gpu)[None, :, None, :], table)
        idx, sgn, _, _, _, _, _ = pool.export_flat(table[0], 20)
        assert torch.equal(idx[0].cpu(), want.mse_indices) and torch.equal(sgn[0].cpu(), want.qjl_signs)


@pytest.mark.parametrize("vb,Hq,Hkv,dtype", [(2, 16, 1, torch.bfloat16), (4, 8, 2, torch.float16)])
def test_decode_head_dim_576_with_4_bit_keys(gpu, vb, Hq, Hkv, dtype):
    """head_dim 576 with 4-bit keys (3-bit indices in nibbles): the shape of the only 576 table the reference
    ships, through the page kernel against the oracle on the same store."""
    _progress(f"decode d=576 kb=4 vb={vb} Hq={Hq} Hkv={Hkv} {dtype}")
    worst = _decode_case(gpu, 576, 4, vb, 2, Hq, Hkv, [300, 77], [0, 9], seed=900 + vb, dtype=dtype)
    _progress(f"   worst cosine {worst:.7f}")


# ------------------------------------------------------------------ head sizes above 256 on the matrix cores
@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,dtype,lens,recent,n_split", [
    (576, 4, 4, 8, 1, torch.bfloat16, [300, 77, 1], None, None),
    (576, 4, 2, 16, 1, torch.bfloat16, [300, 77], [0, 9], 3),          # 16 heads per KV head: two groups of 8; exact tail
    (576, 4, 8, 8, 2, torch.bfloat16, [130, 513], None, 2),            # 8-bit values (a ring of two blocks)
    (576, 4, 4, 8, 2, torch.float16, [300, 77], [5, 0], None),         # fp16 pages: zero points on the fp16 MFMA
    (576, 3, 4, 11, 1, torch.bfloat16, [700, 33], None, 4),            # 11 heads: groups of 6 and 5; 3-bit keys
    (512, 3, 4, 8, 2, torch.bfloat16, [300, 77], None, None),          # a multiple of 128: lane-major key words
    (512, 4, 2, 4, 4, torch.bfloat16, [64, 1000], None, 5),
    (320, 3, 2, 5, 1, torch.bfloat16, [257, 31], None, 2),             # five wavefronts, two and a half chunks
    (704, 3, 2, 8, 1, torch.bfloat16, [300, 77], None, None),          # the widest head the kernel takes
    (640, 2, 4, 3, 1, torch.bfloat16, [2100, 500], None, 2)])          # 2-bit keys; table registers move on (more than 64 pages)
def test_decode_wide_heads_on_the_matrix_cores(gpu, d, key_bits, vb, Hq, Hkv, dtype, lens, recent, n_split):
    """Head sizes above 256 (512 / 576: the latent sizes the reference's layer set-up meets, integration/vllm.py:376-381)
    run the matrix-core kernel that works on a block of 32 tokens per workgroup: against the oracle on the same
    store (ragged lengths, splits without tokens, an exact tail), and against the general kernel, which the
    option "wide_heads" = 0 selects."""
    pool, _ = _make_pool(gpu, d, key_bits, vb, Hkv, 4, dtype)
    assert pool.page_kernel() == 2, "the shape has no wide-head kernel"
    outs = {}
    # as shipped (operands packed by the rotation launch; head_dim 512 / 576: the instantiations with constant page
    # geometry); operands packed by every page-kernel workgroup; the instantiation that takes the geometry at run time
    # (what the other head sizes run); the general kernel
    # (bf16 and fp16 queries are rotated and packed on the matrix cores; "prep_mfma" = 0 leaves that to the vector ALU)
    variants = [("shipped", 1, 1, 1), ("packed in the page kernel", 1, 0, 1), ("rotated on the vector ALU", 1, 1, 0)]
    if d in (512, 576):
        variants.append(("geometry at run time", 2, 1, 1))
    variants.append(("general kernel", 0, 1, 1))
    try:
        for name, wide, pre, rot in variants:
            _set_option("wide_heads", wide)
            _set_option("wide_prepack", pre)
            _set_option("prep_mfma", rot)
            _progress(f"decode d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} {dtype} n_split={n_split}: {name}")
            outs[name] = _decode_case(gpu, d, key_bits, vb, len(lens), Hq, Hkv, lens, recent, seed=700 + d + vb,
                                      n_split=n_split, dtype=dtype, return_out=True)
    finally:
        _set_option("wide_heads", 1)
        _set_option("wide_prepack", 1)
        _set_option("prep_mfma", 1)
    for name in ("packed in the page kernel", "rotated on the vector ALU", "general kernel"):
        if name not in outs:
            continue
        c = cosine(outs["shipped"], outs[name])
        _progress(f"   shipped against {name}: cosine {c:.7f}")
        assert c >= COS_GATE
    if "rotated on the vector ALU" in outs:      # the same operands to rounding: outputs within a rounding step of the output type
        a, b = outs["shipped"].float(), outs["rotated on the vector ALU"].float()
        assert float((a - b).abs().max()) <= 2.0 ** -7 * float(a.abs().max())
    if "geometry at run time" in outs:
        assert torch.equal(outs["shipped"], outs["geometry at run time"]), "constant and run-time geometry disagree"


@pytest.mark.parametrize("d,rows", [(128, 20), (576, 20), (576, 7), (256, 33)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rotate_query_entry_point_on_every_input_dtype_and_alignment(gpu, d, rows, dtype):
    """tq_rotate_query: q_rot = q Pi^T, q_sk = q S^T (triton_kernels.py:527-528) in fp32, for queries of every input
    dtype.  Queries that start on a 16-byte boundary are staged with 16-byte loads, others element by element: the same
    bits either way, and within fp32 rounding of a float64 product."""
    import ctypes as C
    from turboquant_amd import _ffi
    from turboquant_amd.quantizer import TurboQuantProd
    tq = TurboQuantProd(d, bits=3, device=gpu, seed=5)
    ly = tq._layer()
    g = torch.Generator().manual_seed(17 * d + rows)
    q = torch.randn(rows, d, generator=g).to(dtype)
    buf = torch.zeros(rows * d + 8, dtype=dtype, device=gpu)
    outs = []
    for shift in (0, 1):                               # element offset of the queries inside a 16-byte aligned buffer
        buf[shift:shift + rows * d] = q.to(gpu).reshape(-1)
        q_rot = torch.empty(rows, d, dtype=torch.float32, device=gpu)
        q_sk = torch.empty(rows, d, dtype=torch.float32, device=gpu)
        with _ffi.on_device(gpu):
            _ffi.check(_ffi.lib().tq_rotate_query(buf.data_ptr() + shift * buf.element_size(), _ffi.dtype_tag(dtype), rows, C.byref(ly),
                                                  q_rot.data_ptr(), q_sk.data_ptr(), _ffi.stream_ptr(gpu)), "tq_rotate_query")
        torch.cuda.synchronize()
        outs.append((q_rot.cpu(), q_sk.cpu()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    q64 = q.double()
    for got, M in ((outs[0][0], tq.mse_quantizer.Pi), (outs[0][1], tq.S)):
        want = q64 @ M.detach().cpu().double().T
        assert float((got.double() - want).abs().max()) <= 1e-5 * float(want.abs().max())


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,lens,recent", [(576, 4, 4, 8, 1, [300, 77, 40], [128, 9, 0]),
                                                              (512, 3, 2, 16, 2, [130, 513], [100, 100])])
def test_hybrid_step_of_wide_heads_with_the_exact_tail_in_the_rotation_launch(gpu, d, key_bits, vb, Hq, Hkv, lens, recent):
    """A whole hybrid step (score.py:99-111 + 138-173) with bf16 queries at head_dim 512 / 576 runs the exact-tail
    workgroups in the launch of the matrix-core rotation.  The stages called apart (rotation, then tail + page
    kernel + merge as launches of their own) do the same arithmetic: same output, bit for bit."""
    g = torch.Generator().manual_seed(31 * d + vb)
    B, max_len = len(lens), max(lens)
    pages_per_seq = (max_len + 15) // 16
    pool, _ = _make_pool(gpu, d, key_bits, vb, Hkv, B * pages_per_seq + 2, torch.bfloat16)
    assert pool.page_kernel() == 2
    table = torch.randperm(B * pages_per_seq + 2, generator=g)[: B * pages_per_seq].to(torch.int32).reshape(B, pages_per_seq).to(gpu)
    k = torch.randn(B, max_len, Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, max_len, Hkv, d, generator=g).bfloat16().to(gpu)
    pool.append(k, v, table)
    q = torch.randn(B, Hq, d, generator=g).bfloat16().to(gpu)
    rk = torch.randn(B, max(recent), Hkv, d, generator=g).bfloat16().to(gpu)
    rv = torch.randn(B, max(recent), Hkv, d, generator=g).bfloat16().to(gpu)
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    rl = torch.tensor(recent, dtype=torch.int32, device=gpu)
    n_split = 3
    _progress(f"hybrid step d={d} lens={lens} recent={recent}: one call, then staged")
    whole = pool.decode_attention(q, table, seq, recent_k=rk, recent_v=rv, recent_len=rl, n_split=n_split, max_len=max_len).clone()
    ws = pool.workspace(B, Hq, n_split)
    staged = torch.empty_like(q)
    for stages in (1, 6):
        pool.decode_attention(q, table, seq, recent_k=rk, recent_v=rv, recent_len=rl, n_split=n_split, max_len=max_len,
                              workspace=ws, out=staged, stages=stages)
    torch.cuda.synchronize()
    assert torch.equal(whole, staged)
    # against the oracle on the first sequence (history and exact tokens)
    kc, vc = _store_from_oracle_view(pool, table[0], lens[0])
    ref = O.hybrid_attention(q[0:1].cpu(), kc, vc, max(lens[0], O.MIN_HISTORY), params_of(pool.quantizer), Hkv,
                             rk[0, :recent[0]].cpu(), rv[0, :recent[0]].cpu())
    assert cosine(whole[0:1].cpu(), ref) >= COS_GATE


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,dtype,lens,recent,n_split", [
    (576, 4, 4, 128, 1, torch.bfloat16, [300, 77], None, 2),           # multi-head latent attention: 128 heads on one latent
    (576, 4, 2, 120, 1, torch.bfloat16, [40, 17, 33, 16, 5, 64, 48, 31, 20], None, 1),     # 1080 query rows: the rotation takes
                                                                       # six row tiles per workgroup, the last tile half full
    (512, 3, 2, 40, 2, torch.bfloat16, [130, 513], [7, 0], None),      # 20 heads per KV head: groups of 7, 7, 6; exact tail
    (128, 3, 4, 71, 1, torch.bfloat16, [200, 37, 512], None, 2),       # multi-query attention with an odd head count
    (128, 4, 2, 64, 2, torch.float16, [300, 77], [9, 0], None),        # 32 heads per KV head, fp16, exact tail
    (256, 3, 2, 48, 2, torch.bfloat16, [700, 33], None, 4),            # 24 heads per KV head: three groups of 8
    (64, 3, 4, 20, 1, torch.bfloat16, [257, 31], None, None),          # head_dim 64: groups of 7, 7, 6
    (128, 3, 2, 40, 2, torch.float32, [200, 37], [5, 0], None),        # fp32 pages: the general kernel, groups of 10
    (192, 3, 4, 33, 1, torch.bfloat16, [300, 77], None, 3)])           # a head size of the general kernel: groups of 11
def test_decode_more_than_sixteen_query_heads_per_kv_head(gpu, d, key_bits, vb, Hq, Hkv, dtype, lens, recent, n_split):
    """_matmul_attend (score.py:138-173) takes any ratio of query heads to KV heads (multi-query and multi-head latent
    attention put 32 - 128 heads on one KV head): the matrix-core page kernels serve a KV head's heads in groups of at
    most 8, whatever their number up to 128, and the general kernel in groups of at most 16.  Every sequence against
    the oracle on the same store."""
    _progress(f"decode d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} {dtype}")
    worst = _decode_case(gpu, d, key_bits, vb, len(lens), Hq, Hkv, lens, recent, seed=1300 + Hq, n_split=n_split, dtype=dtype)
    _progress(f"   worst cosine {worst:.7f}")


def test_decode_head_dim_576_at_the_bench_shape_against_the_oracle(gpu):
    """Two sequences of the 16 x 8192 step bench.py times at head_dim 576 (8 query heads on one KV head, 4-bit keys,
    4-bit values; 16 splits of 16 blocks, the table registers of a workgroup move on): every sequence against the
    oracle on the same store."""
    _progress("decode d=576 at 2 x 8192")
    worst = _decode_case(gpu, 576, 4, 4, 2, 8, 1, [8192, 8000], None, seed=576, n_split=16)
    _progress(f"   worst cosine {worst:.7f}")


# ------------------------------------------------------------------ block tables are bounded on the device
@pytest.mark.parametrize("d,key_bits,vb,dtype,T", [(128, 3, 4, torch.bfloat16, 70), (256, 3, 2, torch.bfloat16, 5000),
                                                     (64, 2, 2, torch.float16, 70), (128, 3, 2, torch.float32, 40),
                                                     (128, 3, 4, torch.bfloat16, 8192)])
def test_append_never_writes_through_a_bad_table_entry(gpu, d, key_bits, vb, dtype, T):
    """A block table is device data the host cannot check.  Entries outside [0, num_pages) (stale, poisoned or
    negative) and runs that continue past the end of the table row must leave every byte of the pool as it
    was and return normally; the tokens of the good pages are written as usual.  (Small and large appends:
    the tile kernels, the chunk kernels, the matrix-core key kernel and the side-stream path.)"""
    H = 8 if T >= 8192 else 2                      # 8192 tokens x 8 heads: large enough for the side-stream path
    n_log = (T + 15) // 16
    n_pages = n_log + 3
    g = torch.Generator().manual_seed(T + d)
    k = torch.randn(1, T, H, d, generator=g).to(dtype).to(gpu)
    v = torch.randn(1, T, H, d, generator=g).to(dtype).to(gpu)
    good = torch.randperm(n_pages, generator=g)[:n_log].to(torch.int32)
    ref, _ = _make_pool(gpu, d, key_bits, vb, H, n_pages, dtype)
    ref.data.fill_(0xA5)                           # (padding bytes of a page are never written)
    ref.append(k, v, good[None].to(gpu))
    _progress(f"append with bad table entries d={d} {dtype} T={T}")
    bad_slots = sorted({0, n_log // 2, n_log - 1})
    for poison in (n_pages, 2 ** 31 - 1, -1, -2 ** 31):
        table = good.clone()
        table[bad_slots] = poison
        pool, _ = _make_pool(gpu, d, key_bits, vb, H, n_pages, dtype)
        pool.data.fill_(0xA5)
        refp = ref.data.clone()
        pool.append(k, v, table[None].to(gpu))
        torch.cuda.synchronize()
        touched = torch.zeros(n_pages, dtype=torch.bool)
        ok_slots = [i for i in range(n_log) if i not in bad_slots]
        touched[good[ok_slots].long()] = True
        assert torch.all(pool.data[~touched] == 0xA5), poison                       # nothing else was written
        # full pages written through good entries equal the reference pool's (the last page may be partial)
        full = [i for i in ok_slots if (i + 1) * 16 <= T]
        assert torch.equal(pool.data[good[full].long()], refp[good[full].long()]), poison
    # a run that starts near the end of the table row and continues past it: the overflow is dropped
    pool, _ = _make_pool(gpu, d, key_bits, vb, H, n_pages, dtype)
    pool.data.fill_(0x5A)
    short = good[:2].clone()
    start = torch.tensor([20], dtype=torch.int32, device=gpu)
    pool.append(k, v, short[None].to(gpu), start)                                   # positions 20 .. 20 + T - 1, row of 2
    torch.cuda.synchronize()
    touched = torch.zeros(n_pages, dtype=torch.bool)
    touched[short.long()] = True
    assert torch.all(pool.data[~touched] == 0x5A)
    # without start positions the host knows the run and refuses it
    if T > 32:
        with pytest.raises((ValueError, RuntimeError)):
            pool.append(k, v, short[None].to(gpu))


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,dtype", [(128, 3, 4, 8, 2, torch.bfloat16), (256, 3, 2, 16, 2, torch.bfloat16),
                                                         (64, 3, 2, 4, 1, torch.bfloat16), (128, 3, 2, 4, 2, torch.float32),
                                                         (576, 4, 4, 8, 1, torch.bfloat16), (512, 3, 2, 4, 2, torch.float16)])
def test_decode_gives_no_weight_to_pages_outside_the_pool(gpu, d, key_bits, vb, Hq, Hkv, dtype):
    """Decode with table entries outside [0, num_pages): those pages' tokens get no weight, so the result is
    the attention over the remaining tokens - checked against the oracle on exactly those tokens
    (score.py:84-173) - and sequence lengths beyond the table row are cut to the row."""
    N, B = 390, 2
    n_log = (N + 15) // 16
    n_pages = B * n_log + 2
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, n_pages, dtype, seed=42)
    g = torch.Generator().manual_seed(31 * d + vb)
    k = torch.randn(B, N, Hkv, d, generator=g).to(dtype)
    v = torch.randn(B, N, Hkv, d, generator=g).to(dtype)
    q = torch.randn(B, Hq, d, generator=g).to(dtype)
    table = torch.randperm(n_pages, generator=g)[: B * n_log].to(torch.int32).view(B, n_log)
    pool.append(k.to(gpu), v.to(gpu), table.to(gpu))
    prm = params_of(tq)
    _progress(f"decode with bad table entries d={d} kb={key_bits} vb={vb} {dtype}")
    # sequence 0 loses its whole first 64-token block, a page in the middle and its last (partial) page;
    # sequence 1 loses one page
    lost = {0: [0, 1, 2, 3, 9, n_log - 1], 1: [5]}
    bad = table.clone()
    for b, slots in lost.items():
        bad[b, slots] = torch.tensor([n_pages, -1, 2 ** 31 - 1, -7, n_pages + 5, 2 ** 30][: len(slots)], dtype=torch.int32)
    seq = torch.tensor([N, N], dtype=torch.int32, device=gpu)
    for n_split in (1, 3, None):
        out = pool.decode_attention(q.to(gpu), bad.to(gpu), seq, n_split=n_split, max_len=N).cpu()
        torch.cuda.synchronize()
        for b in range(B):
            keep = [i for i in range(n_log) if i not in lost[b]]
            tok = torch.cat([torch.arange(16 * i, min(16 * i + 16, N)) for i in keep])
            idx, sgn, norms, rn, vd, vs, vz = [t.cpu()[:, tok] for t in pool.export_flat(table[b], N)]
            want = O.hybrid_attention(q[b:b + 1], key_code(idx, sgn, rn, norms, key_bits - 1), value_code(vd, vs, vz, vb),
                                      len(tok), prm, Hkv, None, None)
            c = cosine(out[b:b + 1], want)
            assert c >= COS_GATE, (n_split, b, c)
    # a sequence length beyond the table row is cut to the row: same result as the full row
    over = pool.decode_attention(q.to(gpu), table.to(gpu), torch.tensor([N + 4000, 10 ** 9], dtype=torch.int32, device=gpu),
                                 n_split=2, max_len=N)
    row_full = pool.decode_attention(q.to(gpu), table.to(gpu), torch.tensor([n_log * 16] * 2, dtype=torch.int32, device=gpu),
                                     n_split=2, max_len=N)
    torch.cuda.synchronize()
    assert torch.equal(over, row_full)
    # every table entry bad: nothing to attend to, zeros
    allbad = torch.full_like(table, -1)
    z = pool.decode_attention(q.to(gpu), allbad.to(gpu), seq, n_split=2, max_len=N)
    torch.cuda.synchronize()
    assert torch.count_nonzero(z) == 0


# ------------------------------------------------------------------ query preparation for every query dtype
_OPTION_DEFAULTS = {"sequence_walkers": -1, "prep_words": -1}     # every other option: 1


def _set_option(name, value):
    from turboquant_amd import _ffi
    _ffi.check(_ffi.lib().tq_set_option(name.encode(), int(value)), "tq_set_option")


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,B,lens,n_split", [
    (256, 3, 2, 16, 2, 2, [5000, 777], 64),
    (256, 3, 2, 16, 2, 2, [5000, 777], 5),
    (128, 3, 4, 32, 8, 3, [900, 64, 300], 4),      # 4 of 8 operand heads exist
    (128, 4, 4, 8, 2, 2, [700, 1], 9),             # 4-bit keys (an extra term plane), odd split count
    (256, 2, 4, 10, 2, 1, [2000], 33),             # 5 heads per group
    (128, 3, 2, 32, 2, 2, [400, 900], 16),         # 16 heads per KV head = two groups of 8
    (128, 3, 2, 3, 1, 1, [130], 1)])               # a single workgroup does everything
def test_decode_step_for_every_query_dtype(gpu, d, key_bits, vb, Hq, Hkv, B, lens, n_split):
    """The query operands of the matrix-core page kernel (triton_kernels.py:527-528: q Pi^T, q S^T, here also
    their fp6 operand form) are prepared by one launch per step for bf16, fp16 and fp32 queries; each must meet
    the oracle (score.py:138-173) on the same store, whatever the split count."""
    g = torch.Generator().manual_seed(d + Hq + n_split)
    pages = (max(lens) + 15) // 16
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, B * pages + 1, torch.bfloat16, seed=42)
    table = torch.randperm(B * pages + 1, generator=g)[: B * pages].to(torch.int32).view(B, pages).to(gpu)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).bfloat16().to(gpu)
    pool.append(k, v, table)
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    _progress(f"query dtypes d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} lens={lens} splits={n_split}")
    prm = params_of(tq)
    stores = [_store_from_oracle_view(pool, table[b], lens[b]) for b in range(B)]
    for qdt in (torch.bfloat16, torch.float16, torch.float32):
        q = torch.randn(B, Hq, d, generator=g).to(qdt)
        out = pool.decode_attention(q.to(gpu), table, seq, n_split=n_split).cpu()
        for b in range(B):
            kc, vc = stores[b]
            want = O.hybrid_attention(q[b:b + 1], kc, vc, max(lens[b], O.MIN_HISTORY), prm, Hkv, None, None)
            assert cosine(out[b:b + 1], want) >= COS_GATE, (qdt, b)


# ------------------------------------------------------------------ 8-bit values in the paged store
@pytest.mark.parametrize("d,key_bits,dtype,gs", [(128, 3, torch.bfloat16, 32), (256, 3, torch.float16, 32),
                                                 (64, 4, torch.float32, 32), (128, 3, torch.bfloat16, 64)])
def test_eight_bit_values_in_pages(gpu, golden, d, key_bits, dtype, gs):
    """quantize_values(bits=8) (kv_cache.py:89-98: one code per byte) through the paged store: the exported flat
    tensors equal the flat quantiser's (which is bit-exact against the reference's *_b8_* vectors), and decode
    attention over those pages matches the oracle on the same store."""
    from turboquant_amd.kv_cache import quantize_values
    H, T = 2, 75
    pool, tq = _make_pool(gpu, d, key_bits, 8, H, 16, dtype, gs=gs)
    g = torch.Generator().manual_seed(8 * d + key_bits)
    k = torch.randn(1, T, H, d, generator=g).to(dtype).to(gpu)
    v = torch.randn(1, T, H, d, generator=g).to(dtype).to(gpu)
    table = torch.randperm(16, generator=g).to(torch.int32).to(gpu)[None, :]
    for a, b in ((0, 20), (20, 21), (21, 75)):             # ragged appends: codes of earlier slots must survive
        pool.append(k[:, a:b], v[:, a:b], table, torch.tensor([a], dtype=torch.int32, device=gpu))
    idx, sgn, norms, rnorms, vdata, vsc, vz = pool.export_flat(table[0], T)
    ref = tq.quantize(k[0].transpose(0, 1))
    refv = quantize_values(v[0].transpose(0, 1), bits=8, group_size=gs)
    torch.cuda.synchronize()
    assert vdata.shape == (H, T, d) and torch.equal(vdata, refv.data)
    assert torch.equal(vsc, refv.scales) and torch.equal(vz, refv.zeros)
    assert torch.equal(idx, ref.mse_indices) and torch.equal(sgn, ref.qjl_signs)
    # the oracle's value quantiser gives the same bytes (kv_cache.py:45-98)
    want = O.quantize_values(v[0].transpose(0, 1).cpu(), 8, gs)
    assert torch.equal(vdata.cpu(), want.data) and torch.equal(vsc.cpu(), want.scales)
    # decode over 8-bit pages
    _progress(f"decode over 8-bit values d={d} {dtype}")
    Hq = 4 * H
    q = torch.randn(1, Hq, d, generator=g).to(dtype)
    out = pool.decode_attention(q.to(gpu), table, torch.tensor([T], dtype=torch.int32, device=gpu), max_len=T).cpu()
    kc, vc = _store_from_oracle_view(pool, table[0], T)
    if gs == 32:            # (the reference's read path de-quantises values with group size 32, score.py:94,127)
        ref_out = O.hybrid_attention(q, kc, vc, T, params_of(tq), H, None, None)
        assert cosine(out, ref_out) >= COS_GATE


def test_compressed_store_with_eight_bit_values(gpu):
    """CompressedKVStore(value_bits=8) (store.py:34-48 passes value_bits straight to quantize_values): chunks
    in, flat cache out, and the hybrid attention on it."""
    from turboquant_amd.score import compute_hybrid_attention
    from turboquant_amd.store import CompressedKVStore
    g = torch.Generator().manual_seed(88)
    H, d, T = 2, 128, 100
    store = CompressedKVStore(d, H, key_bits=3, value_bits=8, device=gpu, layer_idx=1)
    k = torch.randn(T, H, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(T, H, d, generator=g).bfloat16().to(gpu)
    store.append_chunk(k[:40], v[:40])
    store.append_chunk(k[40:], v[40:])
    flat = store.get_flat_cache()
    assert flat.value_q.bits == 8 and flat.value_q.data.shape == (H, T, d)
    want = O.quantize_values(v.transpose(0, 1).cpu(), 8, 32)
    assert torch.equal(flat.value_q.data.cpu(), want.data)
    q = torch.randn(1, 4 * H, d, generator=g).bfloat16().to(gpu)
    out = compute_hybrid_attention(q, store, None, None, num_query_heads=4 * H).cpu()
    kc = key_code(flat.prod_q.mse_indices.cpu(), flat.prod_q.qjl_signs.cpu(), flat.prod_q.residual_norms.cpu(),
                  flat.prod_q.norms.cpu(), 2)
    vc = value_code(flat.value_q.data.cpu(), flat.value_q.scales.cpu(), flat.value_q.zeros.cpu(), 8)
    ref = O.hybrid_attention(q.cpu(), kc, vc, T, params_of(store.quantizer), H, None, None)
    assert cosine(out, ref) >= COS_GATE
    assert store.memory_bytes() > 0


# ------------------------------------------------------------------ head_dim 64 on the matrix-core page kernel
@pytest.mark.parametrize("key_bits,vb,Hq,Hkv,dtype", [(3, 4, 8, 2, torch.bfloat16), (3, 2, 32, 4, torch.bfloat16),
                                                       (2, 2, 6, 2, torch.float16), (4, 4, 16, 2, torch.bfloat16),
                                                       (3, 4, 1, 1, torch.float16), (4, 2, 12, 1, torch.bfloat16)])
def test_decode_head_dim_64_on_the_matrix_cores(gpu, key_bits, vb, Hq, Hkv, dtype):
    """head_dim 64 (the reference ships codebook_d64_b1..4.json) runs the matrix-core page kernel: the score
    contraction still takes 128 coordinates per instruction, half of them zeros.  Ragged lengths, block and
    page boundaries, exact tails, several split counts, against the oracle on the same store."""
    _progress(f"decode d=64 kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} {dtype}")
    worst = _decode_case(gpu, 64, key_bits, vb, 4, Hq, Hkv, [513, 64, 1, 200], [0, 7, 33, 0], seed=640 + Hq, dtype=dtype)
    for n_split in (1, 3, 8):
        worst = min(worst, _decode_case(gpu, 64, key_bits, vb, 2, Hq, Hkv, [1000, 17], None, seed=650 + n_split,
                                        n_split=n_split, dtype=dtype))
    _progress(f"   worst cosine {worst:.7f}")


def _variant_against_default(gpu, option, d, key_bits, vb, Hq, Hkv, dtype, exact, rel=1e-3):
    """Decode with run-time option `option` on and off over ragged lengths (ends inside every page of a block
    and on block boundaries), table entries outside the pool and several split counts; `exact`: the two must
    agree bit for bit, else to `rel` of the largest output.  The option-on result is also checked against the
    oracle (score.py:84-173)."""
    B = 4
    lens = [1000, 17, 16 * 37 + 1, 16 * 6]
    n_log = max((n + 15) // 16 for n in lens)
    n_pages = B * n_log + 1
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, n_pages, dtype, seed=77)
    g = torch.Generator().manual_seed(640 + key_bits + d)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype)
    q = torch.randn(B, Hq, d, generator=g).to(dtype)
    table = torch.randperm(n_pages, generator=g)[: B * n_log].to(torch.int32).view(B, n_log)
    pool.append(k.to(gpu), v.to(gpu), table.to(gpu))
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    bad = table.clone()
    bad[0, [4, 7, 20, 21]] = torch.tensor([n_pages, -1, 2 ** 31 - 1, -9], dtype=torch.int32)
    prm = params_of(tq)
    _progress(f"{option} d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} {dtype}")
    try:
        # a bit-for-bit comparison needs the same partition of the tokens on both sides: the wide workgroups,
        # which only some variants have, halve the split count
        if exact:
            _set_option("wide_workgroups", 0)
        for tab in (table, bad):
            for n_split in (1, 2, 3, 8, 11):
                outs = []
                for on in (1, 0):
                    _set_option(option, on)
                    # every byte of the workspace poisoned first: the preparation only writes the operand rows its page
                    # kernel reads (those of heads 0..3 for the variants of at most four heads), and nothing may
                    # depend on what the other rows, or an earlier call, left behind
                    ws = pool.workspace(B, Hq, n_split)
                    ws.view(torch.uint8).fill_(0xFF)
                    outs.append(pool.decode_attention(q.to(gpu), tab.to(gpu), seq, n_split=n_split, max_len=max(lens),
                                                      workspace=ws).cpu())
                torch.cuda.synchronize()
                if exact:
                    assert torch.equal(outs[0], outs[1]), (n_split, tab is bad)
                else:
                    tol = rel * float(outs[1].float().abs().max()) + 1e-6
                    assert float((outs[0].float() - outs[1].float()).abs().max()) <= tol, (n_split, tab is bad)
        _set_option(option, 1)
        out = pool.decode_attention(q.to(gpu), table.to(gpu), seq, n_split=4, max_len=max(lens)).cpu()
        for b in range(B):
            idx, sgn, norms, rn, vd, vs, vz = [t.cpu() for t in pool.export_flat(table[b], lens[b])]
            want = O.hybrid_attention(q[b:b + 1], key_code(idx, sgn, rn, norms, key_bits - 1), value_code(vd, vs, vz, vb),
                                      lens[b], prm, Hkv, None, None)
            assert cosine(out[b:b + 1], want) >= COS_GATE, b
    finally:
        _set_option(option, _OPTION_DEFAULTS.get(option, 1))
        _set_option("wide_workgroups", 1)


@pytest.mark.parametrize("key_bits,vb,Hq,Hkv,dtype", [(3, 4, 8, 2, torch.bfloat16), (4, 2, 3, 1, torch.float16),
                                                       (2, 2, 2, 2, torch.bfloat16)])
def test_head_dim_64_two_pages_per_score_instruction(gpu, key_bits, vb, Hq, Hkv, dtype):
    """With at most four query heads per KV head the head_dim 64 kernel scores two pages per matrix instruction
    (block-diagonal query operand).  The sums are the same ones in the same order, so the output must equal,
    bit for bit, that of the one-page-per-instruction kernel (option "page_pairs" = 0, itself checked against
    the oracle above)."""
    _variant_against_default(gpu, "page_pairs", 64, key_bits, vb, Hq, Hkv, dtype, exact=True)


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,dtype", [(128, 3, 4, 8, 2, torch.bfloat16), (256, 3, 2, 4, 2, torch.bfloat16),
                                                         (128, 4, 2, 3, 1, torch.float16), (128, 2, 4, 1, 1, torch.bfloat16)])
def test_four_fp6_terms_in_one_operand(gpu, d, key_bits, vb, Hq, Hkv, dtype):
    """With at most four query heads per KV head (head_dim 128 / 256) the four fp6 terms of a head share one
    score operand (option "narrow_rows"): the same products, summed in a different order, so the result agrees
    with the two-operand kernel to rounding and with the oracle to the usual gate."""
    _variant_against_default(gpu, "narrow_rows", d, key_bits, vb, Hq, Hkv, dtype, exact=False)


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,dtype", [(128, 3, 4, 8, 2, torch.bfloat16), (64, 3, 2, 3, 1, torch.float16),
                                                         (128, 4, 2, 4, 2, torch.bfloat16), (64, 2, 4, 8, 2, torch.bfloat16),
                                                         (128, 3, 2, 16, 2, torch.bfloat16), (64, 4, 4, 7, 1, torch.float16)])
def test_eight_wavefronts_per_workgroup_on_half_the_splits(gpu, d, key_bits, vb, Hq, Hkv, dtype):
    """Short contexts at head_dim 64 / 128 run workgroups of eight wavefronts on half the
    split count they were given (option "wide_workgroups"; even split counts only): another partition of the same
    tokens, so the result agrees with the four-wavefront kernel to rounding and with the oracle to the usual
    gate - ragged ends, table entries outside the pool and the in-launch merge included.  (The two partitions
    round their softmax weights against different running maxima and their 16-bit outputs independently: an
    output may differ by one of its own units in the last place, 2^-8 relative.)"""
    _variant_against_default(gpu, "wide_workgroups", d, key_bits, vb, Hq, Hkv, dtype, exact=False, rel=2.0 ** -8)


@pytest.mark.parametrize("key_bits,vb,Hq,Hkv,n_split", [(3, 2, 16, 2, 64), (4, 4, 4, 2, 60), (2, 2, 8, 2, 62)])
def test_unequal_shares_for_the_two_workgroups_of_a_compute_unit(gpu, key_bits, vb, Hq, Hkv, n_split):
    """Head_dim 256 with a launch that fills the compute units twice (here 480 - 512 workgroups on 256 units): the
    workgroups of the first half of the grid take the even splits and a part of their odd neighbours' trips (option
    "split_skew", in sixteenths; 8 moves half of them, which with one or two trips per split leaves odd splits empty).
    Another partition of the same tokens: the result agrees with equal shares to rounding (one unit in the last place
    of a 16-bit output) and with the oracle (score.py:84-173) to the usual gate - ragged ends, a sequence shorter than
    the split count, and table entries outside the pool included."""
    d, B, dtype = 256, 4, torch.bfloat16
    lens = [64 * 130 + 5, 17, 64 * 64, 64 * 301 + 33]
    n_log = max((n + 15) // 16 for n in lens)
    n_pages = B * n_log + 1
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, n_pages, dtype, seed=78)
    g = torch.Generator().manual_seed(911 + key_bits)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype)
    q = torch.randn(B, Hq, d, generator=g).to(dtype)
    table = torch.randperm(n_pages, generator=g)[: B * n_log].to(torch.int32).view(B, n_log)
    pool.append(k.to(gpu), v.to(gpu), table.to(gpu))
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    bad = table.clone()
    bad[0, [4, 7, 200, 201]] = torch.tensor([n_pages, -1, 2 ** 31 - 1, -9], dtype=torch.int32)
    prm = params_of(tq)
    _progress(f"split_skew kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} n_split={n_split}")
    try:
        for tab in (table, bad):
            outs = {}
            for skew in (0, 1, 3, 8):
                _set_option("split_skew", skew)
                outs[skew] = pool.decode_attention(q.to(gpu), tab.to(gpu), seq, n_split=n_split, max_len=max(lens)).cpu()
            torch.cuda.synchronize()
            tol = 2.0 ** -8 * float(outs[0].float().abs().max()) + 1e-6
            for skew in (1, 3, 8):
                assert float((outs[skew].float() - outs[0].float()).abs().max()) <= tol, (skew, tab is bad)
            if tab is table:
                for skew in (1, 8):
                    for b in range(B):
                        idx, sgn, norms, rn, vd, vs, vz = [t.cpu() for t in pool.export_flat(table[b], lens[b])]
                        want = O.hybrid_attention(q[b:b + 1], key_code(idx, sgn, rn, norms, key_bits - 1),
                                                  value_code(vd, vs, vz, vb), lens[b], prm, Hkv, None, None)
                        assert cosine(outs[skew][b:b + 1], want) >= COS_GATE, (skew, b)
    finally:
        _set_option("split_skew", 1)


@pytest.mark.parametrize("d,vb,Hq,Hkv,dtype", [(128, 4, 16, 2, torch.bfloat16), (128, 2, 4, 1, torch.float16),
                                               (256, 2, 16, 2, torch.bfloat16), (256, 4, 6, 2, torch.bfloat16)])
def test_four_bit_keys_staged_through_lds(gpu, d, vb, Hq, Hkv, dtype):
    """4-bit keys (three index planes): the page data of the next block travels HBM -> LDS with LDS-direct
    loads and is copied to registers when its stage starts, instead of waiting in registers that the kernel
    does not have (the register-held variant spills and is not built).  Ragged lengths, a poisoned block table
    and 1 - 11 context splits against the oracle (score.py:84-173), with the splits merged inside the page kernel
    and by the merge kernel (to rounding of each other)."""
    _variant_against_default(gpu, "merge_in_kernel", d, 4, vb, Hq, Hkv, dtype, exact=False, rel=2.0 ** -8)


@pytest.mark.parametrize("option", ["merge_in_kernel", "narrow_rows", "wide_workgroups"])
@pytest.mark.parametrize("vb,Hq,Hkv,dtype", [(4, 16, 2, torch.bfloat16), (2, 3, 1, torch.float16), (4, 32, 2, torch.bfloat16),
                                             (2, 18, 2, torch.bfloat16)])
def test_five_bit_keys_with_the_query_operands_in_lds(gpu, option, vb, Hq, Hkv, dtype):
    """5-bit keys at head_dim 128 (four index planes + the sign plane, nine fp6 terms per query row): the query's
    matrix-core operands do not fit in registers beside the page data, so each workgroup copies its group's
    operands to LDS once and the score stage reads one term plane at a time for all pages of the block.  Groups of
    8, 3 (four-row operands), 16 (two groups of 8) and 9 (5 + 4) query heads per KV head; ragged lengths, a
    poisoned block table and 1 - 11 context splits against the oracle (score.py:84-173), with each of the merge,
    row-count and workgroup-width variants on and off."""
    _variant_against_default(gpu, option, 128, 5, vb, Hq, Hkv, dtype, exact=False, rel=2.0 ** -8)


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,dtype", [(128, 3, 4, 8, 2, torch.bfloat16), (128, 3, 4, 16, 2, torch.bfloat16),
                                                        (128, 4, 2, 3, 1, torch.float16), (64, 3, 4, 4, 1, torch.bfloat16),
                                                        (64, 3, 2, 16, 2, torch.float16), (128, 3, 4, 22, 2, torch.bfloat16),
                                                        (128, 3, 8, 5, 1, torch.bfloat16), (128, 2, 2, 7, 1, torch.bfloat16)])
def test_one_or_two_wavefronts_per_sequence(gpu, d, key_bits, vb, Hq, Hkv, dtype):
    """Many short sequences in one split: one or two wavefronts of a page-kernel workgroup walk a (sequence, group
    of heads) (run-time option "sequence_walkers": 1, 2, or 4 = all of them; by default chosen from the number of
    pairs) instead of all four.  Five sequences - so that the last workgroup has wavefronts without a pair - of
    ragged and zero length, a poisoned block table, head groups of unequal size (22 heads on 2 KV heads: 6 + 5), all
    three endings of the step (output written by the page kernel, partials for the merge kernel, an exact tail's
    partial merged in) against the four-wavefront form and the oracle (score.py:84-173)."""
    lens = [700, 0, 16 * 9 + 1, 64, 333]
    B = len(lens)
    g = torch.Generator().manual_seed(d + Hq + key_bits)
    pages = (max(lens) + 15) // 16
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, B * pages + 1, dtype, seed=43)
    table = torch.randperm(B * pages + 1, generator=g)[: B * pages].to(torch.int32).view(B, pages)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype).to(gpu)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype).to(gpu)
    pool.append(k, v, table.to(gpu))
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    q = torch.randn(B, Hq, d, generator=g).to(dtype)
    bad = table.clone()
    bad[0, [3, 8, 20]] = torch.tensor([B * pages + 1, -1, 2 ** 31 - 1], dtype=torch.int32)
    R = 24
    rk = torch.randn(B, R, Hkv, d, generator=g).to(dtype).to(gpu)
    rv = torch.randn(B, R, Hkv, d, generator=g).to(dtype).to(gpu)
    rl = torch.tensor([R, 3, 0, R, 11], dtype=torch.int32, device=gpu)
    _progress(f"one or two wavefronts per sequence d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} {dtype}")

    def runs():
        outs = []
        for tab in (table, bad):
            for merge_in_kernel in (1, 0):
                _set_option("merge_in_kernel", merge_in_kernel)
                ws = pool.workspace(B, Hq, 1)
                ws.view(torch.uint8).fill_(0xFF)
                outs.append(pool.decode_attention(q.to(gpu), tab.to(gpu), seq, n_split=1, workspace=ws).float().cpu())
            outs.append(pool.decode_attention(q.to(gpu), tab.to(gpu), seq, recent_k=rk, recent_v=rv, recent_len=rl,
                                              n_split=1).float().cpu())
        torch.cuda.synchronize()
        return outs

    try:
        _set_option("sequence_walkers", 4)
        want = runs()
        _set_option("sequence_walkers", 1)
        got = runs()
        _set_option("sequence_walkers", 2)
        got2 = runs()
    finally:
        _set_option("sequence_walkers", -1)
        _set_option("merge_in_kernel", 1)
    for i, (a, a2, b_) in enumerate(zip(got, got2, want)):
        assert torch.isfinite(a).all() and torch.isfinite(a2).all(), i
        assert (a - b_).abs().max() <= 2 ** -7 * b_.abs().max() + 1e-6, i        # one bf16 step of the largest value
        assert (a2 - b_).abs().max() <= 2 ** -7 * b_.abs().max() + 1e-6, i
    prm = params_of(tq)
    for b in range(B):
        if lens[b] == 0:
            assert torch.count_nonzero(got[0][b]) == 0
            continue
        kc, vc = _store_from_oracle_view(pool, table[b].to(gpu), lens[b])
        ref = O.hybrid_attention(q[b:b + 1], kc, vc, max(lens[b], O.MIN_HISTORY), prm, Hkv, None, None)
        assert cosine(got[0][b:b + 1], ref) >= COS_GATE, b


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv", [(128, 3, 4, 8, 2), (128, 4, 2, 3, 1), (256, 3, 2, 16, 2), (256, 2, 4, 5, 1),
                                                  (128, 3, 4, 22, 2), (128, 5, 4, 4, 1)])
def test_preparation_with_a_plane_word_per_wavefront(gpu, d, key_bits, vb, Hq, Hkv):
    """Large matrix-core preparations run a workgroup per tile of query rows whose wavefronts take a plane word each
    (run-time option "prep_words" 1), small ones a workgroup per (tile, word) (0): the same products in the same order,
    so the packed operands, and with them the step's output, are the same bits (score.py:84-173 through the oracle
    for the first form)."""
    _variant_against_default(gpu, "prep_words", d, key_bits, vb, Hq, Hkv, torch.bfloat16, exact=True)


@pytest.mark.parametrize("B,Hq,Hkv,d,key_bits,vb,dtype", [(201, 4, 1, 128, 3, 4, torch.bfloat16), (201, 2, 1, 128, 4, 2, torch.bfloat16),
                                                           (101, 3, 1, 256, 3, 2, torch.float16), (401, 1, 1, 64, 3, 4, torch.bfloat16),
                                                           (70, 12, 2, 128, 2, 4, torch.bfloat16)])
def test_preparation_with_several_groups_of_heads_per_workgroup(gpu, B, Hq, Hkv, d, key_bits, vb, dtype):
    """A launch of more (group of query heads, 32 coordinates) units than the card holds at once packs as many whole
    groups as fit eight rows into one preparation workgroup (two groups of 4 heads, four of 2, eight of 1; an odd
    number of groups leaves the last workgroup partly empty).  The operands of a group do not depend on its
    neighbours: the batch must equal, bit for bit, the same sequences decoded 32 at a time (one group per workgroup),
    compressed-only and with exact recent tokens, and a sequence of it the oracle (score.py:84-173)."""
    g = torch.Generator().manual_seed(B + 7 * Hq + d)
    lens = [int(x) for x in torch.randint(20, 90, (B,), generator=g)]
    lens[3] = 0
    ring = 24
    n_log = 6
    n_pages = B * n_log + 1
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, n_pages, dtype, seed=81)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).to(dtype)
    q = torch.randn(B, Hq, d, generator=g).to(dtype).to(gpu)
    table = torch.randperm(n_pages, generator=g)[: B * n_log].to(torch.int32).view(B, n_log).to(gpu)
    pool.append(k.to(gpu), v.to(gpu), table)
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    cache = torch.randn(2, n_pages, 16, Hkv, d, generator=g).to(dtype).to(gpu)
    _progress(f"packed preparation B={B} Hq={Hq} Hkv={Hkv} d={d} kb={key_bits} {dtype}")
    # (the vector-ALU preparation is what packs groups; bf16 queries would otherwise take the matrix-core preparation,
    # which has a test of its own and sums the rotation in another order)
    _set_option("prep_mfma", 0)
    try:
        whole = pool.decode_attention(q, table, seq, n_split=2, max_len=max(lens)).clone()
        whole_h = pool.decode_attention_ring(q, table, seq, cache[0], cache[1], ring, n_split=2, max_len=max(lens)).clone()
        for b0 in range(0, B, 32):
            sl = slice(b0, min(B, b0 + 32))
            part = pool.decode_attention(q[sl], table[sl], seq[sl], n_split=2, max_len=max(lens))
            part_h = pool.decode_attention_ring(q[sl], table[sl], seq[sl], cache[0], cache[1], ring, n_split=2, max_len=max(lens))
            torch.cuda.synchronize()
            assert torch.equal(whole[sl], part), b0
            assert torch.equal(whole_h[sl], part_h), b0
    finally:
        _set_option("prep_mfma", 1)
    assert torch.count_nonzero(whole[3]) == 0
    # the kernels that read the operand rows of all eight heads (the variants for few heads switched off) must find
    # zeros in the rows of the heads a group does not have, whichever workgroup shape wrote the operands: a
    # workspace filled with NaN bit patterns first
    try:
        _set_option("narrow_rows", 0)
        _set_option("page_pairs", 0)
        for on_matrix_cores in (0, 1):                       # both preparation kernels write those zeros
            _set_option("prep_mfma", on_matrix_cores)
            ws = pool.workspace(B, Hq, 2)
            ws.view(torch.int32).fill_(0x7fc00000)
            wide_rows = pool.decode_attention(q, table, seq, n_split=2, workspace=ws, max_len=max(lens)).clone()
            ws32 = pool.workspace(32, Hq, 2)
            for b0 in range(0, B, 32):
                sl = slice(b0, min(B, b0 + 32))
                ws32.view(torch.int32).fill_(0x7fc00000)
                part = pool.decode_attention(q[sl], table[sl], seq[sl], n_split=2, workspace=ws32, max_len=max(lens))
                torch.cuda.synchronize()
                assert torch.equal(wide_rows[sl], part), (on_matrix_cores, b0)
            assert not torch.isnan(wide_rows.float()).any()
    finally:
        _set_option("narrow_rows", 1)
        _set_option("page_pairs", 1)
        _set_option("prep_mfma", 1)
    for b in (0, B - 1):
        idx, sgn, norms, rn, vd, vs, vz = [t.cpu() for t in pool.export_flat(table[b], lens[b])]
        ref = O.hybrid_attention(q[b:b + 1].cpu(), key_code(idx, sgn, rn, norms, key_bits - 1), value_code(vd, vs, vz, vb),
                                 lens[b], params_of(tq), Hkv, None, None)
        assert cosine(whole[b:b + 1].cpu(), ref) >= COS_GATE, b


@pytest.mark.parametrize("rows,n_parts,d,dtype", [(64, 64, 256, torch.bfloat16), (64, 65, 256, torch.float16),
                                                  (3, 9, 256, torch.float32), (100, 33, 128, torch.bfloat16),
                                                  (7, 5, 128, torch.float32), (129, 17, 128, torch.float16),
                                                  (5, 40, 64, torch.bfloat16), (2, 19, 576, torch.float32),
                                                  (300, 3, 256, torch.bfloat16), (1, 1, 128, torch.float32),
                                                  (16, 20, 512, torch.float32), (8, 12, 192, torch.bfloat16),
                                                  (4, 70, 384, torch.float16), (33, 66, 768, torch.bfloat16)])
def test_merge_of_split_partials(gpu, rows, n_parts, d, dtype):
    """tq_decode_merge on its own: the log-sum-exp merge of per-split partials (m, l, acc[d]) - the segments of
    score.py:84-173 - against a float64 computation of the same formula, with empty parts (l = 0, which carry no
    weight whatever their m says), maxima of very different size, and row counts on both sides of what makes the
    kernel give a row to several workgroups (option "merge_row_groups": both settings are run and must agree)."""
    from turboquant_amd import _ffi
    g = torch.Generator().manual_seed(rows * 1000 + n_parts * 10 + d)
    parts = torch.empty(rows, n_parts, d + 2, dtype=torch.float32)
    parts[..., 0] = torch.randn(rows, n_parts, generator=g) * 20.0                       # m
    parts[..., 1] = torch.rand(rows, n_parts, generator=g) * 50.0 + 0.5                  # l
    parts[..., 2:] = torch.randn(rows, n_parts, d, generator=g) * parts[..., 1:2]        # acc
    empty = torch.rand(rows, n_parts, generator=g) < 0.2
    empty[0, :] = n_parts > 1                                                            # a row without any token
    empty[0, 0] = False
    if rows > 1:
        empty[1, :] = True                                                               # ... and one that is all empty
    parts[..., 1][empty] = 0.0
    parts[..., 2:][empty] = 0.0
    parts[..., 0][empty] = 1e30                                                          # must not count
    p64 = parts.double()
    live = p64[..., 1] > 0
    m = torch.where(live, p64[..., 0], torch.full_like(p64[..., 0], -1e300))
    M = m.max(dim=1, keepdim=True).values
    w = torch.where(live, torch.exp(m - M), torch.zeros_like(m))
    den = (w * p64[..., 1]).sum(dim=1, keepdim=True)
    want = torch.where(den > 0, (w[..., None] * p64[..., 2:]).sum(dim=1) / den.clamp_min(1e-300), torch.zeros(rows, d, dtype=torch.float64))
    dt = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    dev_parts = parts.to(gpu)
    outs = []
    _progress(f"merge rows={rows} n_parts={n_parts} d={d} {dtype}")
    try:
        for on in (1, 0):
            _set_option("merge_row_groups", on)
            out = torch.full((rows, d), float("nan"), dtype=dtype, device=gpu)
            _ffi.check(_ffi.lib().tq_decode_merge(dev_parts.data_ptr(), rows, n_parts, d, dt, out.data_ptr(),
                                                  torch.cuda.current_stream().cuda_stream), "tq_decode_merge")
            torch.cuda.synchronize()
            outs.append(out.cpu())
    finally:
        _set_option("merge_row_groups", 1)
    eps = {torch.float32: 2.0 ** -20, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    for out in outs:
        err = (out.double() - want).abs()
        assert bool((err <= eps * want.abs() + 1e-5).all()), float(err.max())
    assert float((outs[0].double() - outs[1].double()).abs().max()) <= 2 * eps * float(want.abs().max())


@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv,lens,n_split", [
    (128, 3, 4, 32, 8, [900, 1, 16, 0, 517], 4),
    (128, 3, 2, 8, 1, [2100], 8),
    (256, 3, 2, 16, 2, [1500, 700], 5),
    (256, 4, 4, 10, 2, [333, 64], 2),              # 5 heads per group
    (64, 3, 4, 8, 2, [800, 130, 65], 3),
    (128, 3, 4, 32, 2, [640], 1)])                 # 16 heads per KV head = two groups of 8, a single split
def test_splits_merged_inside_the_page_kernel(gpu, d, key_bits, vb, Hq, Hkv, lens, n_split):
    """With at most eight context splits the workgroup that finishes last among the splits of a (sequence, group
    of query heads) merges them inside the page kernel's launch (the log-sum-exp merge of score.py:84-173's
    segments), instead of a merge kernel: same result up to the order of the sums, for ragged and empty
    sequences, on consecutive calls (the arrival counters are reset by each step's preparation), and against the
    oracle."""
    B = len(lens)
    g = torch.Generator().manual_seed(d + Hq + n_split)
    pages = (max(lens) + 15) // 16
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, B * pages + 1, torch.bfloat16, seed=42)
    table = torch.randperm(B * pages + 1, generator=g)[: B * pages].to(torch.int32).view(B, pages).to(gpu)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).bfloat16().to(gpu)
    pool.append(k, v, table)
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    q = torch.randn(B, Hq, d, generator=g).bfloat16()
    _progress(f"in-launch merge d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv} lens={lens} splits={n_split}")
    try:
        _set_option("merge_in_kernel", 0)
        want = pool.decode_attention(q.to(gpu), table, seq, n_split=n_split).float().cpu()
        _set_option("merge_in_kernel", 1)
        got = pool.decode_attention(q.to(gpu), table, seq, n_split=n_split).float().cpu()
        again = pool.decode_attention(q.to(gpu), table, seq, n_split=n_split).float().cpu()
        torch.cuda.synchronize()
    finally:
        _set_option("merge_in_kernel", 1)
    assert torch.equal(got, again)
    assert (got - want).abs().max() <= 2 ** -7 * want.abs().max() + 1e-6        # one bf16 step of the largest value
    # the same with an exact tail (its partial is one more part of the in-launch merge)
    R = 40
    rk = torch.randn(B, R, Hkv, d, generator=g).bfloat16().to(gpu)
    rv = torch.randn(B, R, Hkv, d, generator=g).bfloat16().to(gpu)
    rl = torch.tensor([R if i % 2 == 0 else 7 for i in range(B)], dtype=torch.int32, device=gpu)
    try:
        _set_option("merge_in_kernel", 0)
        want_h = pool.decode_attention(q.to(gpu), table, seq, recent_k=rk, recent_v=rv, recent_len=rl, n_split=n_split).float().cpu()
        _set_option("merge_in_kernel", 1)
        got_h = pool.decode_attention(q.to(gpu), table, seq, recent_k=rk, recent_v=rv, recent_len=rl, n_split=n_split).float().cpu()
        torch.cuda.synchronize()
    finally:
        _set_option("merge_in_kernel", 1)
    assert (got_h - want_h).abs().max() <= 2 ** -7 * want_h.abs().max() + 1e-6
    prm = params_of(tq)
    for b in range(B):
        if lens[b] == 0:
            assert torch.count_nonzero(got[b]) == 0
            continue
        kc, vc = _store_from_oracle_view(pool, table[b], lens[b])
        ref = O.hybrid_attention(q[b:b + 1], kc, vc, max(lens[b], O.MIN_HISTORY), prm, Hkv, None, None)
        assert cosine(got[b:b + 1], ref) >= COS_GATE, b


def test_in_launch_merge_over_thousands_of_consecutive_steps(gpu):
    """The hand-off of the in-launch merge (every workgroup's partial, then the arrival counter, then the last
    arriver's reads) over 3,000 consecutive decode steps of the 16 x 8192, 32 q / 8 KV head shape on ONE
    workspace.  The queries rotate among four, so a partial that the merging workgroup read before its producer's
    stores had landed would be the previous step's, a different query's.  The in-launch merge sums in a fixed
    order, so every step must reproduce its query's first result bit for bit; that first result is held to the
    merge kernel's (merge_in_kernel 0) at one bf16 step.  Stops at the first mismatch (checked every 50 steps)."""
    d, Hq, Hkv, B, N = 128, 32, 8, 16, 8192
    g = torch.Generator().manual_seed(77)
    pages = N // 16
    pool, tq = _make_pool(gpu, d, 3, 4, Hkv, B * pages, torch.bfloat16, seed=42)
    table = torch.randperm(B * pages, generator=g).to(torch.int32).view(B, pages).to(gpu)
    for b0 in range(0, B, 4):
        k = torch.randn(4, N, Hkv, d, generator=g).bfloat16().to(gpu)
        v = torch.randn(4, N, Hkv, d, generator=g).bfloat16().to(gpu)
        pool.append(k, v, table[b0:b0 + 4])
    seq = torch.full((B,), N, dtype=torch.int32, device=gpu)
    qs = [torch.randn(B, Hq, d, generator=g).bfloat16().to(gpu) for _ in range(4)]
    n_split = pool.default_splits(B, N, Hq)
    ws = pool.workspace(B, Hq, n_split)
    _progress(f"in-launch merge soak: {B} x {N}, {Hq} q / {Hkv} KV heads, {n_split} splits, 3000 steps")
    try:
        _set_option("merge_in_kernel", 0)
        sep = [pool.decode_attention(q, table, seq, n_split=n_split, workspace=ws).clone() for q in qs]
        _set_option("merge_in_kernel", 1)
        first = [pool.decode_attention(q, table, seq, n_split=n_split, workspace=ws).clone() for q in qs]
        torch.cuda.synchronize()
        for a, b_ in zip(first, sep):
            assert (a.float() - b_.float()).abs().max() <= 2 ** -7 * b_.float().abs().max() + 1e-6
        assert not torch.equal(first[0], first[1])
        out = torch.empty_like(qs[0])
        bad = torch.zeros((), dtype=torch.int64, device=gpu)
        steps = torch.arange(1, 3001, device=gpu)
        for step in range(3000):
            i = step % 4
            pool.decode_attention(qs[i], table, seq, n_split=n_split, workspace=ws, out=out)
            # step number of the first mismatch (0 = none so far), kept on the card
            differs = (out != first[i]).any()
            bad = torch.where((bad == 0) & differs, steps[step], bad)
            if step % 50 == 49:
                at = int(bad.item())
                assert at == 0, f"in-launch merge differs from its first result at step {at - 1}"
    finally:
        _set_option("merge_in_kernel", 1)


@pytest.mark.parametrize("d,Hq,Hkv,vb,key_bits", [(128, 32, 8, 2, 3), (128, 32, 8, 4, 3), (128, 16, 2, 4, 4), (256, 16, 2, 2, 3)])
def test_decode_over_a_store_with_outlier_channels(gpu, d, Hq, Hkv, vb, key_bits):
    """Decode over a store built from the prefill workload's kind of data: bf16 N(0,1) keys and values with four
    channels per (tensor, head) scaled by 20 (CPU generator seed 1, picked by randperm as in that workload), so
    that a value group's scale and zero point are dominated by its outlier channel and the weight x scale and
    weight x zero operands of the value stage carry large numbers.  Queries of three kinds per sequence - diffuse
    (small norm: near-uniform weights over 4096 tokens), ordinary N(0,1), and peaked (aligned with one stored
    key, so that a single token takes nearly all the weight) - against the oracle's de-quantise-everything
    attention on the same store (score.py:138-173): cosine >= 0.9999 over a sequence's output, as everywhere.
    Per query head the gate is 0.9995: the kernel rounds weight x scale and weight to bf16 (relative 2^-9 per
    token), and in a group with an outlier channel sum(w zero) and sum(w scale code) are sixty times the value
    they add up to, so a head whose mean value happens to be small shows 1 - cos of 1e-4 (measured worst head
    1.4e-4 with 2-bit values and diffuse weights; the sequence's output is at 3e-5).  The margins are printed."""
    g = torch.Generator().manual_seed(1)
    B, N = 3, 4096
    pages = N // 16
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, B * pages + 2, torch.bfloat16, seed=42)
    table = torch.randperm(B * pages + 2, generator=g)[: B * pages].to(torch.int32).view(B, pages).to(gpu)
    k = torch.randn(B, N, Hkv, d, generator=g)
    v = torch.randn(B, N, Hkv, d, generator=g)
    for t in (k, v):
        for h in range(Hkv):
            t[:, :, h, torch.randperm(d, generator=g)[:4]] *= 20.0
    k, v = k.bfloat16(), v.bfloat16()
    pool.append(k.to(gpu), v.to(gpu), table)
    G = Hq // Hkv
    q = torch.randn(B, Hq, d, generator=g)
    q[0] *= 0.02                                                       # diffuse
    for hq in range(Hq):                                               # peaked: along key 1000 + hq of the head's KV head
        kk = k[2, 1000 + hq, hq // G].float()
        q[2, hq] = 6.0 * kk / kk.norm() * (d ** 0.5) / 8.0
    q = q.bfloat16()
    seq = torch.full((B,), N, dtype=torch.int32, device=gpu)
    _progress(f"outlier store d={d} Hq={Hq} Hkv={Hkv} vb={vb} kb={key_bits}")
    out = pool.decode_attention(q.to(gpu), table, seq).cpu()
    prm = params_of(tq)
    for b, kind in enumerate(("diffuse", "ordinary", "peaked")):
        kc, vc = _store_from_oracle_view(pool, table[b], N)
        want = O.hybrid_attention(q[b:b + 1], kc, vc, N, prm, Hkv, None, None)
        per_head = [cosine(out[b, hq:hq + 1], want[0, hq:hq + 1]) for hq in range(Hq)]
        c = cosine(out[b:b + 1], want)
        _progress(f"   {kind}: cosine {c:.8f} (1 - cos = {1 - c:.2e}), worst head {min(per_head):.8f}")
        assert c >= COS_GATE, (kind, c)
        assert min(per_head) >= 0.9995, (kind, min(per_head))


@pytest.mark.parametrize("B,Hq,Hkv,d,key_bits,vb", [(5, 8, 2, 128, 3, 4), (3, 21, 3, 128, 3, 2), (7, 10, 2, 128, 4, 4),
                                                      (2, 6, 1, 256, 3, 2), (9, 12, 4, 128, 2, 4), (33, 16, 2, 256, 3, 2),
                                                      (4, 1, 1, 128, 3, 4), (3, 16, 1, 128, 3, 8)])
def test_query_preparation_on_the_matrix_cores(gpu, B, Hq, Hkv, d, key_bits, vb):
    """bf16 queries are rotated (q Pi^T), sketched (q S^T; triton_kernels.py:527-528) and packed into the page
    kernel's fp6 operands by a matrix-core kernel: three-term bf16 products that are fp32-accurate but summed in
    another order than the vector-ALU preparation.  On the same store the two preparations must agree to the
    rounding of the bf16 output (group sizes 1 to 8, a last row tile that is partly empty, 16 heads per KV head as
    two groups), both with the page kernels that read all eight operand rows of a group on a workspace poisoned
    with NaN patterns, and each must meet the oracle (score.py:138-173)."""
    g = torch.Generator().manual_seed(B + 7 * Hq + d)
    lens = [int(x) for x in torch.randint(40, 400, (B,), generator=g)]
    pages = (max(lens) + 15) // 16
    pool, tq = _make_pool(gpu, d, key_bits, vb, Hkv, B * pages + 1, torch.bfloat16, seed=42)
    table = torch.randperm(B * pages + 1, generator=g)[: B * pages].to(torch.int32).view(B, pages).to(gpu)
    k = torch.randn(B, max(lens), Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, max(lens), Hkv, d, generator=g).bfloat16().to(gpu)
    pool.append(k, v, table)
    seq = torch.tensor(lens, dtype=torch.int32, device=gpu)
    q = torch.randn(B, Hq, d, generator=g).bfloat16()
    _progress(f"matrix-core preparation B={B} Hq={Hq} Hkv={Hkv} d={d} kb={key_bits} vb={vb}")
    outs = {}
    try:
        for narrow in (1, 0):
            _set_option("narrow_rows", narrow)
            _set_option("page_pairs", narrow)
            for mode in (2, 0):
                _set_option("prep_mfma", mode)
                ws = pool.workspace(B, Hq, 3)
                ws.view(torch.int32).fill_(0x7fc00000)
                outs[(narrow, mode)] = pool.decode_attention(q.to(gpu), table, seq, n_split=3, workspace=ws).float().cpu()
        torch.cuda.synchronize()
    finally:
        _set_option("prep_mfma", 1)
        _set_option("narrow_rows", 1)
        _set_option("page_pairs", 1)
    for narrow in (1, 0):
        a, b = outs[(narrow, 2)], outs[(narrow, 0)]
        assert not torch.isnan(a).any() and not torch.isnan(b).any()
        assert (a - b).abs().max() <= 2 ** -7 * b.abs().max() + 1e-6, narrow
    assert torch.equal(outs[(1, 2)], outs[(0, 2)]) or (outs[(1, 2)] - outs[(0, 2)]).abs().max() <= 2 ** -7 * outs[(0, 2)].abs().max()
    prm = params_of(tq)
    for b in (0, B - 1):
        kc, vc = _store_from_oracle_view(pool, table[b], lens[b])
        want = O.hybrid_attention(q[b:b + 1], kc, vc, lens[b], prm, Hkv, None, None)
        assert cosine(outs[(1, 2)][b:b + 1], want) >= COS_GATE, b
        assert cosine(outs[(1, 0)][b:b + 1], want) >= COS_GATE, b
