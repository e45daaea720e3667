"""GPU: the decode entry point that allocates nothing (tq_decode_attn_paged_noalloc) against the workspace
form it is a variant of (tq_decode_attn_paged), through the C ABI.  The two run the same kernels with the
same split count, so the outputs must be identical bit for bit - on two calls in a row, the second with a
smaller input, since every call on a GPU reuses the same static scratch area and finds the last call's
contents in it."""

import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _pool(gpu, d, key_bits, vb, Hkv, n_pages, dtype=torch.bfloat16):
    from turboquant_amd.paged import PagedKVPool
    from turboquant_amd.quantizer import TurboQuantProd
    tq = TurboQuantProd(d, bits=key_bits, device=gpu, seed=42)
    return PagedKVPool(tq, Hkv, n_pages, value_bits=vb, dtype=dtype, device=gpu), tq


def _both(gpu, pool, tq, q, table, seq, n_split, rk=None, rv=None, rl=None):
    """(workspace form, static-scratch form) straight through ctypes."""
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    B, Hq, d = q.shape
    ws = torch.empty(lib.tq_decode_workspace_bytes(B, Hq, d, n_split) // 4, dtype=torch.float32, device=gpu)
    want, got = torch.empty_like(q), torch.full_like(q, float("nan"))
    ly = tq._layer()
    rows = 0 if rk is None else rk.shape[1]
    rs = (0, 0, 0) if rk is None else rk.stride()[:3]
    common = (q.data_ptr(), _ffi.dtype_tag(q.dtype), B, Hq, pool.num_kv_heads, pool.data.data_ptr(), pool.num_pages,
              table.data_ptr(), table.shape[1], seq.data_ptr(), 1.0 / d ** 0.5, C.byref(ly), C.byref(pool.layout),
              _ffi.ptr(rk), _ffi.ptr(rv), rows, rs[0], rs[1], rs[2], _ffi.ptr(rl))
    st = _ffi.stream_ptr(gpu)
    with torch.cuda.device(gpu):
        _ffi.check(lib.tq_decode_attn_paged(*common, want.data_ptr(), ws.data_ptr(), n_split, st), "workspace form")
        _ffi.check(lib.tq_decode_attn_paged_noalloc(*common, got.data_ptr(), n_split, st), "static form")
    torch.cuda.synchronize()
    return want, got


# (8-bit values and 5-bit keys at head_dim 128 run the matrix-core kernel too; the last case, 5-bit keys at head_dim 64,
# has no matrix-core kernel: the general page kernel runs on the static area)
@pytest.mark.parametrize("d,key_bits,vb,Hq,Hkv", [(128, 3, 4, 8, 2), (256, 3, 2, 16, 2), (64, 3, 2, 4, 1), (128, 3, 8, 8, 2),
                                                   (128, 5, 4, 8, 2), (64, 5, 2, 10, 2), (576, 4, 4, 8, 1)])
def test_static_scratch_decode_equals_the_workspace_form_on_consecutive_calls(gpu, d, key_bits, vb, Hq, Hkv):
    g = torch.Generator().manual_seed(d + Hq)
    B, N = 3, 900
    pages = (N + 15) // 16
    pool, tq = _pool(gpu, d, key_bits, vb, Hkv, B * pages + 1)
    table = torch.randperm(B * pages + 1, generator=g)[: B * pages].to(torch.int32).view(B, pages).to(gpu)
    k = torch.randn(B, N, Hkv, d, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, N, Hkv, d, generator=g).bfloat16().to(gpu)
    pool.append(k, v, table)
    q = torch.randn(B, Hq, d, generator=g).bfloat16().to(gpu)
    rk = torch.randn(B, 9, Hkv, d, generator=g).bfloat16().to(gpu)
    rv = torch.randn(B, 9, Hkv, d, generator=g).bfloat16().to(gpu)
    rl = torch.tensor([9, 0, 4], dtype=torch.int32, device=gpu)
    print(f"[no-alloc] d={d} kb={key_bits} vb={vb} Hq={Hq} Hkv={Hkv}: first call, B=3, 5 splits, exact tail", flush=True)
    seq = torch.tensor([N, 37, 512], dtype=torch.int32, device=gpu)
    want, got = _both(gpu, pool, tq, q, table, seq, 5, rk, rv, rl)
    assert torch.equal(got, want) and not torch.isnan(got.float()).any()
    print("[no-alloc] second call: one sequence, 2 splits, no tail", flush=True)
    seq1 = torch.tensor([300], dtype=torch.int32, device=gpu)
    want, got = _both(gpu, pool, tq, q[1:2].contiguous(), table[2:3].contiguous(), seq1, 2)
    assert torch.equal(got, want) and not torch.isnan(got.float()).any()
    # and through the host mirror
    out = pool.decode_attention(q, table, seq, n_split=5, recent_k=rk, recent_v=rv, recent_len=rl, static_scratch=True)
    ref = pool.decode_attention(q, table, seq, n_split=5, recent_k=rk, recent_v=rv, recent_len=rl)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)


def test_static_scratch_decode_rejects_what_does_not_fit(gpu):
    """A call whose partials exceed the static area (16 MiB) is refused with TQ_ETOOBIG before anything is
    launched; bad arguments are refused as in the workspace form."""
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    d, Hq, Hkv, B = 128, 32, 8, 64
    pool, tq = _pool(gpu, d, 3, 4, Hkv, 8)
    q = torch.zeros(B, Hq, d, dtype=torch.bfloat16, device=gpu)
    table = torch.zeros(B, 4, dtype=torch.int32, device=gpu)
    seq = torch.full((B,), 50, dtype=torch.int32, device=gpu)
    out = torch.full_like(q, 7.0)
    ly = tq._layer()
    args = lambda n_split: (q.data_ptr(), _ffi.TQ_BF16, B, Hq, Hkv, pool.data.data_ptr(), pool.num_pages, table.data_ptr(), 4,
                            seq.data_ptr(), 0.1, C.byref(ly), C.byref(pool.layout), None, None, 0, 0, 0, 0, None,
                            out.data_ptr(), n_split, _ffi.stream_ptr(gpu))
    need = 4 * B * Hq * 33 * (d + 2)
    assert need > 16 << 20
    # the exported size rule is what the entry point applies: refused exactly when it exceeds the area
    assert lib.tq_noalloc_init() == 0
    assert lib.tq_decode_noalloc_bytes(B, Hq, Hkv, 32, C.byref(ly)) > 16 << 20 >= lib.tq_decode_noalloc_bytes(B, Hq, Hkv, 1, C.byref(ly))
    assert lib.tq_decode_noalloc_bytes(B, Hq, Hkv, 32, C.byref(ly)) >= need
    assert lib.tq_decode_noalloc_bytes(B, Hq, Hkv, 0, C.byref(ly)) == 0
    assert lib.tq_decode_attn_paged_noalloc(*args(32)) == -4
    torch.cuda.synchronize()
    assert torch.all(out == 7.0)                                   # nothing ran
    with pytest.raises(ValueError, match="TQ_ETOOBIG"):
        pool.decode_attention(q, table, seq, n_split=32, static_scratch=True)
    assert lib.tq_decode_attn_paged_noalloc(*args(0)) == -1
    assert lib.tq_decode_attn_paged_noalloc(*args(1)) == 0         # the same call with one split fits
    torch.cuda.synchronize()
