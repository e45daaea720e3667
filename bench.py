"""Headline benchmark: compressed-KV decode attention GB/s (and % of HBM peak)
plus quantize tokens/s, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-backend-step]

A step is one pass of the fused decode-attention path (query rotation, page
streaming kernel, merge) over the long-context configuration: 4 sequences x
131 072 context tokens, 16 query heads over 2 KV heads, head_dim 256, 3-bit keys
(2-bit Lloyd-Max + 1-bit QJL), 2-bit values in groups of 32, 16-token pages.
The compressed pools are resident in HBM before timing starts; steps rotate
over several pools so that no step finds its pages in the 256 MB Infinity
Cache.  `value` = algorithmic KV bytes per step / step time, with the
reference's own byte accounting (norms, residual norms, scales and zeros at
2 bytes): 196 B per (token, KV head).

The same JSON line carries
  roofline     : the page-streaming kernel alone (hipEvents around that stage),
                 algorithmic bytes / its mean duration, against 8 TB/s;
  quantize     : tokens/s of the fused paged quantise call on the prefill
                 configuration (32 768 tokens x 8 KV heads, head_dim 128), with the
                 paged key kernel's own time against the bf16 matrix peak and
                 the whole append against the HBM peak;
  decode_gqa   : the 16 x 8192-token GQA decode configuration (and the same with
                 4-bit keys, the reference's default for the first four layers);
  round_trip   : the 4096-key x 32-query round trip (quantise + all scores);
  backend_decode_step : a full decode step of a random-init 32-layer dense
                 transformer (batch 32 x 32 768 context) whose attention layers run
                 through the batch-aware backend hooks on compressed KV;
  cpu_baseline : the CPU oracle's de-quantise-everything attention (the
                 reference's production read path) timed on the host cores on
                 one of the four sequences; every sequence's GPU output is checked
                 against it (cosine).
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def student_t(shape, nu, gen):
    """z / sqrt(chi2_nu / nu) element-wise on the CPU generator, chi2 as the sum of nu squared normals."""
    import torch
    z = torch.randn(*shape, generator=gen)
    chi = torch.zeros(shape)
    for _ in range(nu):
        chi.add_(torch.randn(*shape, generator=gen).square_())
    return z.div_(chi.div_(nu).sqrt_())


def algorithmic_bytes_per_token_head(d, mse_bits, value_bits, group):
    eff = 1 if mse_bits == 1 else (2 if mse_bits == 2 else 4)
    return d * eff // 8 + d // 8 + 2 + 2 + d * value_bits // 8 + 2 * 2 * (d // group)


class DecodeWorkload:
    """B sequences of N compressed tokens in `n_pools` separate pools."""

    def __init__(self, name, B, N, Hq, Hkv, d, key_bits, value_bits, n_pools, seed, dist, device, device_data=False):
        import torch
        from turboquant_amd.paged import PagedKVPool
        from turboquant_amd.quantizer import TurboQuantProd
        self.name, self.B, self.N, self.Hq, self.Hkv, self.d = name, B, N, Hq, Hkv, d
        self.key_bits, self.value_bits = key_bits, value_bits
        gen = torch.Generator().manual_seed(seed)            # a CPU generator: the same data on every machine
        # (device_data: the bulk of the keys and values from the card's generator instead - timing-only tables)
        dgen = torch.Generator(device=device).manual_seed(seed) if device_data else None
        self.tq = TurboQuantProd(d, bits=key_bits, device=device)
        pages_per_seq = (N + 15) // 16
        n_pages = B * pages_per_seq
        self.pools = []
        perm = torch.randperm(n_pages, generator=gen).to(torch.int32).to(device)
        self.table = perm.reshape(B, pages_per_seq).contiguous()
        first = PagedKVPool(self.tq, Hkv, n_pages, value_bits=value_bits, value_group_size=32,
                            dtype=torch.bfloat16, device=device)
        chunk = 32768
        for b in range(B):                      # sequence by sequence, in chunks, to bound the bf16 staging memory
            for t0 in range(0, N, chunk):
                t1 = min(N, t0 + chunk)
                shape = (1, t1 - t0, Hkv, d)
                if dist == "student_t5":
                    k, v = student_t(shape, 5, gen), student_t(shape, 5, gen)
                elif dgen is not None:
                    k = torch.randn(*shape, generator=dgen, device=device)
                    v = torch.randn(*shape, generator=dgen, device=device)
                else:
                    k = torch.randn(*shape, generator=gen)
                    v = torch.randn(*shape, generator=gen)
                first.append(k.bfloat16().to(device), v.bfloat16().to(device), self.table[b:b + 1],
                             torch.tensor([t0], dtype=torch.int32, device=device))
        self.pools.append(first)
        for _ in range(n_pools - 1):
            p = PagedKVPool(self.tq, Hkv, n_pages, value_bits=value_bits, value_group_size=32,
                            dtype=torch.bfloat16, device=device)
            p.data.copy_(first.data)
            self.pools.append(p)
        self.q = torch.randn(B, Hq, d, generator=gen).bfloat16().to(device)
        self.seq = torch.full((B,), N, dtype=torch.int32, device=device)
        self.n_split = first.default_splits(B, N, Hq)
        self.ws = first.workspace(B, Hq, self.n_split)
        self.out = torch.empty_like(self.q)
        self.bytes = B * Hkv * N * algorithmic_bytes_per_token_head(d, key_bits - 1, value_bits, 32)
        self.stored_bytes = B * Hkv * pages_per_seq * first.page_bytes

    def step(self, i, stages=7):
        pool = self.pools[i % len(self.pools)]
        pool.decode_attention(self.q, self.table, self.seq, n_split=self.n_split, workspace=self.ws, out=self.out,
                              max_len=self.N, stages=stages)


def hybrid_step_bench(work, steps, warmup, ring=128):
    """The same decode step in hybrid mode: the newest `ring` tokens of every sequence attended to exactly,
    read in place from a paged exact cache (synthetic bf16 rows) through the block table, the tokens before
    them from the compressed pages."""
    import torch
    dev = work.q.device
    n_blocks = work.pools[0].num_pages
    gen = torch.Generator(device=dev).manual_seed(11)
    cache = torch.randn(2, n_blocks, 16, work.Hkv, work.d, generator=gen, device=dev, dtype=torch.float32).bfloat16()

    def step(i):
        pool = work.pools[i % len(work.pools)]
        pool.decode_attention_ring(work.q, work.table, work.seq, cache[0], cache[1], ring, n_split=work.n_split,
                                   workspace=work.ws, out=work.out, max_len=work.N)
    ms, _ = time_steps(step, steps, warmup)
    del cache
    per_tok = algorithmic_bytes_per_token_head(work.d, work.key_bits - 1, work.value_bits, 32)
    nbytes = work.B * work.Hkv * ((work.N - ring) * per_tok + ring * 2 * work.d * 2)     # pages + exact bf16 K and V rows
    return {"exact_tokens": ring, "ms_per_step": ms, "bytes_per_step": nbytes, "GBps": nbytes / (ms * 1e-3) / 1e9,
            "pct_hbm_peak": 100.0 * nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}


def launches_per_step(work):
    """Kernel launches of one compressed-only decode step on the matrix-core path, by the library's rule: the query
    preparation (which also carries the page-prefetch workgroups), the page kernel, and a merge kernel when the
    step has more than 8 context splits (with at most 8 the page kernel's last-arriving workgroups merge; the
    head_dim 64 / 128 kernels run half the splits they are given when workgroups of 8 wavefronts apply)."""
    wide = work.d in (64, 128) and work.n_split % 2 == 0 and (work.N + 63) // 64 <= 16 * 4 * work.n_split
    eff = work.n_split // 2 if wide else work.n_split
    return 2 if eff <= 8 else 3


RAMP_SECONDS = 0.25      # --ramp-seconds


def clock_ramp(fn, n_indices):
    """Untimed: keeps the card busy with the leg's own step for RAMP_SECONDS, so that the W warm-up and K timed
    steps that follow run at the steady clocks of a serving loop whatever W is (a card that has idled needs
    ~0.2 s of sustained work to get there)."""
    import torch
    t0, i = time.perf_counter(), 0
    while RAMP_SECONDS > 0 and time.perf_counter() - t0 < RAMP_SECONDS:
        for _ in range(50):
            fn(i % max(n_indices, 1))
            i += 1
        torch.cuda.synchronize()


def time_steps(fn, steps, warmup, ramp=True):
    """(mean ms per step, wall ms per step) with HIP events on the launch stream."""
    import torch
    if ramp:
        clock_ramp(fn, warmup + steps)
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(warmup + i)
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall


def time_kernel_stage(work, steps, warmup):
    """Mean execution time of the page-streaming kernel alone, inside whole steps: every timed step
    runs all three stages as usual, and the library attaches a HIP event pair to the dispatch of the
    page kernel itself (tq_time_next_page_kernel), so that the elapsed time is the kernel's own
    begin-to-end time - the quantity a profiler's kernel trace reports - without the dispatch gaps
    that markers between launches would add."""
    import torch
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    evs = []
    for _ in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(); b.record()                      # creates the underlying events
        evs.append((a, b))
    torch.cuda.synchronize()
    clock_ramp(work.step, warmup + steps)
    for i in range(warmup):                         # the timed steps follow the warm-up without a pause
        work.step(i)
    for i, (a, b) in enumerate(evs):
        lib.tq_time_next_page_kernel(a.cuda_event, b.cuda_event)
        work.step(warmup + i)
    lib.tq_time_next_page_kernel(None, None)        # (nothing is left armed once the events go away)
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in evs) / steps


def stream_read_peak(work, steps, warmup):
    """Read bandwidth the card delivers to a kernel that only reads (GB/s): tq_stream_read over the same
    rotating pools the decode workload streams, best of a few launch shapes, timed with events on the
    stream of the launches."""
    import torch
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    st = torch.cuda.current_stream().cuda_stream
    best = None
    for wg_per_cu, flight in ((4, 4), (8, 4), (8, 1), (16, 1), (4, 8)):
        def one(i):
            pool = work.pools[i % len(work.pools)].data
            nbytes = pool.numel() * pool.element_size() // 16 * 16
            rc = lib.tq_stream_read(pool.data_ptr(), nbytes, wg_per_cu, flight, None, st)
            if rc:
                raise RuntimeError(f"tq_stream_read failed: {rc}")
            return nbytes
        nbytes = one(0)
        ms, _ = time_steps(one, steps, warmup)
        gbs = nbytes / (ms * 1e-3) / 1e9
        if best is None or gbs > best["GBps"]:
            best = {"GBps": gbs, "workgroups_per_cu": wg_per_cu, "loads_in_flight": flight, "bytes": nbytes,
                    "us_per_launch": ms * 1e3}
    return best


def cpu_decode_baseline(work, n_seq=None, runs=3):
    """The oracle's de-quantise-all + dense attention (the reference's production read path, score.py:84-173)
    on the host cores: every sequence of the workload once (so that the GPU result of every sequence is
    checked), the first one `runs` times for the timing."""
    import torch
    from oracle import tq_oracle as O
    from tests.helpers import key_code, value_code, params_of
    pool = work.pools[0]
    prm = params_of(work.tq)
    n_seq = work.B if n_seq is None else n_seq
    work.step(0)
    torch.cuda.synchronize()
    gpu_out = work.out.float().cpu()
    times, cosines = [], []
    for b in range(n_seq):
        idx, sgn, norms, rn, vd, vs, vz = [t.cpu() for t in pool.export_flat(work.table[b], work.N)]
        kc = key_code(idx, sgn, rn, norms, work.key_bits - 1)
        vc = value_code(vd, vs, vz, work.value_bits)
        q = work.q[b:b + 1].cpu()
        for _ in range(runs if b == 0 else 1):
            t0 = time.perf_counter()
            out = O.hybrid_attention(q, kc, vc, work.N, prm, work.Hkv, None, None)
            if b == 0:
                times.append(time.perf_counter() - t0)
        got, want = gpu_out[b].flatten(), out.float().flatten()
        cosines.append(float((got @ want) / (got.norm() * want.norm())))
    sec = sorted(times)[len(times) // 2]
    sample_bytes = work.bytes // work.B
    return {"value": sample_bytes / sec / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "seconds": sec,
            "sample": f"1 of {work.B} sequences ({work.N} tokens x {work.Hkv} KV heads), median of {runs} runs, "
                      f"full-job time = x{work.B}",
            "gpu_vs_oracle_cosine": min(cosines), "gpu_vs_oracle_cosine_per_sequence": cosines,
            "sequences_checked": n_seq}


def time_key_kernel(step, steps, warmup):
    """Mean execution time of the paged matrix-core key-quantise kernel alone, inside whole appends (the
    library attaches a HIP event pair to that kernel's own dispatch, tq_time_next_key_kernel)."""
    import torch
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    evs = []
    for _ in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(); b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    clock_ramp(step, warmup + steps)
    for i in range(warmup):
        step(i)
    for i, (a, b) in enumerate(evs):
        lib.tq_time_next_key_kernel(a.cuda_event, b.cuda_event)
        step(warmup + i)
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in evs) / steps


def quantize_bench(device, steps, warmup):
    import torch
    from turboquant_amd.paged import PagedKVPool
    from turboquant_amd.quantizer import TurboQuantProd
    T, H, d = 32768, 8, 128
    # the prefill workload's own recipe, on the CPU generator (the same data on every machine): K, V = randn(1, 8,
    # 32768, 128) in that order, then per (tensor, head) four channels picked by randperm(128)[:4] scaled by 20, bf16
    gen = torch.Generator().manual_seed(1)
    k = torch.randn(1, H, T, d, generator=gen)
    v = torch.randn(1, H, T, d, generator=gen)
    for t in (k, v):
        for h in range(H):
            t[0, h, :, torch.randperm(d, generator=gen)[:4]] *= 20.0
    k = k.bfloat16().transpose(1, 2).contiguous().to(device)          # (1, T, H, d), the layout an engine hands over
    v = v.bfloat16().transpose(1, 2).contiguous().to(device)
    tq = TurboQuantProd(d, bits=3, device=device)
    pool = PagedKVPool(tq, H, T // 16, value_bits=2, value_group_size=32, dtype=torch.bfloat16, device=device)
    table = torch.arange(T // 16, dtype=torch.int32, device=device)[None]
    ms, _ = time_steps(lambda i: pool.append(k, v, table), steps, warmup)
    # The three d x d contractions of the key quantiser are the matrix-core part of the path.  The kernel issues
    # y = u Pi^T as 3 and p = r S^T as 6 exact bf16 term products (one fp32-accurate product each), and the centroid
    # contraction x_hat = c[idx] Pi as 2 bit planes x 5 fp6 digits on the block-scaled fp6 x fp4 MFMA.  The roofline
    # that bounds it is the matrix pipe: `frac` = the time the issued work takes at the peaks of its instruction
    # types (bf16 2500 TFLOP/s, fp6 / fp4 10100 TFLOP/s) over the measured time; `achieved` / `peak` are the issued
    # FLOP rate and the blend of the two peaks that this mix could reach.  In the product the key kernel runs beside
    # the value kernel (a second stream); an event pair around it inside such an append also covers time it spends
    # waiting for its share of the machine.  So: `frac` is taken over the WHOLE append (both kernels, fork and
    # join), and the kernel's own duration is measured with the value kernel switched off (tq_set_option
    # "append_parts" = 1, events attached to the kernel's dispatch).
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    _ffi.check(lib.tq_set_option(b"append_parts", 1), "tq_set_option")
    try:
        key_ms = time_key_kernel(lambda i: pool.append(k, v, table), steps, warmup)
    finally:
        _ffi.check(lib.tq_set_option(b"append_parts", 3), "tq_set_option")
    flops = 3 * 2 * d * d * T * H
    bf16_flop = (3 + 6) * 2 * d * d * T * H                     # term products of the first and the third contraction
    fp6_flop = 2 * 5 * 2 * d * d * T * H                        # planes x digits of the centroid contraction
    at_peak_s = bf16_flop / 2500e12 + fp6_flop / 10100e12
    issued = (bf16_flop + fp6_flop) / (ms * 1e-3) / 1e12
    blend_peak = (bf16_flop + fp6_flop) / at_peak_s / 1e12
    nbytes = T * (2 * H * d * 2 + H * 100)
    return {"tokens_per_s": T / (ms * 1e-3), "ms": ms, "tokens": T, "kv_heads": H, "head_dim": d,
            "workload": "prefill quantize, 32768 tok x 8 KV heads, d=128, 3b keys + 2b values, pages of 16",
            "hbm_gbs": nbytes / (ms * 1e-3) / 1e9, "hbm_bytes": nbytes,
            "hbm_frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "roofline": {"bound": "mfma", "kernel": "key_mfma_kernel (paged sink) beside value_chunk_kernel",
                         "append_ms": ms, "achieved": issued, "peak": blend_peak, "unit": "TFLOP/s",
                         "frac": at_peak_s / (ms * 1e-3), "algorithmic_tflops": flops / (ms * 1e-3) / 1e12,
                         "frac_issued": at_peak_s / (ms * 1e-3),
                         "frac_algorithmic_of_bf16_peak": flops / (ms * 1e-3) / 2500e12,
                         "frac_hbm": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                         "issued_bf16_gflop": bf16_flop / 1e9, "issued_fp6_fp4_gflop": fp6_flop / 1e9,
                         "key_kernel_alone_ms": key_ms, "key_kernel_alone_frac": at_peak_s / (key_ms * 1e-3),
                         "note": "three views of the same append: frac_issued = frac (below), frac_algorithmic_of_bf16_peak = "
                                 "the 6 d^2 FLOP per vector the reference formulates over the bf16 matrix peak, frac_hbm = "
                                 "bytes in and out over the HBM peak.  frac: "
                                 "issued matrix work of the key kernel (9 bf16 term products + 10 fp6 x fp4 plane/digit "
                                 "products per vector and d x d contraction size) over the whole append time, against "
                                 "the peaks of the two instruction types; key_kernel_alone_* = the same work over the "
                                 "kernel's own duration when the value kernel does not run beside it"}}, (pool, k, v, table, tq)


def round_trip_bench(device, steps, warmup, with_cpu):
    """The CPU-runnable round trip (4096 keys x 128, 32 queries, 3-bit keys, seed 0): quantise the keys and
    estimate all 32 x 4096 inner products, on the GPU and (oracle) on the host cores."""
    import torch
    from turboquant_amd.quantizer import TurboQuantProd
    g = torch.Generator().manual_seed(0)
    K = torch.randn(4096, 128, generator=g)
    K = K / K.norm(dim=-1, keepdim=True) * (0.5 + 1.5 * torch.rand(4096, generator=g)).unsqueeze(-1)
    Q = torch.randn(32, 128, generator=g)
    Q = Q / Q.norm(dim=-1, keepdim=True) * (0.5 + 1.5 * torch.rand(32, generator=g)).unsqueeze(-1)
    tq = TurboQuantProd(128, bits=3, device=device)
    Kd, Qd = K.to(device), Q.to(device)

    def step(i):
        code = tq.quantize(Kd)
        return tq.attention_score(Qd, code)
    ms, _ = time_steps(step, steps, warmup)
    out = {"workload": "4096 keys x 128 fp32, 32 queries, 3-bit keys: quantise + all 32 x 4096 estimates",
           "ms": ms, "keys_per_s": 4096 / (ms * 1e-3)}
    if with_cpu:
        from oracle import tq_oracle as O
        from tests.helpers import params_of
        prm = params_of(tq)
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            code = O.prod_quantize(K, prm)
            ref = O.attention_score(Q, code, prm)
            times.append(time.perf_counter() - t0)
        sec = sorted(times)[2]
        out["cpu_baseline"] = {"seconds": sec, "keys_per_s": 4096 / sec, "cores": torch.get_num_threads(), "kind": "port",
                               "sample": "the whole workload, median of 5 runs"}
        # end to end the GPU quantiser may flip a coordinate that sits on a threshold (fp32 summation order);
        # the score gate itself is taken on identical bytes in the tests
        gcode = tq.quantize(Kd)
        got = tq.attention_score(Qd, gcode)
        torch.cuda.synchronize()
        out["index_bytes_differing"] = int((gcode.mse_indices.cpu() != code.mse_indices).sum())
        out["sign_bytes_differing"] = int((gcode.qjl_signs.cpu() != code.qjl_signs).sum())
        rms = float(ref.pow(2).mean().sqrt())
        same = (gcode.mse_indices.cpu() == code.mse_indices).all(dim=-1) & (gcode.qjl_signs.cpu() == code.qjl_signs).all(dim=-1)
        diff = (got.float().cpu() - ref).abs()
        out["scores_max_abs_over_rms_on_keys_with_identical_bytes"] = float(diff[:, same].max()) / rms
    return out


def backend_step_bench(device, steps, warmup, n_layers=32, batch=32, context=32768):
    """Full decode step through the attention-backend hooks: a random-init bf16 dense transformer (hidden 4096,
    32 q / 8 KV heads of 128, SwiGLU 14336, vocabulary 128256) with compressed KV (3b keys, 4b values) in every
    layer and no exact KV cache.  The prior tokens' K/V are drawn N(0,1) straight into the pools (running the
    25-PFLOP prefill that would produce them is not part of the step being timed)."""
    import torch
    from turboquant_amd.integration import batched, vllm as hooks
    from turboquant_amd.integration.harness import MinimalRunner
    hidden, hq, hkv, d, ffn, vocab = 4096, 32, 8, 128, 14336, 128256
    slack = 64 + 4 * (warmup + steps)
    runner = MinimalRunner(n_layers, hidden, hq, hkv, d, ffn, vocab, batch, context + slack, device,
                           exact_cache=False, seed=4)
    states = batched.install_batched_hooks(runner, num_blocks=runner.num_blocks, key_bits=3, value_bits=4,
                                           initial_layers_count=0, mode=hooks.MODE_FULL_TQ, no_alloc=True)
    gen = torch.Generator(device=device).manual_seed(4)
    chunk = 8192
    zero = torch.zeros(batch, dtype=torch.int32)
    for st in states.values():
        for c0 in range(0, context, chunk):
            k = torch.randn(batch, chunk, hkv, d, generator=gen, device=device, dtype=torch.bfloat16)
            v = torch.randn(batch, chunk, hkv, d, generator=gen, device=device, dtype=torch.bfloat16)
            st.pool.append(k, v, runner.block_table, start_pos=zero + c0)
    del k, v
    runner.seq_lens = [context] * batch
    toks = torch.randint(0, vocab, (warmup + steps, batch), generator=gen, device=device)
    ms, _ = time_steps(lambda i: runner.decode_step(toks[i]), steps, warmup, ramp=False)
    # the same step captured once as a HIP graph and replayed (what a serving loop does)
    replay, _ = runner.capture_decode_step(context + slack, toks[0])
    graph_ms, _ = time_steps(lambda i: replay(toks[i]), steps, warmup, ramp=False)
    # the compressed-KV part of a step alone: every layer's page write and fused decode attention
    meta = runner.decode_metadata()
    q1 = torch.randn(batch, hq, d, generator=gen, device=device, dtype=torch.bfloat16)
    k1 = torch.randn(batch, hkv, d, generator=gen, device=device, dtype=torch.bfloat16)

    def kv_part(i):
        for st in states.values():
            st.write(k1, k1, meta)
            st.attend(q1, meta)
    kv_ms, _ = time_steps(kv_part, steps, warmup)
    attn_bytes = n_layers * batch * context * hkv * algorithmic_bytes_per_token_head(d, 2, 4, 32)
    weight_bytes = 2 * (n_layers * (hidden * (hq + 2 * hkv) * d + hq * d * hidden + 3 * hidden * ffn) + hidden * vocab)
    out = {"workload": f"full decode step through the attention-backend hooks: {n_layers} layers, hidden {hidden}, "
                       f"{hq} q / {hkv} KV heads of {d}, SwiGLU {ffn}, batch {batch} x {context} context, "
                       "compressed KV (3b keys, 4b values) in every layer, no exact KV cache; prior K/V synthetic",
           "tokens_per_s": batch / (graph_ms * 1e-3), "ms_per_step": graph_ms, "steps": steps,
           "eager_ms_per_step": ms, "eager_tokens_per_s": batch / (ms * 1e-3),
           "compressed_kv_bytes_read_per_step": attn_bytes, "weight_bytes_read_per_step": weight_bytes,
           "hbm_gbs": (attn_bytes + weight_bytes) / (graph_ms * 1e-3) / 1e9,
           "compressed_kv_ms_per_step": kv_ms, "compressed_kv_gbs": attn_bytes / (kv_ms * 1e-3) / 1e9,
           "compressed_kv_gib": sum(s.memory_bytes() for s in states.values()) / 2 ** 30}
    hooks.set_mode(hooks.MODE_CAPTURE_ONLY)
    del runner, states
    torch.cuda.empty_cache()
    return out


def cpu_quantize_baseline(k, v, tq, sample_tokens=32768):
    import torch
    from oracle import tq_oracle as O
    from tests.helpers import params_of
    prm = params_of(tq)
    kk = k[0, :sample_tokens].transpose(0, 1).contiguous().cpu()      # (H, T, d)
    vv = v[0, :sample_tokens].transpose(0, 1).contiguous().cpu()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        O.prod_quantize(kk, prm)
        O.quantize_values(vv, 2, 32)
        times.append(time.perf_counter() - t0)
    sec = sorted(times)[1]
    return {"tokens_per_s": sample_tokens / sec, "cores": torch.get_num_threads(), "kind": "port", "seconds": sec,
            "sample": f"{sample_tokens} of 32768 tokens x 8 KV heads, median of 3 runs"}


# (sequences, context, query heads, KV heads, head_dim, key bits, value bits): every family of decode kernels -
# head_dim 64 / 128 / 256 on the matrix cores with 2- / 3- / 4-bit keys and 2- / 4- / 8-bit values, 1 to 16 query
# heads per KV head (11 as 6 + 5), 5-bit keys at head_dim 128, short and long contexts - and the head sizes of latent
# attention (512, 576) on the kernel that works on a block per workgroup
SHAPE_TABLE = [
    (4, 131072, 16, 2, 256, 3, 2), (4, 131072, 16, 2, 256, 2, 2), (4, 131072, 16, 2, 256, 4, 2),
    (4, 131072, 16, 2, 256, 3, 4), (4, 131072, 8, 2, 256, 3, 2), (4, 131072, 2, 2, 256, 3, 2),
    (8, 65536, 16, 2, 256, 3, 2), (4, 65536, 32, 4, 256, 3, 2), (32, 8192, 16, 2, 256, 3, 2), (1, 524288, 16, 2, 256, 3, 2),
    (16, 8192, 32, 8, 128, 3, 4), (16, 8192, 32, 8, 128, 2, 4), (16, 8192, 32, 8, 128, 4, 4), (16, 8192, 32, 8, 128, 3, 2),
    (16, 8192, 64, 8, 128, 3, 4), (16, 8192, 8, 8, 128, 3, 4), (16, 8192, 128, 8, 128, 3, 4),
    (32, 32768, 32, 8, 128, 3, 4), (8, 131072, 32, 8, 128, 3, 4), (64, 2048, 32, 8, 128, 3, 4), (256, 1024, 32, 8, 128, 3, 4),
    (1, 131072, 32, 8, 128, 3, 4),
    (16, 8192, 32, 8, 64, 3, 4), (16, 8192, 32, 8, 64, 2, 2), (16, 8192, 32, 8, 64, 4, 4), (16, 8192, 64, 8, 64, 3, 4),
    (32, 32768, 32, 8, 64, 3, 4),
    (16, 8192, 8, 1, 576, 4, 4), (32, 8192, 8, 1, 576, 4, 4), (4, 32768, 16, 1, 576, 4, 4), (16, 8192, 8, 1, 512, 3, 4),
    (16, 8192, 32, 8, 128, 5, 4), (16, 8192, 64, 8, 128, 5, 4), (16, 8192, 32, 8, 128, 3, 8),
    (16, 8192, 88, 8, 128, 3, 4),
    (16, 8192, 128, 1, 576, 4, 4), (16, 8192, 64, 1, 128, 3, 4),      # 128 heads on one latent; multi-query attention
]


def shape_table(device, steps, warmup, table=None):
    """Whole-step and page-kernel times of SHAPE_TABLE's decode shapes (timing only; N(0,1) data from the card's
    generator), compressed-only and with the newest 128 tokens exact."""
    import torch
    rows = []
    for (B, N, Hq, Hkv, d, kb, vb) in (table or SHAPE_TABLE):
        w = DecodeWorkload("shape", B, N, Hq, Hkv, d, kb, vb, n_pools=2 if B * N * Hkv >= 1 << 22 else 4, seed=5,
                           dist="normal", device=device, device_data=True)
        ms, _ = time_steps(w.step, steps, warmup)
        kern = time_kernel_stage(w, steps, warmup)
        hyb = hybrid_step_bench(w, steps, warmup)
        rows.append({"sequences": B, "context": N, "q_heads": Hq, "kv_heads": Hkv, "head_dim": d, "key_bits": kb,
                     "value_bits": vb, "n_split": w.n_split, "bytes_per_step": w.bytes,
                     "page_kernel": ("general (vector ALU)", "matrix cores, a block per wavefront",
                                     "matrix cores, a block per workgroup")[w.pools[0].page_kernel()],
                     "step_us": round(ms * 1e3, 2), "step_pct_hbm_peak": round(100.0 * w.bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 1),
                     "page_kernel_us": round(kern * 1e3, 2),
                     "page_kernel_pct_hbm_peak": round(100.0 * w.bytes / (kern * 1e-3) / 1e9 / HBM_PEAK_GBS, 1),
                     "hybrid_step_us": round(hyb["ms_per_step"] * 1e3, 2)})
        print(json.dumps(rows[-1]), file=sys.stderr, flush=True)
        del w
        torch.cuda.empty_cache()
    return rows


def phase_stamps(device, reps=40):
    """Mean time (microseconds after the first wavefront's start) at which the wavefronts of the page kernel reach
    its phase boundaries, with and without the page prefetch of the preparation launch.  Needs a library built
    with -DTQ_STAMPS: lane 0 of every wavefront then stores the 100 MHz real-time counter at each boundary."""
    import ctypes
    import numpy as np
    import torch
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    if not hasattr(lib, "tq_debug_stamps"):
        raise SystemExit("this libtq_hip.so has no stamps: build it with TQ_EXTRA_HIPCC_FLAGS=-DTQ_STAMPS")
    names = ["start", "operands loaded", "first block requested, table scanned", "loop done", "epilogue barrier",
             "walkers in LDS", "partial stores issued", "partial stores acknowledged"]
    order = [0, 1, 2, 3, 6, 7, 4, 5]
    out = []
    for label, shape, fn_name, n_wg, nw in (("4 x 131072, head_dim 256", (4, 131072, 16, 2, 256, 3, 2), "tq_debug_stamps", 512, 4),
                                            ("16 x 8192, head_dim 128", (16, 8192, 32, 8, 128, 3, 4), "tq_debug_stamps_d128", 256, 8)):
        B, N, Hq, Hkv, d, kb, vb = shape
        w = DecodeWorkload(label, B, N, Hq, Hkv, d, kb, vb, n_pools=4, seed=3, dist="normal", device=device, device_data=True)
        fn = getattr(lib, fn_name)
        fn.argtypes = [ctypes.c_void_p, ctypes.c_int]
        for trips in (1, 0):
            _ffi.check(lib.tq_set_option(b"prefetch_trips", trips), "tq_set_option")
            for i in range(600):
                w.step(i)
            torch.cuda.synchronize()
            acc = []
            for r in range(reps):
                w.step(r)
                torch.cuda.synchronize()
                buf = (ctypes.c_ulonglong * (n_wg * 64))()
                if fn(buf, n_wg * 64) != 0:
                    raise SystemExit("reading the stamps failed")
                a = np.frombuffer(buf, dtype=np.uint64).reshape(n_wg, 8, 8).astype(np.int64)[:, :nw, :]
                acc.append((a - a[:, :, 0].min()) / 100.0)
            a = np.mean(acc, axis=0)
            out.append({"workload": label, "prefetch_trips": trips,
                        "reached_us": {names[i]: round(float(a[:, :, k].mean()), 2) for i, k in enumerate(order)},
                        "last_wavefront_done_us": round(float(a[:, :, 5].max()), 2),
                        "loop_done_first_half_of_grid_us": round(float(a[: n_wg // 2, :, 3].mean()), 2),
                        "loop_done_second_half_of_grid_us": round(float(a[n_wg // 2:, :, 3].mean()), 2)})
            print(json.dumps(out[-1]), file=sys.stderr, flush=True)
        _ffi.check(lib.tq_set_option(b"prefetch_trips", 1), "tq_set_option")
        del w
        torch.cuda.empty_cache()
    return out


def wide_phases(device, reps=20):
    """Time the wavefronts of one workgroup of the wide-head page kernel (head_dim 576) spend in each part of its loop,
    summed over the workgroup's blocks.  Needs a library built with -DWD_PROF (every wavefront of workgroup (0, 0, 0)
    then sums the 100 MHz real-time counter between the parts)."""
    import ctypes
    import numpy as np
    import torch
    from turboquant_amd import _ffi
    lib = _ffi.lib()
    if not hasattr(lib, "tq_debug_wide_prof"):
        raise SystemExit("this libtq_hip.so has no phase sums: build it with TQ_EXTRA_HIPCC_FLAGS=-DWD_PROF")
    fn = lib.tq_debug_wide_prof
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int]
    B, N, Hq, Hkv, d, kb, vb = 16, 8192, 8, 1, 576, 4, 4
    w = DecodeWorkload("wide head", B, N, Hq, Hkv, d, kb, vb, n_pools=2, seed=5, dist="normal", device=device, device_data=True)
    for i in range(300):
        w.step(i)
    torch.cuda.synchronize()
    kern = time_kernel_stage(w, 100, 20)
    acc = []
    for r in range(reps):
        w.step(r)
        torch.cuda.synchronize()
        buf = (ctypes.c_ulonglong * 96)()
        if fn(buf, 96) != 0:
            raise SystemExit("reading the phase sums failed")
        acc.append(np.frombuffer(buf, dtype=np.uint64).reshape(12, 8).astype(np.float64))
    a = np.mean(acc, axis=0) / 100.0                      # microseconds
    names = {0: "wait for page data", 1: "barrier", 2: "page requests", 3: "values", 4: "scores", 5: "softmax", 7: "loop overhead"}
    nw = d // 64
    n_waves = nw + (2 if nw + 2 <= 12 else 1)      # channel wavefronts + helpers
    return {"workload": f"{B} x {N}, {Hq} q / {Hkv} KV heads, head_dim {d}, keys {kb}b, values {vb}b", "n_split": w.n_split,
            "blocks_per_workgroup": (N // 32) // w.n_split, "kernel_us_with_the_counters_in": round(kern * 1e3, 2),
            "sums_over_the_loop_us": [{"wavefront": wv, **{names[k]: round(float(a[wv, k]), 2) for k in names},
                                       "total": round(float(a[wv].sum()), 2)} for wv in range(n_waves)]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=3000,
                    help="untimed steps before the timed ones; the card needs ~0.2 s of sustained work to reach its "
                         "steady clocks (with 50 steps the same build measures 5 %% slower decode steps and 17 %% "
                         "slower quantise passes)")
    ap.add_argument("--ramp-seconds", type=float, default=0.25,
                    help="untimed busy time before each leg's warm-up (clock ramp); 0 disables it")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-backend-step", action="store_true",
                    help="skip the full-decode-step leg (32-layer transformer through the backend hooks, ~60 GB)")
    ap.add_argument("--context", type=int, default=131072, help="context tokens per sequence of the main workload")
    ap.add_argument("--shapes", action="store_true",
                    help="time the decode step over SHAPE_TABLE instead (one JSON line with a row per shape; rows also "
                         "go to stderr as they finish)")
    ap.add_argument("--phase-stamps", action="store_true",
                    help="per-phase times inside the page kernel of the long-context and the 16 x 8192 workloads, from "
                         "the real-time counter stamps of a library built with TQ_EXTRA_HIPCC_FLAGS=-DTQ_STAMPS "
                         "(a profiling build; the shipped one has no stamps and this mode then exits)")
    ap.add_argument("--shape", action="append", default=[], metavar="B,N,Hq,Hkv,d,key_bits,value_bits",
                    help="with --shapes semantics, time this decode shape instead of the table (repeatable)")
    ap.add_argument("--wide-phases", action="store_true",
                    help="per-part time sums of the wide-head page kernel's loop (needs a library built with -DWD_PROF)")
    ap.add_argument("--quantize-only", action="store_true",
                    help="run the prefill-quantize leg alone and print its object (for profiles of its kernels)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path has no cross-GPU step and this build runs on a single MI355X; "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)

    global RAMP_SECONDS
    RAMP_SECONDS = max(0.0, args.ramp_seconds)
    import torch
    from turboquant_amd import _ffi
    if not os.path.exists(_ffi.library_path()):
        raise SystemExit("turboquant_amd/libtq_hip.so is missing; run `python -m turboquant_amd.build` first")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.shapes or args.shape:
        table = [tuple(int(x) for x in sh.split(",")) for sh in args.shape] or SHAPE_TABLE
        if any(len(sh) != 7 for sh in table):
            raise SystemExit("--shape takes seven comma-separated integers: B,N,Hq,Hkv,d,key_bits,value_bits")
        import contextlib
        with contextlib.redirect_stdout(sys.stderr):      # (a head size without a shipped codebook announces its computation)
            rows = shape_table(device, args.steps, args.warmup, table)
        print(json.dumps({"metric": "decode step over a table of shapes, 1 GPU", "steps": args.steps, "warmup": args.warmup,
                          "shapes": rows}))
        return

    if args.wide_phases:
        print(json.dumps({"metric": "wide-head page kernel, time per part of the loop, 1 GPU", "phases": wide_phases(device)}))
        return

    if args.phase_stamps:
        print(json.dumps({"metric": "page kernel phases, 1 GPU", "phases": phase_stamps(device)}))
        return

    if args.quantize_only:
        quant, _keep = quantize_bench(device, args.steps, args.warmup)
        print(json.dumps({"quantize": quant}))
        return

    main_w = DecodeWorkload("long-context decode", 4, args.context, 16, 2, 256, 3, 2, n_pools=4, seed=3,
                            dist="student_t5", device=device)
    ms, wall = time_steps(main_w.step, args.steps, args.warmup)
    kern_ms = time_kernel_stage(main_w, args.steps, args.warmup)
    value = main_w.bytes / (ms * 1e-3) / 1e9
    achieved = main_w.bytes / (kern_ms * 1e-3) / 1e9

    stream = stream_read_peak(main_w, max(20, args.steps // 4), max(5, args.warmup // 5))

    hybrid_main = hybrid_step_bench(main_w, max(20, args.steps // 4), max(5, args.warmup // 5))

    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "decode_pages_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            t = json.load(f)
        if t.get("context") == args.context:
            traffic = t.get("hbm_bytes_per_launch")
            traffic_source = ("stored profile figure, not measured in this run: profiles/decode_pages_traffic.json "
                              "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, scaled by a copy kernel)")

    gqa_w = DecodeWorkload("gqa decode", 16, 8192, 32, 8, 128, 3, 4, n_pools=4, seed=2, dist="normal", device=device)
    gqa_ms, _ = time_steps(gqa_w.step, args.steps, args.warmup)
    gqa_kern = time_kernel_stage(gqa_w, args.steps, args.warmup)
    hybrid_gqa = hybrid_step_bench(gqa_w, max(20, args.steps // 4), max(5, args.warmup // 5))
    gqa_cpu = None
    if not args.no_cpu:
        gqa_cpu = cpu_decode_baseline(gqa_w, runs=3)

    def side_leg(d, key_bits, text):
        w = DecodeWorkload(text, 16, 8192, 32, 8, d, key_bits, 4, n_pools=4, seed=2, dist="normal", device=device)
        ms_, _ = time_steps(w.step, args.steps, args.warmup)
        kern_ = time_kernel_stage(w, args.steps, args.warmup)
        leg = {"workload": text, "launches_per_step": launches_per_step(w),
               "bytes_per_step": w.bytes, "GBps": w.bytes / (ms_ * 1e-3) / 1e9, "ms_per_step": ms_,
               "pct_hbm_peak": 100.0 * w.bytes / (ms_ * 1e-3) / 1e9 / HBM_PEAK_GBS,
               "kernel_ms": kern_, "kernel_GBps": w.bytes / (kern_ * 1e-3) / 1e9,
               "kernel_frac": w.bytes / (kern_ * 1e-3) / 1e9 / HBM_PEAK_GBS}
        del w
        torch.cuda.empty_cache()
        return leg
    # the same shape with 4-bit keys (3-bit indices in nibbles + sign plane): the reference's default for the
    # first four layers (integration/vllm.py:358-359)
    kb4 = side_leg(128, 4, "16 seq x 8192 ctx, 32 q heads / 8 KV heads, head_dim 128, keys 4b, values 4b")
    # the smallest head size the reference ships codebooks for (codebooks/codebook_d64_b*.json); with 4 query heads
    # per KV head the kernel scores two pages per matrix instruction
    d64 = side_leg(64, 3, "16 seq x 8192 ctx, 32 q heads / 8 KV heads, head_dim 64, keys 3b, values 4b")

    quant, (qpool, qk, qv, qtable, qtq) = quantize_bench(device, max(5, args.steps // 5), max(2, args.warmup // 5))
    round_trip = round_trip_bench(device, max(5, args.steps // 5), max(2, args.warmup // 5), not args.no_cpu)

    backend = None
    if not args.no_backend_step:
        try:                     # a secondary leg (needs ~60 GB): its failure must not cost the headline line
            backend = backend_step_bench(device, min(20, max(5, args.steps // 10)), min(5, max(2, args.warmup // 10)))
        except Exception as exc:                                     # noqa: BLE001
            backend = {"error": f"{type(exc).__name__}: {exc}"}
            torch.cuda.empty_cache()

    cpu = None
    if not args.no_cpu:
        cpu = cpu_decode_baseline(main_w, runs=3)
        quant["cpu_baseline"] = cpu_quantize_baseline(qk, qv, qtq)

    line = {
        "metric": "compressed-KV decode attn GB/s (% HBM peak) + quantize tokens/s, 1 GPU",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 packed codes; scores: 4-term fp6 (e2m3) query x fp4 bit planes on the matrix cores, fp32 accumulate; "
                 "values: bf16-rounded weight x scale operands x exact bf16-denormal codes on the matrix cores, "
                 "fp32 accumulate; softmax fp32",
        "data": "synthetic (CPU generator seed 3; Student-t nu=5 K/V, N(0,1) queries, bf16; pages in a random permutation)",
        "config": {"workload": f"long-context decode: 4 seq x {args.context} ctx, 16 q heads / 2 KV heads, head_dim 256, "
                               "keys 3b (2b Lloyd-Max + 1b QJL, m=256), values 2b group 32, pages of 16, bf16 query",
                   "algorithmic_bytes_per_step": main_w.bytes, "stored_bytes_per_step": main_w.stored_bytes,
                   "n_split": main_w.n_split, "kv_pools_rotated": len(main_w.pools),
                   "launches_per_step": launches_per_step(main_w)},
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
        "wall_ms_per_step": wall, "clock_ramp_s": RAMP_SECONDS,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "decode_mfma_kernel", "kernel_ms": kern_ms, "stream_read": stream,
                     "frac_of_stream_read": achieved / stream["GBps"]},
        "quantize": quant,
        "round_trip": round_trip,
        "decode_gqa": {"workload": "16 seq x 8192 ctx, 32 q heads / 8 KV heads, head_dim 128, keys 3b, values 4b",
                       "launches_per_step": launches_per_step(gqa_w),
                       "note": "with at most 8 context splits the page kernel merges them itself (its last-arriving "
                               "workgroups), so kernel_ms includes that merge and no merge kernel follows",
                       "bytes_per_step": gqa_w.bytes, "GBps": gqa_w.bytes / (gqa_ms * 1e-3) / 1e9, "ms_per_step": gqa_ms,
                       "kernel_ms": gqa_kern, "kernel_GBps": gqa_w.bytes / (gqa_kern * 1e-3) / 1e9,
                       "kernel_frac": gqa_w.bytes / (gqa_kern * 1e-3) / 1e9 / HBM_PEAK_GBS,
                       "pct_hbm_peak": 100.0 * gqa_w.bytes / (gqa_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                       "cpu_baseline": gqa_cpu},
        "decode_gqa_kb4": kb4,
        "decode_gqa_d64": d64,
        "decode_hybrid": {"note": "whole step with the newest 128 tokens exact, read in place from a paged bf16 cache "
                                  "(tq_decode_attn_paged_ring); bytes = pages of the older tokens + the exact rows",
                          "long_context": hybrid_main, "gqa": hybrid_gqa},
        "backend_decode_step": backend,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
