// Page kernel on the matrix cores for wide heads: head_dim a multiple of 64 above 256, up to 704 (512 and 576 are the
// latent sizes of multi-head latent attention; the reference ships a codebook for 576, codebooks/codebook_d576_b3.json,
// and sizes its layers from impl.head_size / impl.kv_lora_rank, integration/vllm.py:376-381).  Same semantics as the
// other page kernels (score.py:114-173 over compressed pages): partials (m, l, acc[d]) per context split.
//
// A wide head does not fit the per-wavefront design of the head_dim 64 / 128 / 256 kernel (its query operands and
// accumulators would need several hundred registers), so here a whole workgroup works on one block of 32 tokens
// (two pages) at a time:
//   * one wavefront per 64 channels plus two helper wavefronts (one, when twelve wavefronts do not hold two), one
//     workgroup per compute unit;
//   * the pages travel HBM -> LDS as they lie in memory (LDS-direct loads, a kilobyte per instruction, all issued by a
//     helper wavefront): the key part of a page (bit planes, norms) and its value part (codes, scales, zero points)
//     into rings of their own, two or three blocks deep, so that the next block(s) arrive while the current ones
//     are worked on;
//   * the fp6 query operands of v_mfma_scale_f32_16x16x128_f8f6f4 (four terms per value, as the preparation
//     kernel of the other sizes packs them) are built by the workgroup itself from the fp32 rotated / sketched
//     queries and stay in LDS;
//   * scores: the (page, 128-coordinate chunk) pairs of a block are dealt to the wavefronts, the stored bit
//     planes are the fp4 operand, partial sums meet in LDS;
//   * softmax: a helper wavefront, online, log2 domain, against a reference that moves lazily;
//   * values: every channel wavefront takes the two groups of 32 channels it owns: codes masked in place are bf16
//     denormals (B operand), softmax weight x group scale is the A operand (rows 0..7 the heads with the even
//     group's scales, rows 8..15 with the odd group's), zero points through one more MFMA.
// The stages are pipelined over the blocks, three a block apart between two barriers: the values of block t, the
// softmax of block t + 1, the scores of block t + 2.  The step's other launches (rotation, exact tail, merge) are
// those of the general kernel.

#include "tq_decode_mfma_impl.h"

namespace tq {

constexpr int WD_BLK = 32;                 // tokens per iteration (two pages)
constexpr int WD_MAX_WAVES = 12;           // head_dim 768
constexpr int WD_MAX_CHUNKS = 6;           // 128-coordinate chunks of head_dim 768
constexpr int WD_SMALL_FLOATS = 2 * (256 + 256 + 8 + 8 + 64) + 32 + 16 + 16 + WD_MAX_WAVES * 32;   // two of (s_p, s_pv, s_alpha, s_flag, s_meta), s_stat, s_mult, s_coef, s_z
constexpr int WD_LDS_BYTES = 160 * 1024;

// -DWD_PROF (a profiling build, never the shipped one): every wavefront of workgroup (0, 0, 0) sums the time it
// spends in each part of an iteration (100 MHz counter); tq_debug_wide_prof copies the sums out.
#ifdef WD_PROF
__device__ unsigned long long wd_prof[WD_MAX_WAVES * 8];
__device__ unsigned long long wd_prof2[WD_MAX_WAVES * 8];   // prologue / epilogue stamps (absolute)
#define WD_P(k) do { wd_p[k] = wall_clock64(); } while (0)
#define WD_T(k) do { const unsigned long long t_ = wall_clock64(); wd_t[k] += t_ - wd_last; wd_last = t_; } while (0)
#else
#define WD_T(k)
#define WD_P(k)
#endif

__device__ __forceinline__ void wd_wait_vm(int n) {
#define WD_W(k) case k: stage_wait<k>(); break;
  switch (n) {
    WD_W(0) WD_W(1) WD_W(2) WD_W(3) WD_W(4) WD_W(5) WD_W(6) WD_W(7) WD_W(8) WD_W(9) WD_W(10) WD_W(11) WD_W(12) WD_W(13) WD_W(14) WD_W(15)
    WD_W(16) WD_W(17) WD_W(18) WD_W(19) WD_W(20) WD_W(21) WD_W(22) WD_W(23) WD_W(24) WD_W(25) WD_W(26) WD_W(27) WD_W(28) WD_W(29) WD_W(30)
    WD_W(31) WD_W(32) WD_W(33) WD_W(34) WD_W(35) WD_W(36) WD_W(37) WD_W(38) WD_W(39) WD_W(40) WD_W(41) WD_W(42) WD_W(43) WD_W(44) WD_W(45)
    WD_W(46) WD_W(47) WD_W(48)
    default: stage_wait<0>(); break;       // (stricter than asked: always safe)
  }
#undef WD_W
}

// The page geometry tq_page_layout_init gives 16-bit pages with groups of 32, and the kernel's LDS plan, as functions
// the compiler can evaluate: the instantiations for the head sizes 512 and 576 have every offset, slot size and trip
// count as a constant (a wavefront's scalar registers hold a fraction of what the run-time version keeps in them).
struct WideGeom { int off_meta, off_vdata, off_vscale, off_vzero, page_bytes, key_lane_major; };
__host__ __device__ constexpr WideGeom wide_geom(int d, int mb, int vb) {
  WideGeom g{};
  int off = (mb + 1) * (d / 8) * TQ_PAGE_TOKENS;
  g.off_meta = off;   off += 8 * TQ_PAGE_TOKENS;
  g.off_vdata = off;  off += d * vb * 2;
  g.off_vscale = off; off += (d / 32) * TQ_PAGE_TOKENS * 2;
  g.off_vzero = off;  off += (d / 32) * TQ_PAGE_TOKENS * 2;
  g.page_bytes = (off + 127) & ~127;
  g.key_lane_major = (d % 128 == 0 || d == 64) ? 1 : 0;
  return g;
}
struct WidePlan { int nring, kslot, vslot, smem; bool ok; };
__host__ __device__ constexpr WidePlan wide_plan_of(int d, int mb, int off_vdata, int page_bytes) {
  WidePlan p{};
  const int wplt = (d + 127) / 128, ntp = mb + (mb == 3 ? 1 : (mb == 4 ? 4 : 0)) + 1;
  p.kslot = off_vdata;                          // (multiples of 16; a slot is as long as its part of the page)
  p.vslot = page_bytes - off_vdata;
  const int qa_stride = wplt * WD_QA_OP - (d % 128 ? WD_QA_OP / 2 : 0);
  const int fixed = ntp * 2 * qa_stride * 4 + 2 * 2 * wplt * 1024 + WD_SMALL_FLOATS * 4;
  const int block = 2 * (p.kslot + p.vslot);
  p.nring = fixed + 3 * block <= WD_LDS_BYTES ? 3 : 2;
  // (the waits count the requests of the iteration behind the current one: an immediate operand, sixteen at most;
  // a wavefront keeps the constants of at most four requests of a kind)
  const int nw = d / 64, ops_k = (2 * ((p.kslot + 1023) / 1024) + nw - 1) / nw, ops_v = (2 * ((p.vslot + 1023) / 1024) + nw - 1) / nw;
  p.ok = p.kslot >= 1024 && p.vslot >= 1024 && fixed + 2 * block <= WD_LDS_BYTES && (p.nring == 2 || 2 * ((p.kslot + 1023) / 1024 + (p.vslot + 1023) / 1024) <= 48);
  (void)ops_k; (void)ops_v;
  p.smem = fixed + p.nring * block;
  return p;
}

// MB stored index planes; the codebooks the quantiser makes have NX = 0, 0, 1, 4 multi-bit Walsh terms for
// MB = 1..4, so MB + NX + 1 term planes go through the score MFMAs.
// D: the head size as a constant (512, 576), or 0: taken from the layer at run time.  F16P: fp16 pages.
template <int D, int VB, int MB, bool F16P>
__global__ void __launch_bounds__(768)
decode_wide_kernel(const float* __restrict__ q_rot, const float* __restrict__ q_sk, int Hq, int Hkv, int kv_div,
                   const uint8_t* __restrict__ pool, const int32_t* __restrict__ block_table, int bt_stride,
                   const int32_t* __restrict__ seq_lens, float sm_scale, tq_layer ly, tq_page_layout L_rt,
                   float* __restrict__ parts, int n_parts, int n_split, int len_sub, int max_pages, int num_pages,
                   int nring_rt, int kslot_rt, int vslot_rt, const uint32_t* __restrict__ qa_pre,
                   const float* __restrict__ q_stat_pre) {
  constexpr int NX = MB == 3 ? 1 : (MB == 4 ? 4 : 0), NTP = MB + NX + 1;
  constexpr bool f16p = F16P;                   // fp16 pages: scales and zero points are fp16 numbers
  const int d = D ? D : ly.d, W = d >> 5, WPLT = (d + 127) >> 7;
  // the page geometry and the LDS plan: constants when the head size is one
  constexpr WideGeom GC = wide_geom(D ? D : 512, MB, VB);
  constexpr WidePlan PC = wide_plan_of(D ? D : 512, MB, GC.off_vdata, GC.page_bytes);
  tq_page_layout L = L_rt;
  if (D) {
    L.d = D; L.mse_bits = MB; L.value_bits = VB; L.group_size = 32; L.key_lane_major = GC.key_lane_major; L.off_keys = 0;
    L.off_meta = GC.off_meta; L.off_vdata = GC.off_vdata; L.off_vscale = GC.off_vscale; L.off_vzero = GC.off_vzero;
    L.page_bytes = GC.page_bytes;
  }
  const int nring = D ? PC.nring : nring_rt, kslot = D ? PC.kslot : kslot_rt, vslot = D ? PC.vslot : vslot_rt;
  const int tid = threadIdx.x, lane = tid & 63;
  // NW wavefronts own 64 channels each and take a score unit each.  Wavefront NW owns no channels: it runs the softmax.
  // The last wavefront of the workgroup - a second helper, or the same one when the workgroup has no room for two -
  // issues the page requests and takes the score units the channel wavefronts leave over (head_dim 576: nine
  // channel wavefronts, ten units), so that no wavefront's chain in an iteration is much longer than values + one unit.
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), NWS = (int)blockDim.x >> 6, NW = D ? D / 64 : ly.d >> 6;
  const bool helper = wave == NW;
  const int n = lane & 15, kb = lane >> 4;
  const int split = blockIdx.x, b = blockIdx.z;
  // the query heads of a KV head form kv_div groups of at most 8 (consecutive groups read the same pages)
  const int g_tot = Hq / Hkv, kvh = (int)blockIdx.y / kv_div, grp = (int)blockIdx.y - kvh * kv_div;
  const int g_max = (g_tot + kv_div - 1) / kv_div;
  const int qbase = kvh * g_tot + grp * g_max;
  const int G = min(g_max, g_tot - grp * g_max);
  if (G <= 0) return;

#ifdef WD_PROF
  unsigned long long wd_p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#endif
  WD_P(0);
  extern __shared__ __align__(16) unsigned char smem_raw[];
  // Query operands: per (term plane, row set) the chunks one after another; a last chunk of 64 coordinates (head_dim
  // not a multiple of 128) takes half an operand - the slots of the lanes of its upper two coordinate quarters do not
  // exist: those lanes read what follows (always finite as fp6) against key words that are zero.
  const bool half_chunk = (d & 127) != 0;
  const int QA_STRIDE = WPLT * WD_QA_OP - (half_chunk ? WD_QA_OP / 2 : 0);    // dwords per (term plane, row set)
  uint32_t* qa_lds = (uint32_t*)smem_raw;                         // [NTP][2 row sets][QA_STRIDE]
  float* s_part = (float*)(qa_lds + NTP * 2 * QA_STRIDE);         // [2][2 WPLT units][64 lanes][4]
  float* s_p = s_part + 2 * 2 * WPLT * 256;                       // [2][8 heads][32 tokens] softmax weights
  float* s_pv = s_p + 2 * 256;                                    // [2]... the same weights times 2^(80 - bit position of the token's code)
  float* s_alpha = s_pv + 2 * 256;                                // [2][8]
  int* s_flag = (int*)(s_alpha + 2 * 8);                          // [2][8], [0] used: the block's softmax moved a reference
  float* s_meta = s_alpha + 4 * 8;                                // [2][2 pages][16 tokens][norm, residual norm]
  float* s_stat = s_meta + 2 * 64;                                // [8][4]: E_index, E_sign, constant parts of the score
  float* s_mult = s_stat + 32;                                    // [8][2]: multipliers of q_rot / q_sk
  float* s_coef = s_mult + 16;                                    // [16] coefficient of each term plane
  float* s_z = s_coef + 16;                                       // [waves][16 rows][2 groups] zero-point sums
  unsigned char* kring = (unsigned char*)(s_z + WD_MAX_WAVES * 32);   // [nring][2 pages][kslot]: bytes [0, off_vdata) of a page
  unsigned char* vring = kring + nring * 2 * kslot;                   // [nring][2 pages][vslot]: bytes [off_vdata, page_bytes)

  // ---------------------------------------------------------------- work range
  const int seq_len = max(min(seq_lens[b], max_pages * TQ_PAGE_TOKENS) - len_sub, 0);
  const int n_pages = (seq_len + TQ_PAGE_TOKENS - 1) / TQ_PAGE_TOKENS;
  const int n_blocks = (seq_len + WD_BLK - 1) / WD_BLK;
  const int per_split = (n_blocks + n_split - 1) / n_split;
  const int blk_begin = split * per_split, blk_end = min(blk_begin + per_split, n_blocks);
  if (blk_begin >= blk_end) {                                     // nothing to read: an empty partial
    for (int o = tid; o < G * (d + 2); o += blockDim.x) {
      const int g = o / (d + 2), e = o - g * (d + 2);
      parts[(((int64_t)b * Hq + qbase + g) * n_parts + split) * (d + 2) + e] = e == 0 ? MF_NEG * 0.6931471805599453f : 0.0f;
    }
    return;
  }
  const int32_t* bt = block_table + (int64_t)b * bt_stride;
  const uint8_t* pool_h = pool + (int64_t)kvh * L.page_bytes;
  const uint32_t page_stride32 = (uint32_t)((int64_t)Hkv * L.page_bytes);
  // Page numbers: lane l of tbl_a holds the table entry of page pbase + l, tbl_b that of page pbase + 64 + l (entries
  // past the end of the sequence repeat the last one, whose tokens are masked by position; an entry outside the
  // pool becomes page 0 with the top bit set: its tokens get no weight).  Looked up with a lane read; the pair
  // moves on 64 pages at a time, long before the entries are needed.
  int pbase = 2 * blk_begin;
  auto load_tbl = [&](int first) -> int {
    const int raw = bt[min(first + lane, n_pages - 1)];
    return (unsigned)raw < (unsigned)num_pages ? raw : (int)0x80000000;
  };
  // Block tables are device data nobody has checked: every wavefront looks once at the entries of the workgroup's
  // range, a lane per entry; only a workgroup that finds one outside the pool looks at the entries again, block by block.
  bool has_bad;
  {
    bool bad = false;
    const int e1 = min(2 * blk_end, n_pages);
    for (int e = 2 * blk_begin + lane; e < e1; e += 64) bad |= (unsigned)bt[e] >= (unsigned)num_pages;
    has_bad = __builtin_amdgcn_ballot_w64(bad) != 0;
  }
  int tbl_a = load_tbl(pbase), tbl_b = load_tbl(pbase + 64);
  // (used here, so that the compiler waits for the loads here and knows of no pending load inside the loop: a wait of
  // its own there would be for everything outstanding, the page requests included)
  asm volatile("" : "+v"(tbl_a), "+v"(tbl_b));
  auto page_entry = [&](int page) -> int {
    const int rel = __builtin_amdgcn_readfirstlane(min(page, n_pages - 1) - pbase);
    const int ea = __builtin_amdgcn_readlane(tbl_a, rel & 63), eb = __builtin_amdgcn_readlane(tbl_b, rel & 63);
    return rel < 64 ? ea : eb;
  };
  // Requests for the key part / value part of the next block of each kind into its ring slot, a kilobyte per
  // instruction.  Blocks are requested in order, so the block and its slot are running counters (every wavefront keeps
  // them); behind the last block of the range the requests repeat it (into the slot it already has).
  const int kbytes = L.off_vdata, vbytes = L.page_bytes - L.off_vdata;
  const int PK = (kbytes + 1023) >> 10, PV = (vbytes + 1023) >> 10;
  // One wavefront - the last of the workgroup, a helper - issues every request (the channel wavefronts' chains are the
  // longest of an iteration; a request costs a wavefront a third of a microsecond of its time whoever issues it).
  const bool requester = wave == NWS - 1;
  struct Req { int blk, slot; };
  Req rq_k{blk_begin, 0}, rq_v{blk_begin, 0};
  const uint32_t kring_lds = (uint32_t)(uintptr_t)kring, vring_lds = (uint32_t)(uintptr_t)vring;
  auto issue = [&](Req& r, uint32_t ring_lds, int slot_bytes, int pieces, int part_off, int part_bytes) __attribute__((always_inline)) {
    if (requester) {
      const uint32_t slot_lds = ring_lds + (uint32_t)(r.slot * 2 * slot_bytes);
      for (int pg = 0; pg < 2; ++pg) {
        const uint32_t pid = (uint32_t)page_entry(2 * r.blk + pg) & 0x7fffffffu;
        const uint8_t* base = pool_h + (uint64_t)pid * page_stride32 + part_off + lane * 16;
        for (int pc = 0; pc < pieces; ++pc) {
          const int at = min(pc * 1024, part_bytes - 1024);     // (the last piece overlaps the one before it: a slot is as long as its part)
          dma16<0>(base + at, (uint32_t)__builtin_amdgcn_readfirstlane((int)(slot_lds + (uint32_t)(pg * slot_bytes + at))));
        }
      }
    }
    if (r.blk < blk_end - 1) {
      ++r.blk;
      r.slot = r.slot + 1 == nring ? 0 : r.slot + 1;
    }
  };
  auto issue_keys = [&]() __attribute__((always_inline)) { issue(rq_k, kring_lds, kslot, PK, 0, kbytes); };
  auto issue_vals = [&]() __attribute__((always_inline)) { issue(rq_v, vring_lds, vslot, PV, kbytes, vbytes); };
  const int OPS_K = requester ? 2 * PK : 0, OPS_V = requester ? 2 * PV : 0;     // this wavefront's requests per block
  // the keys of the first blocks are on their way while the operands are prepared
  WD_P(1);
  for (int i = 0; i < nring - 1; ++i) issue_keys();
  WD_P(2);

  // ---------------------------------------------------------------- query operands
  int xpl = 0;                                  // four bits per multi-bit term: the stored planes it XORs
  {
    int seen = 0;
    for (int t = 0; t < ly.n_terms; ++t) {
      if (__builtin_popcount(ly.term_mask[t]) > 1 && seen < NX) {
        int pl = 0;
        for (int k2 = 0; k2 < MB; ++k2)
          if (ly.term_mask[t] & (1 << k2)) pl |= 1 << (MB - 1 - k2);
        xpl |= pl << (4 * seen++);
      }
    }
    xpl = __builtin_amdgcn_readfirstlane(xpl);
  }
  if (qa_pre != nullptr) {
    // Packed by the step's rotation launch, one copy per group of heads: fetched as they lie in memory, a kilobyte per
    // instruction, every wavefront its share; the statistics of the group's rows with them.
    const int total = NTP * 2 * QA_STRIDE * 4;  // bytes
    const uint8_t* src = (const uint8_t*)(qa_pre + ((int64_t)b * gridDim.y + blockIdx.y) * (NTP * 2 * QA_STRIDE));
    const uint32_t qa_at = (uint32_t)(uintptr_t)qa_lds;
    for (int pc = wave; pc < (total + 1023) >> 10; pc += NWS) {
      const int at = min(pc * 1024, total - 1024);
      dma16<0>(src + at + lane * 16, (uint32_t)__builtin_amdgcn_readfirstlane((int)(qa_at + (uint32_t)at)));
    }
    if (tid < 32) s_stat[tid] = (tid >> 2) < G ? q_stat_pre[((int64_t)b * Hq + qbase + (tid >> 2)) * 4 + (tid & 3)] : 0.0f;
    stage_wait<0>();
    __syncthreads();
    WD_P(3);
    // rows of the heads the group does not have: zero (nobody wrote them)
    for (int item = tid; item < NTP * (8 - G) * W; item += blockDim.x) {
      const int g = G + item % (8 - G), rest = item / (8 - G), j = rest % W, tp = rest / W;
      uint32_t* op0 = qa_lds + (tp * 2) * QA_STRIDE + (j >> 2) * WD_QA_OP;
      const int slot0 = 2 * g + 16 * (j & 3);
      const int hi_at = half_chunk && (j >> 2) == WPLT - 1 ? 32 * 4 : 64 * 4;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        uint32_t* op = op0 + (t >> 1) * QA_STRIDE;
        *(u32x4*)(op + (slot0 + (t & 1)) * 4) = u32x4{0, 0, 0, 0};
        *(uint2*)(op + hi_at + (slot0 + (t & 1)) * 2) = make_uint2(0u, 0u);
      }
    }
    __syncthreads();
    WD_P(4);
  } else {
  // packed here, as the preparation kernel of the other head sizes packs them
  float cmax = 0.0f;
  for (int t = 0; t < ly.n_terms; ++t) cmax = fmaxf(cmax, fabsf(ly.term_coef[t]));
  if (tid < 16) {
    float coef = 1.0f;                          // the sign plane
    if (tid < MB) {
      coef = 0.0f;
      for (int t = 0; t < ly.n_terms; ++t)
        if (ly.term_mask[t] == (1 << (MB - 1 - tid))) coef = ly.term_coef[t];
    } else if (tid < MB + NX) {
      coef = 0.0f;
      int seen = 0;
      for (int t = 0; t < ly.n_terms; ++t) {
        if (__builtin_popcount(ly.term_mask[t]) > 1) {
          if (seen == tid - MB) coef = ly.term_coef[t];
          ++seen;
        }
      }
    }
    s_coef[tid] = coef;
  }
  // row statistics, a wavefront per head: the largest |q_rot_j| / |q_sk_j| bound the operands (a power of two
  // 2^E above the bound goes into the MFMA's block scale), the sums give the constant parts of the score
  for (int r = wave; r < 8; r += NWS) {
    float mr = 0.0f, ms = 0.0f, s1 = 0.0f, s2 = 0.0f;
    if (r < G) {
      const float* xr = q_rot + ((int64_t)b * Hq + qbase + r) * d;
      const float* xs = q_sk + ((int64_t)b * Hq + qbase + r) * d;
      float x[WD_MAX_WAVES], y[WD_MAX_WAVES];   // (all loads first: one memory latency)
#pragma unroll
      for (int k = 0; k < WD_MAX_WAVES; ++k) {
        const int c = min(lane + 64 * k, d - 1);
        x[k] = xr[c];
        y[k] = xs[c];
      }
#pragma unroll
      for (int k = 0; k < WD_MAX_WAVES; ++k) {
        const bool in = lane + 64 * k < d;
        mr = fmaxf(mr, in ? fabsf(x[k]) : 0.0f);
        ms = fmaxf(ms, in ? fabsf(y[k]) : 0.0f);
        s1 += in ? x[k] : 0.0f;
        s2 += in ? y[k] : 0.0f;
      }
    }
    mr = wave_max_fast(mr); ms = wave_max_fast(ms);
    s1 = wave_sum_fast(s1); s2 = wave_sum_fast(s2);
    if (lane == 0) {
      const float k = sm_scale * 1.4426950408889634f;
      // bound < 2^e: e = exponent field - 126, kept within +-100
      const int e1 = min(max((int)((__float_as_uint(fabsf(k) * mr * cmax) >> 23) & 255u) - 126, -100), 100);
      const int e2 = min(max((int)((__float_as_uint(2.0f * fabsf(k * ly.qjl_scale) * ms) >> 23) & 255u) - 126, -100), 100);
      const bool live = r < G;
      s_stat[r * 4 + 0] = live ? (float)e1 : 0.0f;
      s_stat[r * 4 + 1] = live ? (float)e2 : 0.0f;
      s_stat[r * 4 + 2] = live ? k * ly.term_const * s1 : 0.0f;
      s_stat[r * 4 + 3] = live ? -k * ly.qjl_scale * s2 : 0.0f;
      s_mult[r * 2 + 0] = live ? k * __uint_as_float((uint32_t)(127 - e1) << 23) : 0.0f;
      s_mult[r * 2 + 1] = live ? 2.0f * k * ly.qjl_scale * __uint_as_float((uint32_t)(127 - e2) << 23) : 0.0f;
    }
  }
  __syncthreads();
  WD_P(3);
  // one lane per (term plane, head, plane word): the word's 32 values as four fp6 terms (the packing conversion
  // of gfx950 and its inverse for the residual), written where lane (row 2 head + term % 2, quarter word % 4) of
  // operand (plane, chunk word / 4, row set term / 2) reads them.  Rows of absent heads and the words past the
  // head's last one (a head that is not a multiple of 128 wide) are zero.
  {
    typedef float f32x16_t __attribute__((ext_vector_type(16)));
    typedef float f32x32_t __attribute__((ext_vector_type(32)));
    typedef uint32_t u32x6_t __attribute__((ext_vector_type(6)));
    const int n_items = NTP * 8 * 4 * WPLT;
    for (int item = tid; item < n_items; item += blockDim.x) {
      const int g = item & 7, j = (item >> 3) % (4 * WPLT), tp = (item >> 3) / (4 * WPLT);
      const bool is_sign = tp == NTP - 1, live = g < G && j < W;
      if (j >= W) continue;                 // (no slot: see half_chunk)
      uint32_t* op0 = qa_lds + (tp * 2) * QA_STRIDE + (j >> 2) * WD_QA_OP;
      const int slot0 = 2 * g + 16 * (j & 3);
      const int hi_at = half_chunk && (j >> 2) == WPLT - 1 ? 32 * 4 : 64 * 4;      // the operand's [lanes][2] part
      if (!live) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          uint32_t* op = op0 + (t >> 1) * QA_STRIDE;
          *(u32x4*)(op + (slot0 + (t & 1)) * 4) = u32x4{0, 0, 0, 0};
          *(uint2*)(op + hi_at + (slot0 + (t & 1)) * 2) = make_uint2(0u, 0u);
        }
        continue;
      }
      const float base = 4.0f * (is_sign ? s_mult[2 * g + 1] : s_coef[tp] * s_mult[2 * g]);
      // (the rows start on 8-byte boundaries of the workspace, not always on 16-byte ones)
      const float2* src = (const float2*)((is_sign ? q_sk : q_rot) + ((int64_t)b * Hq + qbase + g) * d + 32 * j);
      float x[32];
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const float2 v2 = src[k];
        x[2 * k] = v2.x; x[2 * k + 1] = v2.y;
      }
      f32x16_t va, vb;                      // contraction indices 0, 2, 4, ... and 1, 3, 5, ...
#pragma unroll
      for (int kloc = 0; kloc < 32; ++kloc) {
        const int c = 4 * (kloc & 7) + (kloc >> 3), t4 = kloc >> 3;      // coordinate within the word
        // (the page kernel takes three of a nibble's four bits in place, as the fp4 numbers 0.5, 1, 2)
        const float v = x[c] * (base * (t4 == 1 ? 0.5f : (t4 == 2 ? 0.25f : 1.0f)));
        if (kloc & 1) vb[kloc >> 1] = v;
        else va[kloc >> 1] = v;
      }
      const float one = 1.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        u32x6_t code;
        asm volatile("v_cvt_scalef32_2xpk16_fp6_f32 %0, %1, %2, %3" : "=&v"(code) : "v"(va), "v"(vb), "v"(one));
        uint32_t* op = op0 + (t >> 1) * QA_STRIDE;
        *(u32x4*)(op + (slot0 + (t & 1)) * 4) = u32x4{code[0], code[1], code[2], code[3]};
        *(uint2*)(op + hi_at + (slot0 + (t & 1)) * 2) = make_uint2(code[4], code[5]);
        if (t < 3) {
          f32x32_t r;
          asm volatile("v_cvt_scalef32_pk32_f32_fp6 %0, %1, %2" : "=&v"(r) : "v"(code), "v"(one));
#pragma unroll
          for (int k = 0; k < 16; ++k) {
            va[k] = (va[k] - r[2 * k]) * 32.0f;
            vb[k] = (vb[k] - r[2 * k + 1]) * 32.0f;
          }
        }
      }
    }
  }
  __syncthreads();
  WD_P(4);
  }
  // E8M0 block-scale codes of this lane's operand row (head n / 2; row 2g + t holds term t of row set 0 and term
  // t + 2 of row set 1): index planes row set 0, 1, sign plane row set 0, 1.  4 v / 2^E is stored, so term t
  // carries 2^(E - 2 - 5t); the fp4 bit value 0.5 carries 2^1.
  int sa;
  {
    const int e1 = 127 + (int)s_stat[(n >> 1) * 4 + 0], e2 = 127 + (int)s_stat[(n >> 1) * 4 + 1];
    const int t01 = (n & 1) ? 7 : 2, t23 = t01 + 10;
    sa = (e1 - t01) | ((e1 - t23) << 8) | ((e2 - t01) << 16) | ((e2 - t23) << 24);
  }
  const int sb = 127 + 1;
  // constant parts of the scores of the heads the helper wavefront sees in the softmax (heads 2 kb, 2 kb + 1)
  const float c_idx0 = s_stat[(2 * kb) * 4 + 2], c_idx1 = s_stat[(2 * kb + 1) * 4 + 2];
  const float c_sgn0 = s_stat[(2 * kb) * 4 + 3], c_sgn1 = s_stat[(2 * kb + 1) * 4 + 3];

  // ---------------------------------------------------------------- state
  f32x4 acc[4];                                 // channel tiles 4 wave .. 4 wave + 3
#pragma unroll
  for (int c = 0; c < 4; ++c) acc[c] = f32x4{0, 0, 0, 0};
  f32x4 zacc = {0, 0, 0, 0};
  float m_run[2] = {MF_NEG, MF_NEG}, l_run[2] = {0.0f, 0.0f};     // helper wavefront: heads 2 kb, 2 kb + 1
  const uint32_t m0 = VB == 2 ? 0x00030003u : (VB == 4 ? 0x000F000Fu : 0x00FF00FFu);
  const uint32_t m1 = VB == 2 ? 0x000C000Cu : 0x00F000F0u, m2 = 0x00300030u, m3 = 0x00C000C0u;
  // existing tokens of page pg of block blk: a prefix (none on a page outside the pool)
  auto tokens_of = [&](int blk, int pg) -> int {
    if (has_bad && page_entry(2 * blk + pg) < 0) return 0;
    return min(max(seq_len - blk * WD_BLK - 16 * pg, 0), 16);
  };

  // ---- scores of block blk: unit u = (page u % 2, chunk u / 2)
  auto score_units = [&](int ring_slot, int pb) __attribute__((always_inline)) {
    const unsigned char* kslot0 = kring + (ring_slot * 2) * kslot;
    float* part = s_part + pb * (2 * WPLT * 256);
    // unit `wave` for a channel wavefront; the units from NW on for the last wavefront of the workgroup (the second
    // helper, or the only one)
    const bool leftovers = wave == NWS - 1;
    for (int u = wave < NW ? wave : (leftovers ? NW : 2 * WPLT); u < 2 * WPLT; u += leftovers ? 1 : 2 * WPLT) {
      const int pg = u & 1, i = u >> 1;
      const unsigned char* kp = kslot0 + pg * kslot;
      const int j = 4 * i + kb;
      const int hi_at = half_chunk && i == WPLT - 1 ? 32 * 4 : 64 * 4;
      // (the unit of a page's first chunk hands the page's norms to the softmax, which runs an iteration later)
      if (i == 0 && kb == 0) *(f32x2*)(s_meta + pb * 64 + pg * 32 + n * 2) = *(const f32x2*)(kp + L.off_meta + n * 8);
      const bool jl = j < W;
      const int jc = jl ? j : W - 1;
      // the key words, then the planes in groups of at most five: every LDS read of a group (its operands of both row
      // sets) before the group's first MFMA
      uint32_t kw[MB + 1];
#pragma unroll
      for (int p = 0; p <= MB; ++p) {
        const uint32_t w = *(const uint32_t*)(kp + key_word_off(L, p, jc, n));
        kw[p] = jl ? w : 0u;
      }
      f32x4 dm0 = {0, 0, 0, 0}, dm1 = {0, 0, 0, 0}, dq0 = {0, 0, 0, 0}, dq1 = {0, 0, 0, 0};
      constexpr int TPG = NTP > 5 ? 5 : NTP;
#pragma unroll
      for (int t0 = 0; t0 < NTP; t0 += TPG) {
        i32x8 a[TPG][2];
#pragma unroll
        for (int q = 0; q < TPG; ++q)
#pragma unroll
          for (int rs = 0; rs < 2; ++rs) {
            const int tp = t0 + q < NTP ? t0 + q : NTP - 1;
            const uint32_t* op = qa_lds + (tp * 2 + rs) * QA_STRIDE + i * WD_QA_OP;
            const u32x4 lo = *(const u32x4*)(op + lane * 4);
            const uint2 hi = *(const uint2*)(op + hi_at + lane * 2);
            a[q][rs] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi.x, (int)hi.y, 0, 0};
          }
#pragma unroll
        for (int q = 0; q < TPG; ++q) {
          const int tp = t0 + q;
          if (tp < NTP) {
            uint32_t x;
            if (tp == NTP - 1) x = kw[MB];
            else if (tp < MB) x = kw[tp < MB ? tp : 0];
            else {
              const int pl = (xpl >> (4 * (tp - MB))) & 15;
              x = 0;
#pragma unroll
              for (int p = 0; p < MB; ++p) x ^= ((pl >> p) & 1) ? kw[p] : 0u;
            }
            const uint32_t b0 = x & 0x11111111u, b1 = x & 0x22222222u, b2 = x & 0x44444444u, b3 = (x >> 3) & 0x11111111u;
            if (tp == NTP - 1) {
              dq0 = mfma_f8f4<2>(a[q][0], b0, b1, b2, b3, dq0, sa, sb);
              dq1 = mfma_f8f4<3>(a[q][1], b0, b1, b2, b3, dq1, sa, sb);
            } else {
              dm0 = mfma_f8f4<0>(a[q][0], b0, b1, b2, b3, dm0, sa, sb);
              dm1 = mfma_f8f4<1>(a[q][1], b0, b1, b2, b3, dm1, sa, sb);
            }
          }
        }
        if (NTP > TPG) __builtin_amdgcn_sched_barrier(0);       // (the next group's operands after this group's MFMAs)
      }
      // lane (token n, rows 4 kb .. 4 kb + 3 = terms of heads 2 kb, 2 kb + 1)
      *(f32x4*)(part + (u * 64 + lane) * 4) = f32x4{(dm0[0] + dm0[1]) + (dm1[0] + dm1[1]), (dm0[2] + dm0[3]) + (dm1[2] + dm1[3]),
                                                      (dq0[0] + dq0[1]) + (dq1[0] + dq1[1]), (dq0[2] + dq0[3]) + (dq1[2] + dq1[3])};
    }
  };

  // ---- softmax of block blk (log2 domain, running reference), the helper wavefront: lane (token n of either page, heads
  // 2 kb, 2 kb + 1)
  auto softmax = [&](int blk, int pb) __attribute__((always_inline)) {
    const float* part = s_part + pb * (2 * WPLT * 256);
    float* sp = s_p + pb * 256;
    float* spv = s_pv + pb * 256;
    float s[2][2];
    bool valid[2];
    f32x4 t[2][WD_MAX_CHUNKS];
    f32x2 meta[2];
#pragma unroll
    for (int pg = 0; pg < 2; ++pg) {
      meta[pg] = *(const f32x2*)(s_meta + pb * 64 + pg * 32 + n * 2);
#pragma unroll
      for (int i = 0; i < WD_MAX_CHUNKS; ++i) t[pg][i] = *(const f32x4*)(part + ((2 * min(i, WPLT - 1) + pg) * 64 + lane) * 4);
    }
#pragma unroll
    for (int pg = 0; pg < 2; ++pg) {
      f32x4 sum = t[pg][0];
#pragma unroll
      for (int i = 1; i < WD_MAX_CHUNKS; ++i) {
        const f32x4 v = t[pg][i];
        sum += i < WPLT ? v : f32x4{0, 0, 0, 0};
      }
      valid[pg] = n < tokens_of(blk, pg);
      const float v0 = fmaf(meta[pg][0], sum[0] + c_idx0, meta[pg][1] * (sum[2] + c_sgn0));
      const float v1 = fmaf(meta[pg][0], sum[1] + c_idx1, meta[pg][1] * (sum[3] + c_sgn1));
      s[0][pg] = valid[pg] ? v0 : MF_NEG;
      s[1][pg] = valid[pg] ? v1 : MF_NEG;
    }
    // The reference of a head (weights are exp2(score - reference)) only moves when a score exceeds it by more than
    // a small slack, so the usual block rescales nothing; weights are at most 2^REF_SLACK.
    constexpr float REF_SLACK = 4.0f;
    // 2^(80 - s), s the bit position the code of token n has in its 16-bit half of a value operand register
    const float kpow = VB == 2 ? ((n & 3) == 0 ? 0x1p80f : ((n & 3) == 1 ? 0x1p78f : ((n & 3) == 2 ? 0x1p76f : 0x1p74f)))
                               : (VB == 4 ? ((n & 1) ? 0x1p76f : 0x1p80f) : 0x1p80f);
    bool moved = false;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int g = 2 * kb + jj;
      const float mx = row_max16(fmaxf(s[jj][0], s[jj][1]));
      const bool move = mx > m_run[jj] + REF_SLACK;
      const float m_new = move ? mx : m_run[jj];
      const float alpha = move ? __builtin_amdgcn_exp2f(m_run[jj] - m_new) : 1.0f;
      moved |= move;
      m_run[jj] = m_new;
      const float p0 = valid[0] ? __builtin_amdgcn_exp2f(s[jj][0] - m_new) : 0.0f;
      const float p1 = valid[1] ? __builtin_amdgcn_exp2f(s[jj][1] - m_new) : 0.0f;
      l_run[jj] = fmaf(l_run[jj], alpha, p0 + p1);
      sp[g * 32 + n] = p0;
      sp[g * 32 + 16 + n] = p1;
      spv[g * 32 + n] = p0 * kpow;
      spv[g * 32 + 16 + n] = p1 * kpow;
      if (n == 0) s_alpha[pb * 8 + g] = alpha;
    }
    const bool any_moved = __builtin_amdgcn_ballot_w64(moved) != 0;
    if (lane == 0) s_flag[pb * 8] = any_moved ? 1 : 0;
  };

  // ---- values of block blk: lane = (row n: head n % 8 with the scales of group 2 wave + n / 8; tokens
  // 8 (kb % 2) .. of page kb / 2)
  auto values = [&](int blk, int ring_slot, int pb) __attribute__((always_inline)) {
    const int hd = n & 7, gpar = n >> 3, pg = kb >> 1, u = kb & 1;
    // this lane's page in the value ring; offsets are those of the page record minus the key part
    const unsigned char* vp = vring + (ring_slot * 2 + pg) * vslot - L.off_vdata;
    const float* prow = s_p + pb * 256 + hd * 32 + pg * 16;
    const float* pvrow = s_pv + pb * 256 + hd * 32 + pg * 16;
    const bool rescale = __builtin_amdgcn_readfirstlane(s_flag[pb * 8]) != 0;
    // some tokens of the block do not exist (the ragged end of the sequence, a page outside the pool)
    const bool partial = tokens_of(blk, 0) < 16 || tokens_of(blk, 1) < 16;
    // weights in natural token order 8u .. 8u + 7 (the zero points' operand)
    float pn[8];
    {
      const f32x4 t0 = *(const f32x4*)(prow + 8 * u), t1 = *(const f32x4*)(prow + 8 * u + 4);
      pn[0] = t0[0]; pn[1] = t0[1]; pn[2] = t0[2]; pn[3] = t0[3];
      pn[4] = t1[0]; pn[5] = t1[1]; pn[6] = t1[2]; pn[7] = t1[3];
    }
    // weights (with the code position folded in) and scales of the tokens whose codes this lane's operand registers
    // hold: register r carries token tk(r, 0) in its low half and tk(r, 1) in its high half
    float pw[4][2], sc[4][2];
    const unsigned char* srow = vp + L.off_vscale + ((2 * wave + gpar) * 16) * 2;
    auto widen = [&](uint32_t w, float& lo, float& hi) {
      lo = f16p ? f16_lo(w) : __uint_as_float(w << 16);
      hi = f16p ? f16_hi(w) : __uint_as_float(w & 0xffff0000u);
    };
    if (VB == 2) {
      // tk(r, h) = 4u + r + 8h
      const f32x4 t0 = *(const f32x4*)(pvrow + 4 * u), t1 = *(const f32x4*)(pvrow + 4 * u + 8);
      const uint2 s0 = *(const uint2*)(srow + (4 * u) * 2), s1 = *(const uint2*)(srow + (4 * u + 8) * 2);
      float f0[4], f1[4];
      widen(s0.x, f0[0], f0[1]); widen(s0.y, f0[2], f0[3]);
      widen(s1.x, f1[0], f1[1]); widen(s1.y, f1[2], f1[3]);
#pragma unroll
      for (int r = 0; r < 4; ++r) { pw[r][0] = t0[r]; pw[r][1] = t1[r]; sc[r][0] = f0[r]; sc[r][1] = f1[r]; }
    } else {
      const f32x4 t0 = *(const f32x4*)(pvrow + 8 * u), t1 = *(const f32x4*)(pvrow + 8 * u + 4);
      const float pv[8] = {t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
      const u32x4 sv = *(const u32x4*)(srow + (8 * u) * 2);
      float f[8];
      widen(sv[0], f[0], f[1]); widen(sv[1], f[2], f[3]); widen(sv[2], f[4], f[5]); widen(sv[3], f[6], f[7]);
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int k = VB == 4 ? r + 4 * h : 4 * (r >> 1) + (r & 1) + 2 * h;     // token - 8u
          pw[r][h] = pv[k];
          sc[r][h] = f[k];
        }
    }
    u32x4 bz = *(const u32x4*)(vp + L.off_vzero + ((2 * wave + (n & 1)) * 16 + 8 * u) * 2);
    uint32_t fw[4][VB == 8 ? 2 : 1];
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const uint32_t* field = (const uint32_t*)(vp + L.off_vdata + (n * (d >> 4) + 4 * wave + cc) * (VB * 2));
      if (VB == 2) fw[cc][0] = field[0] >> (8 * u);
      else if (VB == 4) fw[cc][0] = field[u];
      else { fw[cc][0] = field[2 * u]; fw[cc][VB == 8 ? 1 : 0] = field[2 * u + 1]; }
    }
    if (rescale) {
      const f32x4 a4 = *(const f32x4*)(s_alpha + pb * 8 + 4 * (kb & 1));   // accumulator rows 4 kb .. 4 kb + 3 = heads 4 (kb % 2) ..
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] *= a4;
      zacc *= a4;
    }
    // a code masked in place at bit s of its 16-bit half is the bf16 number code x 2^(s - 133); the weight carries 2^(80 - s)
    u32x4 aw;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float w0 = pw[r][0] * sc[r][0], w1 = pw[r][1] * sc[r][1];
      if (partial) {      // (a slot past the end of the sequence may hold any scale: its weight is an exact zero)
        w0 = pw[r][0] != 0.0f ? w0 : 0.0f;
        w1 = pw[r][1] != 0.0f ? w1 : 0.0f;
      }
      aw[r] = pack_bf16(w0, w1);
    }
    // zero points of this wavefront's two groups (columns n % 2; the other columns repeat them)
    {
      u32x4 ap;
#pragma unroll
      for (int r = 0; r < 4; ++r) ap[r] = f16p ? pack_f16(pn[2 * r], pn[2 * r + 1]) : pack_bf16(pn[2 * r], pn[2 * r + 1]);
      if (partial) {
        const int left = tokens_of(blk, pg) - 8 * u;            // existing tokens among this lane's eight
#pragma unroll
        for (int r = 0; r < 4; ++r) bz[r] &= (2 * r < left ? 0x0000ffffu : 0u) | (2 * r + 1 < left ? 0xffff0000u : 0u);
      }
      zacc = f16p ? mfma_f16(ap, bz, zacc) : mfma(ap, bz, zacc);
    }
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      u32x4 bc;
      if (VB == 2) {
        const uint32_t x = fw[cc][0];
        bc = u32x4{x & m0, x & m1, x & m2, x & m3};
      } else if (VB == 4) {
        const uint32_t x = fw[cc][0], x8 = x >> 8;
        bc = u32x4{x & m0, x & m1, x8 & m0, x8 & m1};
      } else {
        const uint32_t x = fw[cc][0], y = fw[cc][VB == 8 ? 1 : 0];
        bc = u32x4{x & m0, (x >> 8) & m0, y & m0, (y >> 8) & m0};
      }
      acc[cc] = mfma(aw, bc, acc[cc]);
    }
  };

  // ---------------------------------------------------------------- the blocks
  // Three stages, a block apart, between two barriers: iteration t accumulates the values of block t, runs the
  // softmax of block t + 1 (the helper) and scores block t + 2; the score sums, the norms and the softmax weights are
  // double-buffered (block % 2).  Iteration t requests the keys of block t + nring + 1 and the values of block
  // t + nring - 1 into the slots the blocks t + 1 and t - 1 had, so at its top the requests of iteration t - nring + 1
  // (keys t + 2, values t) have to have landed and those of the nring - 2 iterations after it may be outstanding.
  int ks = 0, vs = 0;                           // ring slots of the keys of block t + 2 and the values of block t
#ifdef WD_PROF
  unsigned long long wd_t[8] = {0, 0, 0, 0, 0, 0, 0, 0}, wd_last = wall_clock64();
#endif
  for (int t = blk_begin - 2; t < blk_end; ++t) {
    WD_T(7);
    // (the iterations before block 0's values are requested issue keys only)
    wd_wait_vm(nring == 2 ? 0 : OPS_K + (t - 1 >= blk_begin - nring + 1 ? OPS_V : 0));
    WD_T(0);
    __syncthreads();
    WD_T(1);
    if (t >= blk_begin && 2 * t >= pbase + 64) {                  // (uniform) the table registers move on
      pbase += 64;
      tbl_a = tbl_b;
      tbl_b = load_tbl(pbase + 64);
      asm volatile("" : "+v"(tbl_b));           // (the wait for this load: here, once in 32 blocks)
    }
    issue_keys();
    if (t >= blk_begin - nring + 1) issue_vals();
    WD_T(2);
    if (t >= blk_begin) {
      if (wave < NW) values(t, vs, t & 1);
      vs = vs + 1 == nring ? 0 : vs + 1;
    }
    WD_T(3);
    if (t + 2 < blk_end) score_units(ks, t & 1);
    ks = ks + 1 == nring ? 0 : ks + 1;
    WD_T(4);
    if (helper && t + 1 >= blk_begin && t + 1 < blk_end) softmax(t + 1, (t + 1) & 1);
    WD_T(5);
  }
  WD_P(5);
#ifdef WD_PROF
  if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && lane == 0)
    for (int k = 0; k < 8; ++k) wd_prof[wave * 8 + k] = wd_t[k];
#endif

  // ---------------------------------------------------------------- the partial (m, l, acc[d]) of every head
  stage_wait<0>();                              // the surplus requests of the last trips have landed
  __syncthreads();
  if (n < 2 && wave < NW) {
#pragma unroll
    for (int i = 0; i < 4; ++i) s_z[(wave * 16 + 4 * kb + i) * 2 + n] = zacc[i];
  }
  if (helper) {
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const float lsum = row_sum16(l_run[jj]);
      const int g = 2 * kb + jj;
      if (n == 0 && g < G) {
        float* r = parts + (((int64_t)b * Hq + qbase + g) * n_parts + split) * (d + 2);
        r[0] = m_run[jj] * 0.6931471805599453f;     // natural-log domain
        r[1] = lsum;
      }
    }
  }
  __syncthreads();
  // accumulator rows 0..7 hold the heads for the tiles of the even group (tiles 0, 1), rows 8..15 for the odd
  // group (tiles 2, 3); the zero-point sums have the same rows in both halves
  if (wave < NW) {
    const int par = kb >> 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int g = 4 * (kb & 1) + i;
      if (g < G) {
        const float z = s_z[(wave * 16 + 4 * kb + i) * 2 + par];
        float* row = parts + (((int64_t)b * Hq + qbase + g) * n_parts + split) * (d + 2) + 2 + 64 * wave + 32 * par + n;
        row[0] = fmaf(par ? acc[2][i] : acc[0][i], 0x1p53f, z);
        row[16] = fmaf(par ? acc[3][i] : acc[1][i], 0x1p53f, z);
      }
    }
  }
  WD_P(6);
#ifdef WD_PROF
  if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && lane == 0)
    for (int k = 0; k < 8; ++k) wd_prof2[wave * 8 + k] = wd_p[k];
#endif
}

// LDS plan of the kernel for a layer: ring depth, slot sizes, bytes; false when it does not fit
static bool wide_plan(const tq_layer& ly, const tq_page_layout& L, int& nring, int& kslot, int& vslot, size_t& smem) {
  const int mb = ly.mse_bits;
  int nx = 0;
  for (int t = 0; t < ly.n_terms; ++t)
    if (__builtin_popcount(ly.term_mask[t]) > 1) ++nx;
  if (mb < 1 || mb > 4 || nx != (mb == 3 ? 1 : (mb == 4 ? 4 : 0))) return false;
  const WidePlan p = wide_plan_of(ly.d, mb, L.off_vdata, L.page_bytes);
  nring = p.nring; kslot = p.kslot; vslot = p.vslot; smem = (size_t)p.smem;
  return p.ok;
}

// whether the page layout is the one the constant-geometry instantiations assume
static bool wide_geom_matches(const tq_page_layout& L) {
  const WideGeom g = wide_geom(L.d, L.mse_bits, L.value_bits);
  return L.off_keys == 0 && L.off_meta == g.off_meta && L.off_vdata == g.off_vdata && L.off_vscale == g.off_vscale &&
         L.off_vzero == g.off_vzero && L.page_bytes == g.page_bytes && L.key_lane_major == g.key_lane_major && L.group_size == 32;
}

bool decode_wide_has_kernel(const tq_layer& ly, const tq_page_layout& L) {
  const int d = ly.d;
  if (opt_wide_heads.load(std::memory_order_relaxed) == 0) return false;
  // (d + 64 threads: at most twelve wavefronts, three per SIMD, with the helper)
  if (d <= 256 || d > 704 || (d & 63) || L.d != d || L.mse_bits != ly.mse_bits) return false;
  if ((L.dtype != TQ_BF16 && L.dtype != TQ_F16) || L.group_size != 32) return false;
  if (L.value_bits != 2 && L.value_bits != 4 && L.value_bits != 8) return false;
  if (ly.n_terms <= 0) return false;
  int nring, kslot, vslot;
  size_t smem;
  return wide_plan(ly, L, nring, kslot, vslot, smem);
}

int decode_wide_term_planes(const tq_layer& ly) {
  const int mb = ly.mse_bits;
  int nx = 0;
  for (int t = 0; t < ly.n_terms; ++t)
    if (__builtin_popcount(ly.term_mask[t]) > 1) ++nx;
  if (mb < 1 || mb > 4 || ly.n_terms <= 0 || nx != (mb == 3 ? 1 : (mb == 4 ? 4 : 0))) return 0;
  return mb + nx + 1;
}

// Returns TQ_EUNSUPPORTED when the shape has no wide-head kernel (nothing was launched).
int launch_decode_wide(const float* q_rot, const float* q_sk, int B, int Hq, int Hkv, const uint8_t* pool,
                       const int32_t* block_table, int bt_stride, const int32_t* seq_lens, float sm_scale,
                       const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts, int n_split, int len_sub,
                       int max_pages, int num_pages, const WidePack& pre, hipStream_t st) {
  if (!decode_wide_has_kernel(ly, L)) return TQ_EUNSUPPORTED;
  const int g_tot = Hq / Hkv, kv_div = (g_tot + 7) / 8;
  if (g_tot < 1 || g_tot > 128 || (int64_t)Hkv * kv_div > 65535) return TQ_EUNSUPPORTED;
  int nring, kslot, vslot;
  size_t smem;
  wide_plan(ly, L, nring, kslot, vslot, smem);
  // helpers beside the d / 64 channel wavefronts: one for the softmax, one for the page requests and the score units the
  // channel wavefronts leave over (one for both when that would be more than twelve wavefronts)
  const int nw = ly.d / 64, units = 2 * ((ly.d + 127) / 128);
  const int helpers = nw + 2 <= WD_MAX_WAVES ? 2 : 1;
  (void)units;
  const dim3 grid(n_split, Hkv * kv_div, B), block((nw + helpers) * 64);
  hipEvent_t t_start = nullptr, t_stop = nullptr;
  const bool timed = take_time_hook(0, t_start, t_stop);
#define TQ_LAUNCH_WIDE(D, VB, MB)                                                                                     \
  {                                                                                                                   \
    auto kern = L.dtype == TQ_F16 ? decode_wide_kernel<D, VB, MB, true> : decode_wide_kernel<D, VB, MB, false>;                                                                        \
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);     \
    if (e != hipSuccess) return (int)e;                                                                               \
    if (timed)                                                                                                        \
      hipExtLaunchKernelGGL(kern, grid, block, smem, st, t_start, t_stop, 0, q_rot, q_sk, Hq, Hkv, kv_div, pool,      \
                            block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts, n_split, len_sub,      \
                            max_pages, num_pages, nring, kslot, vslot, pre.qa, pre.q_stat);                           \
    else                                                                                                              \
      kern<<<grid, block, smem, st>>>(q_rot, q_sk, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, \
                                      ly, L, parts, n_parts, n_split, len_sub, max_pages, num_pages, nring, kslot,    \
                                      vslot, pre.qa, pre.q_stat);                                                     \
  }
#define TQ_LAUNCH_WIDE_MB(D, VB)                        \
  {                                                     \
    if (ly.mse_bits == 1) TQ_LAUNCH_WIDE(D, VB, 1)      \
    else if (ly.mse_bits == 2) TQ_LAUNCH_WIDE(D, VB, 2) \
    else if (ly.mse_bits == 3) TQ_LAUNCH_WIDE(D, VB, 3) \
    else TQ_LAUNCH_WIDE(D, VB, 4)                       \
  }
#define TQ_LAUNCH_WIDE_VB(D)                            \
  {                                                     \
    if (L.value_bits == 2) TQ_LAUNCH_WIDE_MB(D, 2)      \
    else if (L.value_bits == 4) TQ_LAUNCH_WIDE_MB(D, 4) \
    else TQ_LAUNCH_WIDE_MB(D, 8)                        \
  }
  // the head sizes of latent attention have instantiations with constant geometry (for the layout the library makes)
  const bool fixed_geom = wide_geom_matches(L) && opt_wide_heads.load(std::memory_order_relaxed) != 2;
  if (fixed_geom && ly.d == 576) TQ_LAUNCH_WIDE_VB(576)
  else if (fixed_geom && ly.d == 512) TQ_LAUNCH_WIDE_VB(512)
  else TQ_LAUNCH_WIDE_VB(0)
#undef TQ_LAUNCH_WIDE_VB
#undef TQ_LAUNCH_WIDE_MB
#undef TQ_LAUNCH_WIDE
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

}  // namespace tq

#ifdef WD_PROF
extern "C" int tq_debug_wide_prof(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(tq::wd_prof), (size_t)n * 8);
}
extern "C" int tq_debug_wide_prof2(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(tq::wd_prof2), (size_t)n * 8);
}
#endif
