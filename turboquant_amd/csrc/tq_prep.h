// Query preparation of the matrix-core decode kernel (device code shared by two launches).
#pragma once

#include "tq_common.h"
#include "tq_decode_mfma.h"

namespace tq {

constexpr int ROT_MAX_ROWS = 8;      // query heads one preparation workgroup handles

// Fused preparation of the matrix-core decode kernel: rotation, sketch, statistics and
// operand packing in one launch.  A workgroup owns one GQA group (G query heads of one KV
// head) and the 32 output coordinates of one plane word; PREP_SLICES threads share a
// coordinate's contraction.  Nothing depends on another workgroup, because the operands
// are normalised by bounds that every workgroup can compute from the raw query:
// |q_rot_j| <= ||q|| (Pi is orthogonal) and |q_sk_j| <= ||q|| max_j ||S_j||, and the sums
// over all coordinates that the decode kernel needs are q . colsum(Pi), q . colsum(S).
//
// Everything that multiplies a whole score is folded into the operands: with k = sm_scale log2(e)
// the index planes carry  k coef q_rot_j  and the sign plane  2 k qjl_scale q_sk_j, each divided
// by a power of two 2^E >= its bound (E per query head and kind), which the decode kernel gives
// back through the MFMA's per-row block scale.  q_stat per row:
// {E_index, E_sign (as floats), k c0 sum_j q_rot_j, -k qjl_scale sum_j q_sk_j}: the last two
// are the constant parts of the score and start the MFMA accumulators.
//
// qa_pack receives the score-stage A operands of v_mfma_scale_f32_16x16x128_f8f6f4 (A fp6 e2m3, which
// runs at twice the fp8 rate; B fp4) in register order: [kv head][term plane][128-coordinate chunk i]
// [row set][lane][8 dwords, 6 used].  A value v (the normalised query coordinate times the plane's
// coefficient, |v| <= 1) is the sum of four fp6 terms with per-row block scales 2^-2, 2^-7, 2^-12,
// 2^-17: t0 = fp6(4 v), t1 = fp6(32 (4 v - t0)), t2 = fp6(32 (32 (4 v - t0) - t1)), ...; a term's
// rounding error is at most 1/8, so every product stays within the fp6 range and the sum is good to
// 2^-20.  Row set 0 holds terms 0 and 1 (row 2g + t for head g), row set 1 terms 2 and 3, so that
// both accumulate into the same MFMA output registers (8 heads x 4 terms fill the 2 x 16 rows).  For 6-bit operands lane
// (row, block b) holds contraction indices 32b..32b+31, index j at bits 6j..6j+5 of its 192 bits, and
// the key kernel puts coordinate c of plane word w at contraction index 32w + 8 (c % 4) + c / 4.
constexpr int PREP_COLS = 32, PREP_SLICES = 16;

// round to the fp6 e2m3 grid (1 sign, 2 exponent, 3 mantissa bits; steps 1/8 below 2, 1/4 below 4,
// 1/2 up to the maximum 7.5), nearest even; returns the rounded value and its 6-bit code
__device__ __forceinline__ float round_fp6(float v, uint32_t& code) {
  const float a = fminf(fabsf(v), 7.5f);
  const float inv_step = a < 2.0f ? 8.0f : (a < 4.0f ? 4.0f : 2.0f);
  const float step = a < 2.0f ? 0.125f : (a < 4.0f ? 0.25f : 0.5f);
  const float r = rintf(a * inv_step) * step;        // exact (powers of two); may land on the next binade
  const int e = r < 1.0f ? 0 : (r < 2.0f ? 1 : (r < 4.0f ? 2 : 3));
  const float inv_unit = e <= 1 ? 8.0f : (e == 2 ? 4.0f : 2.0f);
  const int m = (int)(r * inv_unit) - (e == 0 ? 0 : 8);
  code = (v < 0.0f && r != 0.0f ? 32u : 0u) | ((uint32_t)e << 3) | (uint32_t)m;
  return v < 0.0f ? -r : r;
}

// sum over the 64 lanes with DPP row operations and four lane reads (no shared-memory permutes)
template <int CTRL>
__device__ __forceinline__ float prep_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v += prep_dpp<0xB1>(v);      // quad_perm [1,0,3,2]
  v += prep_dpp<0x4E>(v);      // quad_perm [2,3,0,1]
  v += prep_dpp<0x141>(v);     // row_half_mirror
  v += prep_dpp<0x140>(v);     // row_mirror: every lane holds its row's sum
  const int b = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
}

// PER = matrix rows per thread = d / PREP_SLICES; DT = element type of the query (a template parameter:
// a run-time switch would put each query load under a branch, and the loads would wait for one another)
// (a device function: the stand-alone kernel and the launch that shares its grid with the exact-tail
// workgroups both run it; `unit` / `word` are the workgroup's coordinates, `sm` its dynamic LDS.)
// A workgroup works on gpw consecutive groups of G heads (gpw x G <= ROT_MAX_ROWS rows; rows of consecutive
// groups are consecutive), the last workgroup possibly on fewer (n_rows = all rows = groups x G).  One group per
// workgroup is the shortest chain and what a launch that fits the card at once wants; a launch of thousands of
// units is bound by how many workgroups it takes, and then two groups of 4 heads, four of 2, ... share one
// (prep_groups_per_workgroup).  `arrivals`: the groups' arrival counters, zeroed here for a page kernel that
// merges its splits itself.
// units = workgroups of the launch with one group each, slots = workgroups the card holds at once
__host__ __device__ inline int prep_groups_per_workgroup(int G, int64_t units, int64_t slots) {
  return units > slots && G >= 1 && G <= ROT_MAX_ROWS ? ROT_MAX_ROWS / G : 1;
}

// PACKED: gpw may exceed 1.  One group per workgroup is a build of its own (no row bounds, no head / group
// arithmetic in the packing lanes): it is the one the latency-bound launches take, and half a microsecond shorter.
// g_tot > 0 (one group per workgroup only): the groups tile runs of g_tot consecutive rows - the query heads of one
// KV head - instead of the whole row range: group i of a run has rows i G .. min((i + 1) G, g_tot) - 1, so the last
// group of every run is shorter when G does not divide g_tot (11 heads per KV head: groups of 6 and 5).
template <int PER, int DT, bool PACKED>
__device__ __forceinline__ void prep_query_body(const void* __restrict__ q, int G, int gpw, int64_t n_rows, int g_tot, const tq_layer& ly,
                                                float sm_scale, float* __restrict__ q_rot, float* __restrict__ q_sk,
                                                float* __restrict__ q_stat, uint32_t* __restrict__ qa_pack,
                                                unsigned long long* __restrict__ arrivals, int head_rows, int64_t unit,
                                                int word, float* sm) {
  const int d = ly.d, tid = threadIdx.x, jl = tid % PREP_COLS, sl = tid / PREP_COLS;
  const int j = word * PREP_COLS + jl;
  const int RG = PACKED ? G * gpw : G;                                 // rows a workgroup has room for
  int64_t row0 = unit * RG;
  const int64_t group0 = PACKED ? unit * gpw : unit;
  int R = PACKED ? (int)(n_rows - row0 < RG ? n_rows - row0 : RG) : G;      // rows of this workgroup (PACKED: a multiple of G)
  if (!PACKED && g_tot > 0) {
    const int per = (g_tot + G - 1) / G;
    const int64_t run = unit / per;
    const int i = (int)(unit - run * per);
    row0 = run * g_tot + (int64_t)i * G;
    R = g_tot - i * G < G ? g_tot - i * G : G;
  }
  if (arrivals != nullptr && word == 0 && tid < (PACKED ? gpw : 1) && tid * G < R) arrivals[group0 + tid] = 0ull;
  // every global load of the kernel is issued here, before anything waits, the query first: loads
  // return in order, so the query can go to shared memory (and its statistics be taken) while the
  // matrix slices, which do not depend on it, are still on their way
  constexpr int QPT = ROT_MAX_ROWS * 256 / (PREP_COLS * PREP_SLICES);   // query elements per thread, d <= 256
  float qv[QPT];
#pragma unroll
  for (int k = 0; k < QPT; ++k) {
    const int o = tid + k * (PREP_COLS * PREP_SLICES);
    const float x = Elem<DT>::load(q, row0 * d + min(o, R * d - 1));      // unconditional, clamped
    qv[k] = o < R * d ? x : 0.0f;
  }
  float mp[PER], ms[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    mp[k] = ly.PiT[(int64_t)(sl * PER + k) * d + j];
    ms[k] = ly.ST[(int64_t)(sl * PER + k) * d + j];
  }
  float cs1[4], cs2[4];                            // column sums at coordinates lane, lane + 64, ...
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int c = (tid & 63) + 64 * k;
    cs1[k] = c < d ? ly.Pi_colsum[c] : 0.0f;
    cs2[k] = c < d ? ly.S_colsum[c] : 0.0f;
  }
  float* sq = sm;                                   // [RG][d] raw query
  float* pa = sq + RG * d;                          // [PREP_SLICES][RG][PREP_COLS]
  float* pb = pa + PREP_SLICES * RG * PREP_COLS;
  float* srot = pb + PREP_SLICES * RG * PREP_COLS;  // [RG][PREP_COLS]
  float* ssk = srot + RG * PREP_COLS;
  float* stat = ssk + RG * PREP_COLS;               // [RG][4]
  float* coefs = stat + 4 * ROT_MAX_ROWS;           // [16]
#pragma unroll
  for (int k = 0; k < QPT; ++k) {
    const int o = tid + k * (PREP_COLS * PREP_SLICES);
    if (o < R * d) sq[o] = qv[k];
  }
  const int mb = ly.mse_bits;
  int nx = 0;
  float cmax = 0.0f;
  for (int t = 0; t < ly.n_terms; ++t) {
    cmax = fmaxf(cmax, fabsf(ly.term_coef[t]));
    if (__builtin_popcount(ly.term_mask[t]) > 1) ++nx;
  }
  const int ntp = mb + nx + 1, wpl = d >= 128 ? d / 128 : 1;      // head_dim 64: one chunk of 128 with its upper half unused
  if (tid < ntp) {
    float coef = 1.0f;
    if (tid < mb) {
      coef = 0.0f;
      for (int t = 0; t < ly.n_terms; ++t)
        if (ly.term_mask[t] == (1 << (mb - 1 - tid))) coef = ly.term_coef[t];
    } else if (tid < mb + nx) {
      coef = 0.0f;
      int seen = 0;
      for (int t = 0; t < ly.n_terms; ++t) {
        if (__builtin_popcount(ly.term_mask[t]) > 1) {
          if (seen == tid - mb) coef = ly.term_coef[t];
          ++seen;
        }
      }
    }
    coefs[tid] = coef;
  }
  __syncthreads();
  {  // row statistics: one wavefront per row
    const int lane = tid & 63, wave = tid >> 6, n_wave = blockDim.x >> 6;
    for (int r = wave; r < R; r += n_wave) {
      float ss = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int c = lane + 64 * k;
        const float x = c < d ? sq[r * d + c] : 0.0f;
        ss = fmaf(x, x, ss);
        s1 = fmaf(x, cs1[k], s1);
        s2 = fmaf(x, cs2[k], s2);
      }
      ss = wave_sum_dpp(ss); s1 = wave_sum_dpp(s1); s2 = wave_sum_dpp(s2);
      if (lane == 0) {
        const float nq = sqrtf(ss), k = sm_scale * 1.4426950408889634f;
        // bound < 2^e: e = exponent field - 126 (the mantissa of frexp is below 1), kept within
        // +-100 (a zero, denormal or huge bound only has to stay finite)
        const int e1 = min(max((int)((__float_as_uint(fabsf(k) * nq * cmax) >> 23) & 255u) - 126, -100), 100);
        const int e2 = min(max((int)((__float_as_uint(2.0f * fabsf(k * ly.qjl_scale) * nq * ly.S_rownorm_max) >> 23) & 255u) - 126, -100), 100);
        stat[r * 4 + 0] = k * __uint_as_float((uint32_t)(127 - e1) << 23);                       // multiplier of coef q_rot_j
        stat[r * 4 + 1] = 2.0f * k * ly.qjl_scale * __uint_as_float((uint32_t)(127 - e2) << 23); // multiplier of q_sk_j
        if (word == 0) {
          q_stat[(row0 + r) * 4 + 0] = (float)e1; q_stat[(row0 + r) * 4 + 1] = (float)e2;
          q_stat[(row0 + r) * 4 + 2] = k * ly.term_const * s1; q_stat[(row0 + r) * 4 + 3] = -k * ly.qjl_scale * s2;
        }
      }
    }
  }
  // contraction over this thread's PER matrix rows
  {
    const int i0 = sl * PER;
    float a[ROT_MAX_ROWS], b[ROT_MAX_ROWS];
#pragma unroll
    for (int r = 0; r < ROT_MAX_ROWS; ++r) a[r] = b[r] = 0.0f;
#pragma unroll
    for (int r = 0; r < ROT_MAX_ROWS; ++r) {
      if (r < R) {
#pragma unroll
        for (int k4 = 0; k4 < PER / 4; ++k4) {
          const float4 x = *(const float4*)(sq + r * d + i0 + 4 * k4);
          const float xs[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            a[r] = fmaf(xs[k], mp[4 * k4 + k], a[r]);
            b[r] = fmaf(xs[k], ms[4 * k4 + k], b[r]);
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < ROT_MAX_ROWS; ++r) {
      if (r < R) {
        pa[(sl * RG + r) * PREP_COLS + jl] = a[r];
        pb[(sl * RG + r) * PREP_COLS + jl] = b[r];
      }
    }
  }
  __syncthreads();
  for (int o2 = tid; o2 < 2 * R * PREP_COLS; o2 += blockDim.x) {      // first half: rotation, second: sketch
    const bool sk = o2 >= R * PREP_COLS;
    const int o = sk ? o2 - R * PREP_COLS : o2, r = o / PREP_COLS, c = o - r * PREP_COLS;
    const float* part = sk ? pb : pa;
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < PREP_SLICES; ++k) acc += part[(k * RG + r) * PREP_COLS + c];
    (sk ? ssk : srot)[o] = acc;
    (sk ? q_sk : q_rot)[(row0 + r) * d + word * PREP_COLS + c] = acc;
  }
  __syncthreads();
  // Operands of this plane word: one lane per (term plane, head) turns the 32 values of its row block into
  // the four fp6 terms with the packing conversion of gfx950 (v_cvt_scalef32_2xpk16_fp6_f32: 32 floats ->
  // 32 six-bit codes in six dwords, round to nearest even, saturating - the grid and rounding of round_fp6,
  // except that a small negative value keeps its sign on the zero code, which adds nothing in the MFMA) and
  // gets the rounded values back for the residual with its inverse (v_cvt_scalef32_pk32_f32_fp6).
  // Code j of a conversion comes from element j / 2 of its first (j even) or second (j odd) operand.
  // Lane (term plane, row g) belongs to head g % G of the workgroup's group g / G.  The operand rows of the heads
  // a group does not have are zero, as far as the page kernel reads them (head_rows: 4 or 8): with one group per
  // workgroup the lanes beyond its heads write them (lane g the rows of head g), with several groups the lane of
  // head h writes those of h + G, h + 2 G, ... below head_rows.
  if (tid < ntp * 8 && ((tid & 7) < R || ((!PACKED || gpw == 1) && (tid & 7) < head_rows))) {
    typedef float f32x16_t __attribute__((ext_vector_type(16)));
    typedef float f32x32_t __attribute__((ext_vector_type(32)));
    typedef uint32_t u32x6_t __attribute__((ext_vector_type(6)));
    const int tp = tid >> 3, g = tid & 7;
    const bool is_sign = tp == ntp - 1, live = g < R;
    const int gi = PACKED && live ? g / G : 0, hg = g - gi * G;      // (not live: head g of the workgroup's only group)
    const int gs = live ? g : 0;
    // the decode kernel extracts three of the four bits of a nibble in place, where they are the fp4
    // numbers 1, 2 and 4 (after its block scale): the query side divides them out
    const float base = live ? 4.0f * (is_sign ? stat[gs * 4 + 1] : coefs[tp] * stat[gs * 4 + 0]) : 0.0f;
    const float4* src = (const float4*)((is_sign ? ssk : srot) + gs * PREP_COLS);
    float x[PREP_COLS];
#pragma unroll
    for (int k = 0; k < PREP_COLS / 4; ++k) {
      const float4 v4 = src[k];
      x[4 * k] = v4.x; x[4 * k + 1] = v4.y; x[4 * k + 2] = v4.z; x[4 * k + 3] = v4.w;
    }
    f32x16_t va, vb;                      // contraction indices 0, 2, 4, ... and 1, 3, 5, ...
#pragma unroll
    for (int kloc = 0; kloc < 32; ++kloc) {
      const int c = 4 * (kloc & 7) + (kloc >> 3), t4 = kloc >> 3;      // coordinate within the word
      const float v = x[c] * (base * (t4 == 1 ? 0.5f : (t4 == 2 ? 0.25f : 1.0f)));
      if (kloc & 1) vb[kloc >> 1] = v;
      else va[kloc >> 1] = v;
    }
    const int i = word >> 2, kw = word & 3;
    uint32_t* dst = qa_pack + (group0 + gi) * (int64_t)(ntp * wpl * 2 * 64 * 8);
    const float one = 1.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      u32x6_t code;
      // (inline assembly with early-clobber results: the conversions read their sources over several passes)
      asm volatile("v_cvt_scalef32_2xpk16_fp6_f32 %0, %1, %2, %3" : "=&v"(code) : "v"(va), "v"(vb), "v"(one));
      uint32_t* o = dst + (((tp * wpl + i) * 2 + (t >> 1)) * 64 + 2 * hg + (t & 1) + 16 * kw) * 8;
      // (whole 32-byte slots, the two unused dwords included: full sectors reach memory without a merge)
      *(uint4*)o = make_uint4(code[0], code[1], code[2], code[3]);
      *(uint4*)(o + 4) = make_uint4(code[4], code[5], 0u, 0u);
      for (int ha = hg + G; PACKED && gpw > 1 && ha < head_rows; ha += G) {   // heads the group does not have
        uint32_t* z = o + (2 * (ha - hg)) * 8;
        *(uint4*)z = make_uint4(0u, 0u, 0u, 0u);
        *(uint4*)(z + 4) = make_uint4(0u, 0u, 0u, 0u);
      }
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

// Stores / loads that are coherent across the whole device on their own (agent-scope atomics: they go
// through the per-XCD L2 to the memory side), so that handing data from one workgroup to another needs no
// cache write-back or invalidation, which cost tens of microseconds when hundreds of wavefronts issue them.
__device__ __forceinline__ void store_coherent(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_coherent(float* p, float v) {
  __hip_atomic_store((uint32_t*)p, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// two floats at an 8-byte aligned address, as one 64-bit store
__device__ __forceinline__ void store_coherent2(float* p, float __attribute__((ext_vector_type(2))) v) {
  __hip_atomic_store((unsigned long long*)p, __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t load_coherent(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float* p) {
  return __uint_as_float(__hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ unsigned long long load_coherent(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Prefetch workgroup p of a preparation launch (see PagePrefetch): reads, and discards, the pages that one
// page-kernel workgroup will ask for first.  Workgroups go to the card's dies in turn, so the page-kernel
// workgroup picked is the one whose position in its grid is congruent to this workgroup's position in this
// grid: when the counts are multiples of eight the reader and the prefetcher share a die and its L2.
template <int THREADS>
__device__ __forceinline__ void prefetch_pages_body(const PagePrefetch& P, int p) {
  int lin = p + P.front;
  lin -= lin >= P.n_wg ? (lin / P.n_wg) * P.n_wg : 0;
  int split = lin % P.gx;
  const int rest = lin / P.gx;
  int h = rest % P.groups, b = rest / P.groups;
  if (P.kv_div > 1) {                                 // the groups of a KV head read the same pages: the first one's twin fetches
    const int kv_heads = P.groups / P.kv_div;
    if (h >= kv_heads) return;
  }
  if (P.skew16 > 0) {
    const int late = b >= P.n_seq;
    b -= late ? P.n_seq : 0;
    split = 2 * split + late;
  }
  int seq_len = P.seq_lens[b];
  seq_len = (seq_len < P.max_pages * TQ_PAGE_TOKENS ? seq_len : P.max_pages * TQ_PAGE_TOKENS) - P.len_sub;
  seq_len = seq_len > 0 ? seq_len : 0;
  const int n_pages = (seq_len + TQ_PAGE_TOKENS - 1) / TQ_PAGE_TOKENS;
  int blk_begin, blk_end;
  decode_block_range(seq_len, P.n_split, split, P.skew16, P.ngrp, blk_begin, blk_end);
  const int blk_stop = blk_begin + P.blocks < blk_end ? blk_begin + P.blocks : blk_end;
  const int pg0 = 4 * blk_begin, pg1 = 4 * blk_stop < n_pages ? 4 * blk_stop : n_pages;
  const int32_t* bt = P.block_table + (int64_t)b * P.bt_stride;
  const uint8_t* base = P.pool + (uint64_t)h * P.page_bytes;
  // 16 bytes per lane; piece i of the range = piece i % pieces of page i / pieces.  Every table load is issued
  // before the first page load and every page load before anything waits: the workgroup costs two memory
  // latencies, whatever its share.  Slots beyond the range re-read the head's page 0 (in the pool, cached).
  constexpr int SLOTS = 6144 / THREADS;                // 16-byte pieces per lane: 96 KB per workgroup
  const int tid = threadIdx.x, pieces = (int)(P.fetch_bytes >> 4), total = (pg1 > pg0 ? pg1 - pg0 : 0) * pieces;
  if (total <= 0) return;
  const float inv_pieces = 1.0f / (float)pieces;
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  uint32_t pid[SLOTS], off[SLOTS];
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    const int i = tid + THREADS * k;
    const int pg = (int)(((float)i + 0.5f) * inv_pieces);       // exact for the few thousand pieces of a range
    const bool live = i < total;
    off[k] = live ? (uint32_t)(i - pg * pieces) * 16u : 0u;
    pid[k] = (uint32_t)bt[live ? pg0 + pg : pg0];              // (unconditional: a load under a branch would be waited for)
  }
  u32x4_t keep = {0u, 0u, 0u, 0u}, got[SLOTS];
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) {
    const uint32_t page = pid[k] < (uint32_t)P.num_pages ? pid[k] : 0u;
    got[k] = *(const u32x4_t*)(base + (uint64_t)page * P.page_stride + off[k]);
  }
#pragma unroll
  for (int k = 0; k < SLOTS; ++k) keep ^= got[k];
  asm volatile("" :: "v"(keep));                      // the loads are wanted for their side effect
}

// ------------------------------------------------------------------------------------------------------
// The same preparation on the matrix cores, for bf16 queries at head_dim 128 / 256: q Pi^T and q S^T are
// (rows x d) x (d x d) products, a bf16 query is an exact single term, and Pi and S already exist as three
// bf16 terms each in MFMA operand order (tq_layer::Pi_split / S_split, built for the key quantiser), so
// v_mfma_f32_16x16x32_bf16 gives the fp32-accurate products with the matrix as the row operand and sixteen
// query rows as the column operand.  A workgroup of four wavefronts owns a tile of up to 16 rows - as many whole
// groups of G heads as fit - and one plane word (32 coordinates); each wavefront owns one of the word's two
// 16-coordinate halves of one of the two products: d / 32 x 3 MFMAs whose matrix operands are all requested before
// the first is used (one memory latency).  The 16 x 32 results meet in LDS and one lane per (term plane, row) packs
// the four fp6 terms exactly as prep_query_body does.  Nothing is read from another workgroup.
// WW (large preparations): a workgroup owns a tile and ALL its plane words - wavefront w takes words w, w + 4, ...,
// computes the four 16 x 16 pieces of a word (two halves x two products) one after the other and packs the word
// itself, so the launch has a quarter (head_dim 128) or an eighth (256) of the workgroups, all four wavefronts pack
// instead of one, and nothing waits for another wavefront.  The operands are the same bits either way.
typedef uint32_t prep_u32x4 __attribute__((ext_vector_type(4)));
typedef float prep_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 prep_bf16x8 __attribute__((ext_vector_type(8)));
constexpr int PREP_MFMA_THREADS = 256, PREP_MFMA_LD = 36;          // LDS row stride of a wavefront's 16 x 32 tile

constexpr int ROT_COLS = 32;          // output columns (one plane word) of a rotation workgroup

// coefficient of term plane tp as the wide-head page kernel orders them: the index planes from the highest bit down,
// the multi-bit Walsh terms, the sign plane
__device__ __forceinline__ float wide_term_plane_coef(const tq_layer& ly, int ntp, int tp) {
  const int mb = ly.mse_bits;
  float coef = 1.0f;                               // the sign plane
  if (tp < mb) {
    coef = 0.0f;
    for (int t = 0; t < ly.n_terms; ++t)
      if (ly.term_mask[t] == (1 << (mb - 1 - tp))) coef = ly.term_coef[t];
  } else if (tp < ntp - 1) {
    coef = 0.0f;
    int seen = 0;
    for (int t = 0; t < ly.n_terms; ++t) {
      if (__builtin_popcount(ly.term_mask[t]) > 1) {
        if (seen == tp - mb) coef = ly.term_coef[t];
        ++seen;
      }
    }
  }
  return coef;
}

// PACK epilogue of the rotation kernels: plane word j (32 coordinates) of nr query rows from row0 on, as the wide-head
// page kernel's fp6 operands.  s_rot / s_sk: [row][32] rotated / sketched values of the word; s_rs: [row][2] the
// rows' multipliers; s_cf: coefficient of each term plane.
__device__ __forceinline__ void wide_pack_word(const WidePack& wp, int d, int nr, int row0, int j, const float* s_rot,
                                               const float* s_sk, const float* s_rs, const float* s_cf, int tid,
                                               int n_threads, int tp_begin, int tp_end) {
  // one lane per (term plane, row): the word's 32 values as four fp6 terms (the packing conversion of gfx950 and its
  // inverse for the residual), written where lane (row 2 g + term % 2, quarter word % 4) of operand (plane, row set
  // term / 2, chunk word / 4) of the row's head group reads them
  typedef float f32x16_t __attribute__((ext_vector_type(16)));
  typedef float f32x32_t __attribute__((ext_vector_type(32)));
  typedef uint32_t u32x6_t __attribute__((ext_vector_type(6)));
  const int ntp = wp.ntp;
  const int qa_stride = wide_qa_stride(d);
  const bool half_op = (d & 127) != 0 && (j >> 2) == ((d + 127) >> 7) - 1;
  const int hi_at = half_op ? 32 * 4 : 64 * 4;
  for (int it = tp_begin * nr + tid; it < tp_end * nr; it += n_threads) {      // (term planes tp_begin .. tp_end - 1)
    const int tp = it / nr, r = it - tp * nr;
    const bool is_sign = tp == ntp - 1;
    // the row's place: sequence, head, group of at most 8 heads of its KV head, slot in the group
    const int row = row0 + r;                        // (32-bit arithmetic: the launcher checks the row count)
    const int bq = row / wp.Hq, head = row - bq * wp.Hq;
    const int g_tot = wp.Hq / wp.Hkv, kvh = head / g_tot, hh = head - kvh * g_tot;
    const int g_max = (g_tot + wp.kv_div - 1) / wp.kv_div, grp = hh / g_max, g = hh - grp * g_max;
    const int64_t group = ((int64_t)bq * wp.Hkv + kvh) * wp.kv_div + grp;
    const float base = 4.0f * (is_sign ? s_rs[2 * r + 1] : s_cf[tp] * s_rs[2 * r]);
    const float4* src = (const float4*)((is_sign ? s_sk : s_rot) + r * ROT_COLS);
    float x[32];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float4 v4 = src[k];
      x[4 * k] = v4.x; x[4 * k + 1] = v4.y; x[4 * k + 2] = v4.z; x[4 * k + 3] = v4.w;
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
    uint32_t* op0 = wp.qa + group * (int64_t)(ntp * 2 * qa_stride) + (tp * 2) * qa_stride + (j >> 2) * WD_QA_OP;
    const int slot0 = 2 * g + 16 * (j & 3);
    const float one = 1.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      u32x6_t code;
      asm volatile("v_cvt_scalef32_2xpk16_fp6_f32 %0, %1, %2, %3" : "=&v"(code) : "v"(va), "v"(vb), "v"(one));
      uint32_t* op = op0 + (t >> 1) * qa_stride;
      *(uint4*)(op + (slot0 + (t & 1)) * 4) = make_uint4(code[0], code[1], code[2], code[3]);
      *(uint2*)(op + hi_at + (slot0 + (t & 1)) * 2) = make_uint2(code[4], code[5]);
      if (t < 3) {
        f32x32_t rr;
        asm volatile("v_cvt_scalef32_pk32_f32_fp6 %0, %1, %2" : "=&v"(rr) : "v"(code), "v"(one));
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          va[k] = (va[k] - rr[2 * k]) * 32.0f;
          vb[k] = (vb[k] - rr[2 * k + 1]) * 32.0f;
        }
      }
    }
  }
}

// The rotation with the PACK epilogue on the matrix cores, for bf16 queries and the split matrices of the layer
// (tq_layer::Pi_split / S_split: three bf16 terms in MFMA operand order; a bf16 query is an exact single term, so
// v_mfma_f32_16x16x32_bf16 gives fp32-accurate products).  A workgroup of four wavefronts owns sixteen consecutive
// query rows, one plane word (32 coordinates) and one of the two products (0: q Pi^T, whose values fill the
// index and term planes of the operands; 1: q S^T, the sign plane) - a compute unit moves 64 bytes per cycle, and the
// matrix terms of both products in one workgroup made the second half of its wavefronts wait 2 us for the first.
// Wavefront (half word jt, contraction half kh) runs KPW = d / 64 contraction steps x 3 terms with the matrix as the
// row operand and the queries as the column operand.  Everything a wavefront needs is requested up front - its
// queries, a share of the column sums for the row statistics, then the matrix terms - so the statistics are summed
// while the terms are on their way: one memory latency in all.  The halves meet in LDS, then the packing.
constexpr int ROTM_THREADS = 256, ROTM_LD = 36;
__host__ __device__ inline int rotate_mfma_smem_floats() {
  return 2 * 16 * ROTM_LD + 4 * 16 * 2 + 16 * ROT_COLS + 2 * 16 + 16;
}

// (id: the workgroup's place among the launch's rotation workgroups; the first ROTM_THREADS threads of a workgroup)
// F16Q: fp16 queries - a value of 11 significant bits is the exact sum of two bf16 terms (the rounded value and the
// remainder), so every matrix term meets two query operands instead of one.
template <int KPW, bool F16Q = false>
__device__ __forceinline__ void rotate_mfma_body(const uint16_t* __restrict__ q, int64_t rows, int n_tiles, const tq_layer& ly,
                                                 float* __restrict__ q_rot, float* __restrict__ q_sk, const WidePack& wp,
                                                 int id, float* sm) {
  constexpr int KS = 2 * KPW, D = 32 * KS;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, kb = lane >> 4;
  const int jt = wave & 1, kh = wave >> 1;
  // Workgroup -> (plane word, product, row tile): workgroups go to the card's eight dies in turn, each die with an L2
  // of its own, so the (word, product) pairs are dealt to the dies - pair p to die p % 8 - and all row tiles of a
  // pair run on its die: the matrix terms are fetched into one L2, not into all eight.
  const int pair = (id & 7) + 8 * ((id >> 3) / n_tiles);
  if (pair >= 2 * KS) return;                        // (the pairs do not divide among eight dies)
  const int word = pair >> 1, m = pair & 1;
  const int64_t row0 = (int64_t)((id >> 3) % n_tiles) * 16;
  const int nr = (int)(rows - row0 < 16 ? rows - row0 : 16);
  float* part = sm;                                  // [kh][16 rows][ROTM_LD]
  float* s_st = part + 2 * 16 * ROTM_LD;             // [4 wavefronts][16 rows][2] partial statistics
  float* s_val = s_st + 4 * 16 * 2;                  // [16][32] the word's rotated (sketched) values
  float* s_rs = s_val + 16 * ROT_COLS;               // [16][2] multipliers of q_rot / q_sk (this product's is set)
  float* s_cf = s_rs + 2 * 16;                       // [16] coefficient of each term plane
  // column operands: lane (row n, block kb) holds q[n][32 ks + 8 kb .. + 7]; rows beyond the last are zero
  const uint16_t* qrow = q + (row0 + (n < nr ? n : nr - 1)) * D + kb * 8;
  prep_u32x4 qb[KPW];
#pragma unroll
  for (int k = 0; k < KPW; ++k) qb[k] = *(const prep_u32x4*)(qrow + (kh * KPW + k) * 32);
  // this wavefront's share of the statistics: steps jt, jt + 2, ... of its contraction half
  constexpr int NS = (KPW + 1) / 2;
  const float* colsum = m ? ly.S_colsum : ly.Pi_colsum;
  prep_u32x4 xq[NS];
  prep_f32x4 cs[NS][2];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int kl = jt + 2 * i < KPW ? jt + 2 * i : 0;                  // (a step that does not exist counts for nothing)
    const int ks = kh * KPW + kl;
    xq[i] = *(const prep_u32x4*)(qrow + ks * 32);
    cs[i][0] = *(const prep_f32x4*)(colsum + ks * 32 + kb * 8);
    cs[i][1] = *(const prep_f32x4*)(colsum + ks * 32 + kb * 8 + 4);
  }
  // row operands: the three bf16 terms of 16 matrix rows
  prep_u32x4 ma[3][KPW];
  {
    const uint16_t* mat = m ? ly.S_split : ly.Pi_split;
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      const uint16_t* base = mat + (((int64_t)(t * (D / 16) + word * 2 + jt) * KS + kh * KPW) * 64 + lane) * 8;
#pragma unroll
      for (int k = 0; k < KPW; ++k) ma[t][k] = *(const prep_u32x4*)(base + k * (64 * 8));
    }
  }
  {
    float ss = 0.0f, s1 = 0.0f;
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const bool real = jt + 2 * i < KPW && n < nr;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float xl = real ? (F16Q ? f16_bits_to_f32((uint16_t)(xq[i][e] & 0xffffu)) : __uint_as_float(xq[i][e] << 16)) : 0.0f;
        const float xh = real ? (F16Q ? f16_bits_to_f32((uint16_t)(xq[i][e] >> 16)) : __uint_as_float(xq[i][e] & 0xffff0000u)) : 0.0f;
        ss = fmaf(xl, xl, fmaf(xh, xh, ss));
        s1 = fmaf(xl, cs[i][e >> 1][2 * (e & 1)], fmaf(xh, cs[i][e >> 1][2 * (e & 1) + 1], s1));
      }
    }
    ss += __shfl_xor(ss, 16, 64); s1 += __shfl_xor(s1, 16, 64);
    ss += __shfl_xor(ss, 32, 64); s1 += __shfl_xor(s1, 32, 64);
    if (kb == 0) *(float2*)(s_st + (wave * 16 + n) * 2) = make_float2(ss, s1);
  }
  if (n >= nr) {
#pragma unroll
    for (int k = 0; k < KPW; ++k) qb[k] = prep_u32x4{0u, 0u, 0u, 0u};
  }
  prep_u32x4 ql[F16Q ? KPW : 1];                                       // fp16 queries: qb becomes the rounded values, ql the remainders
  if constexpr (F16Q) {
#pragma unroll
    for (int k = 0; k < KPW; ++k) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // (the packed conversion rounds to nearest even; the remainders have at most four significant bits: exact)
        typedef float rot_f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 rot_bf16x2 __attribute__((ext_vector_type(2)));
        const rot_f32x2 x = {f16_bits_to_f32((uint16_t)(qb[k][e] & 0xffffu)), f16_bits_to_f32((uint16_t)(qb[k][e] >> 16))};
        const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, rot_bf16x2));
        const rot_f32x2 rem = {x[0] - __uint_as_float(hi << 16), x[1] - __uint_as_float(hi & 0xffff0000u)};
        qb[k][e] = hi;
        ql[k][e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rem, rot_bf16x2));
      }
    }
  }
  prep_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int t = 2; t >= 0; --t) {                                       // the small terms first
    if constexpr (F16Q) {
#pragma unroll
      for (int k = 0; k < KPW; ++k)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(prep_bf16x8, ma[t][k]),
                                                      __builtin_bit_cast(prep_bf16x8, ql[k]), acc, 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < KPW; ++k)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(prep_bf16x8, ma[t][k]),
                                                    __builtin_bit_cast(prep_bf16x8, qb[k]), acc, 0, 0, 0);
  }
  // result register i of lane (row n, quarter kb) is coordinate 16 jt + 4 kb + i of query row n
  *(prep_f32x4*)(part + (kh * 16 + n) * ROTM_LD + jt * 16 + 4 * kb) = acc;
  __syncthreads();
  float* dst = m ? q_sk : q_rot;
#pragma unroll
  for (int o = tid; o < 16 * ROT_COLS; o += ROTM_THREADS) {            // a (row, coordinate) of the word
    const int r = o >> 5, c = o & 31;
    const float v = part[r * ROTM_LD + c] + part[(16 + r) * ROTM_LD + c];
    s_val[o] = v;
    if (r < nr) dst[(row0 + r) * D + word * ROT_COLS + c] = v;
  }
  if (tid < 16) {                                                      // the statistics of row tid
    const int r = tid;
    float ss = 0.0f, s1 = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float2 p = *(const float2*)(s_st + (w * 16 + r) * 2);
      ss += p.x; s1 += p.y;
    }
    const float nq = sqrtf(ss), k = wp.sm_scale * 1.4426950408889634f;
    float* st = wp.q_stat + (row0 + r) * 4;
    // bound < 2^e: e = exponent field - 126, kept within +-100
    if (m == 0) {
      float cmax = 0.0f;
      for (int t = 0; t < ly.n_terms; ++t) cmax = fmaxf(cmax, fabsf(ly.term_coef[t]));
      const int e1 = min(max((int)((__float_as_uint(fabsf(k) * nq * cmax) >> 23) & 255u) - 126, -100), 100);
      s_rs[2 * r] = k * __uint_as_float((uint32_t)(127 - e1) << 23);
      if (word == 0 && r < nr) { st[0] = (float)e1; st[2] = k * ly.term_const * s1; }
    } else {
      const int e2 = min(max((int)((__float_as_uint(2.0f * fabsf(k * ly.qjl_scale) * nq * ly.S_rownorm_max) >> 23) & 255u) - 126, -100), 100);
      s_rs[2 * r + 1] = 2.0f * k * ly.qjl_scale * __uint_as_float((uint32_t)(127 - e2) << 23);
      if (word == 0 && r < nr) { st[1] = (float)e2; st[3] = -k * ly.qjl_scale * s1; }
    }
  } else if (tid >= 64 && tid < 80) {
    s_cf[tid - 64] = wide_term_plane_coef(ly, wp.ntp, tid - 64);
  }
  __syncthreads();
  // the index and term planes from the rotated values, the sign plane from the sketched ones
  wide_pack_word(wp, D, nr, (int)row0, word, s_val, s_val, s_rs, s_cf, tid, ROTM_THREADS, m ? wp.ntp - 1 : 0,
                 m ? wp.ntp : wp.ntp - 1);
}

// The same rotation for thousands of rows (more workgroups than the card holds at once): a workgroup takes `tpw`
// consecutive row tiles of its (plane word, product) pair against ONE fetch of the matrix terms and column sums
// (2048 rows at head_dim 576 as a workgroup per tile pulled 560 MB of terms through the L2s: 61 us, now 46).  First every tile's
// products, sums and statistics - the matrix terms stay in registers, the halves meet in LDS buffers that alternate
// by tile, the results wait in LDS -, then the packing of all tiles, which needs the registers the terms held.
constexpr int ROTM_MAX_TPW = 16;
__host__ __device__ inline int rotate_mfma_tiles_smem_floats(int tpw) {
  return 2 * (2 * 16 * ROTM_LD + 4 * 16 * 2) + tpw * (16 * ROT_COLS + 2 * 16) + 16;
}

template <int KPW>
__device__ __forceinline__ void rotate_mfma_tiles_body(const uint16_t* __restrict__ q, int64_t rows, int n_tiles, int tpw,
                                                       const tq_layer& ly, float* __restrict__ q_rot,
                                                       float* __restrict__ q_sk, const WidePack& wp, int id, float* sm) {
  constexpr int KS = 2 * KPW, D = 32 * KS;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, kb = lane >> 4;
  const int jt = wave & 1, kh = wave >> 1;
  const int n_tg = (n_tiles + tpw - 1) / tpw;
  const int pair = (id & 7) + 8 * ((id >> 3) / n_tg);              // (pair p on die p % 8, as in rotate_mfma_body)
  if (pair >= 2 * KS) return;
  const int word = pair >> 1, m = pair & 1;
  const int tile0 = ((id >> 3) % n_tg) * tpw, tile1 = min(tile0 + tpw, n_tiles);
  float* part = sm;                                  // [2 buffers][kh][16 rows][ROTM_LD]
  float* s_st = part + 2 * 2 * 16 * ROTM_LD;         // [2 buffers][4 wavefronts][16 rows][2]
  float* s_val = s_st + 2 * 4 * 16 * 2;              // [tpw][16][32]
  float* s_rs = s_val + tpw * 16 * ROT_COLS;         // [tpw][16][2]
  float* s_cf = s_rs + tpw * 2 * 16;                 // [16]
  constexpr int NS = (KPW + 1) / 2;
  const float* colsum = m ? ly.S_colsum : ly.Pi_colsum;
  prep_f32x4 cs[NS][2];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int kl = jt + 2 * i < KPW ? jt + 2 * i : 0;
    const int ks = kh * KPW + kl;
    cs[i][0] = *(const prep_f32x4*)(colsum + ks * 32 + kb * 8);
    cs[i][1] = *(const prep_f32x4*)(colsum + ks * 32 + kb * 8 + 4);
  }
  prep_u32x4 ma[3][KPW];
  {
    const uint16_t* mat = m ? ly.S_split : ly.Pi_split;
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      const uint16_t* base = mat + (((int64_t)(t * (D / 16) + word * 2 + jt) * KS + kh * KPW) * 64 + lane) * 8;
#pragma unroll
      for (int k = 0; k < KPW; ++k) ma[t][k] = *(const prep_u32x4*)(base + k * (64 * 8));
    }
  }
  if (tid >= 64 && tid < 80) s_cf[tid - 64] = wide_term_plane_coef(ly, wp.ntp, tid - 64);
  float cmax = 0.0f;
  for (int t = 0; t < ly.n_terms; ++t) cmax = fmaxf(cmax, fabsf(ly.term_coef[t]));
  float* dst = m ? q_sk : q_rot;
#pragma unroll 1
  for (int tile = tile0; tile < tile1; ++tile) {
    const int buf = (tile - tile0) & 1, ti = tile - tile0;
    const int64_t row0 = (int64_t)tile * 16;
    const int nr = (int)(rows - row0 < 16 ? rows - row0 : 16);
    const uint16_t* qrow = q + (row0 + (n < nr ? n : nr - 1)) * D + kb * 8;
    prep_u32x4 qb[KPW];
#pragma unroll
    for (int k = 0; k < KPW; ++k) qb[k] = *(const prep_u32x4*)(qrow + (kh * KPW + k) * 32);
    if (n >= nr) {
#pragma unroll
      for (int k = 0; k < KPW; ++k) qb[k] = prep_u32x4{0u, 0u, 0u, 0u};
    }
    {  // this wavefront's share of the statistics: steps jt, jt + 2, ... of its contraction half
      float ss = 0.0f, s1 = 0.0f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const bool real = jt + 2 * i < KPW;
        // (step 2 i + jt of the operand registers, picked with masks: an index that depends on the wavefront would
        // move the registers to scratch memory)
        const uint32_t odd = jt ? 0xffffffffu : 0u;
        const int KO = 2 * i + 1 < KPW ? 2 * i + 1 : 2 * i;      // (a constant once the loop is unrolled)
        prep_u32x4 x4;
#pragma unroll
        for (int e = 0; e < 4; ++e) x4[e] = (qb[KO][e] & odd) | (qb[2 * i][e] & ~odd);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float xl = real ? __uint_as_float(x4[e] << 16) : 0.0f;
          const float xh = real ? __uint_as_float(x4[e] & 0xffff0000u) : 0.0f;
          ss = fmaf(xl, xl, fmaf(xh, xh, ss));
          s1 = fmaf(xl, cs[i][e >> 1][2 * (e & 1)], fmaf(xh, cs[i][e >> 1][2 * (e & 1) + 1], s1));
        }
      }
      ss += __shfl_xor(ss, 16, 64); s1 += __shfl_xor(s1, 16, 64);
      ss += __shfl_xor(ss, 32, 64); s1 += __shfl_xor(s1, 32, 64);
      if (kb == 0) *(float2*)(s_st + ((buf * 4 + wave) * 16 + n) * 2) = make_float2(ss, s1);
    }
    prep_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 2; t >= 0; --t)
#pragma unroll
      for (int k = 0; k < KPW; ++k)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(prep_bf16x8, ma[t][k]),
                                                      __builtin_bit_cast(prep_bf16x8, qb[k]), acc, 0, 0, 0);
    *(prep_f32x4*)(part + ((buf * 2 + kh) * 16 + n) * ROTM_LD + jt * 16 + 4 * kb) = acc;
    // (one barrier per tile: the buffers alternate, and a thread two tiles ahead has passed the barrier of the tile
    // between, which every reader of this buffer reaches only after its reads)
    __syncthreads();
#pragma unroll
    for (int o = tid; o < 16 * ROT_COLS; o += ROTM_THREADS) {
      const int r = o >> 5, c = o & 31;
      const float v = part[((buf * 2) * 16 + r) * ROTM_LD + c] + part[((buf * 2 + 1) * 16 + r) * ROTM_LD + c];
      s_val[ti * 16 * ROT_COLS + o] = v;
      if (r < nr) dst[(row0 + r) * D + word * ROT_COLS + c] = v;
    }
    if (tid < 16) {
      const int r = tid;
      float ss = 0.0f, s1 = 0.0f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float2 p = *(const float2*)(s_st + ((buf * 4 + w) * 16 + r) * 2);
        ss += p.x; s1 += p.y;
      }
      const float nq = sqrtf(ss), k = wp.sm_scale * 1.4426950408889634f;
      float* st = wp.q_stat + (row0 + r) * 4;
      if (m == 0) {
        const int e1 = min(max((int)((__float_as_uint(fabsf(k) * nq * cmax) >> 23) & 255u) - 126, -100), 100);
        s_rs[ti * 32 + 2 * r] = k * __uint_as_float((uint32_t)(127 - e1) << 23);
        if (word == 0 && r < nr) { st[0] = (float)e1; st[2] = k * ly.term_const * s1; }
      } else {
        const int e2 = min(max((int)((__float_as_uint(2.0f * fabsf(k * ly.qjl_scale) * nq * ly.S_rownorm_max) >> 23) & 255u) - 126, -100), 100);
        s_rs[ti * 32 + 2 * r + 1] = 2.0f * k * ly.qjl_scale * __uint_as_float((uint32_t)(127 - e2) << 23);
        if (word == 0 && r < nr) { st[1] = (float)e2; st[3] = -k * ly.qjl_scale * s1; }
      }
    }
  }
  __syncthreads();
#pragma unroll 1
  for (int tile = tile0; tile < tile1; ++tile) {
    const int ti = tile - tile0;
    const int64_t row0 = (int64_t)tile * 16;
    const int nr = (int)(rows - row0 < 16 ? rows - row0 : 16);
    wide_pack_word(wp, D, nr, (int)row0, word, s_val + ti * 16 * ROT_COLS, s_val + ti * 16 * ROT_COLS, s_rs + ti * 32, s_cf, tid,
                   ROTM_THREADS, m ? wp.ntp - 1 : 0, m ? wp.ntp : wp.ntp - 1);
  }
}

__host__ __device__ inline int prep_mfma_smem_floats() { return 2 * 16 * PREP_MFMA_LD + 32; }

template <int D, bool WW>
__device__ __forceinline__ void prep_mfma_body(const uint16_t* __restrict__ q, int G, int64_t n_rows, const tq_layer& ly,
                                               float sm_scale, float* __restrict__ q_stat, uint32_t* __restrict__ qa_pack,
                                               unsigned long long* __restrict__ arrivals, int head_rows, int64_t tile,
                                               int word_of_wg, float* sm) {
  constexpr int KS = D / 32;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, kb = lane >> 4;
  const int gpt = 16 / G, rows_tile = gpt * G;                     // whole groups per tile
  const int64_t row0 = tile * rows_tile, group0 = tile * gpt;
  const int R = (int)(n_rows - row0 < rows_tile ? n_rows - row0 : rows_tile);
  if (arrivals != nullptr && (WW || word_of_wg == 0) && tid < gpt && tid * G < R) arrivals[group0 + tid] = 0ull;
  // (WW: a region per wavefront)
  float* s_rot = sm + (WW ? wave * prep_mfma_smem_floats() : 0);    // [16 rows][32 coordinates], stride PREP_MFMA_LD
  float* s_sk = s_rot + 16 * PREP_MFMA_LD;
  float* stat = s_sk + 16 * PREP_MFMA_LD;                           // [16 rows][2]: multipliers of coef q_rot_j and q_sk_j
  // column operands: lane (row n, block kb) holds q[n][32 ks + 8 kb .. + 7]; rows beyond the tile are zero
  prep_u32x4 qb[KS];
  {
    const uint16_t* qrow = q + (row0 + (n < R ? n : R - 1)) * D + kb * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qb[ks] = *(const prep_u32x4*)(qrow + ks * 32);
    if (n >= R) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qb[ks] = prep_u32x4{0u, 0u, 0u, 0u};
    }
  }
  // one 16 x 16 piece: half jt of plane word `word`, product m (0: q Pi^T, 1: q S^T).  Row operands: the three bf16
  // terms of 16 matrix rows, all requested before anything waits.
  auto piece = [&](int word, int jt, int m) __attribute__((always_inline)) {
    prep_u32x4 ma[3][KS];
    const uint16_t* mat = m ? ly.S_split : ly.Pi_split;
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      const uint16_t* base = mat + (((int64_t)(t * (D / 16) + word * 2 + jt) * KS) * 64 + lane) * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ma[t][ks] = *(const prep_u32x4*)(base + ks * (64 * 8));
    }
    prep_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 2; t >= 0; --t)                                       // the small terms first
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(prep_bf16x8, ma[t][ks]),
                                                      __builtin_bit_cast(prep_bf16x8, qb[ks]), acc, 0, 0, 0);
    // result register i of lane (row n, quarter kb) is coordinate 16 jt + 4 kb + i of query row n
    *(prep_f32x4*)((m ? s_sk : s_rot) + n * PREP_MFMA_LD + jt * 16 + 4 * kb) = acc;
  };
  // row statistics from the same registers: the four lanes of a row each hold a quarter of its coordinates
  {
    float ss = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const prep_f32x4* c1 = (const prep_f32x4*)(ly.Pi_colsum + ks * 32 + kb * 8);
      const prep_f32x4* c2 = (const prep_f32x4*)(ly.S_colsum + ks * 32 + kb * 8);
      const prep_f32x4 a0 = c1[0], a1 = c1[1], b0 = c2[0], b1 = c2[1];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float xl = __uint_as_float(qb[ks][e] << 16), xh = __uint_as_float(qb[ks][e] & 0xffff0000u);
        const float cl1 = e < 2 ? a0[2 * e] : a1[2 * e - 4], ch1 = e < 2 ? a0[2 * e + 1] : a1[2 * e - 3];
        const float cl2 = e < 2 ? b0[2 * e] : b1[2 * e - 4], ch2 = e < 2 ? b0[2 * e + 1] : b1[2 * e - 3];
        ss = fmaf(xl, xl, fmaf(xh, xh, ss));
        s1 = fmaf(xl, cl1, fmaf(xh, ch1, s1));
        s2 = fmaf(xl, cl2, fmaf(xh, ch2, s2));
      }
    }
    ss += __shfl_xor(ss, 16, 64); s1 += __shfl_xor(s1, 16, 64); s2 += __shfl_xor(s2, 16, 64);
    ss += __shfl_xor(ss, 32, 64); s1 += __shfl_xor(s1, 32, 64); s2 += __shfl_xor(s2, 32, 64);
    float cmax = 0.0f;
    for (int t = 0; t < ly.n_terms; ++t) cmax = fmaxf(cmax, fabsf(ly.term_coef[t]));
    const float nq = sqrtf(ss), k = sm_scale * 1.4426950408889634f;
    const int e1 = min(max((int)((__float_as_uint(fabsf(k) * nq * cmax) >> 23) & 255u) - 126, -100), 100);
    const int e2 = min(max((int)((__float_as_uint(2.0f * fabsf(k * ly.qjl_scale) * nq * ly.S_rownorm_max) >> 23) & 255u) - 126, -100), 100);
    if (kb == 0 && (WW || wave == 0)) {
      stat[n * 2 + 0] = k * __uint_as_float((uint32_t)(127 - e1) << 23);
      stat[n * 2 + 1] = 2.0f * k * ly.qjl_scale * __uint_as_float((uint32_t)(127 - e2) << 23);
      if ((WW ? wave == 0 : word_of_wg == 0) && n < R) {
        float* st = q_stat + (row0 + n) * 4;
        st[0] = (float)e1; st[1] = (float)e2;
        st[2] = k * ly.term_const * s1; st[3] = -k * ly.qjl_scale * s2;
      }
    }
  }
  const int mb = ly.mse_bits;
  int nx = 0;
  for (int t = 0; t < ly.n_terms; ++t)
    if (__builtin_popcount(ly.term_mask[t]) > 1) ++nx;
  const int ntp = mb + nx + 1;
  constexpr int wpl = D / 128;
  constexpr int NPASS = WW ? (D / 32) / 4 : 1;
#pragma unroll 1
  for (int pass = 0; pass < NPASS; ++pass) {
  const int word = WW ? wave + 4 * pass : word_of_wg;
  const int chunk = word >> 2, kw = word & 3;                       // the word's place in the operand layout
  if constexpr (WW) {
    // (the tile of the last word has been read by this wavefront's packing lanes)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int c = 0; c < 4; ++c) piece(word, c & 1, c >> 1);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  } else {
    piece(word, wave & 1, wave >> 1);                               // this wavefront's half of the word, and its product
    __syncthreads();
  }
  // operands of this plane word: one lane per (term plane, row), as in prep_query_body
  for (int idx = WW ? lane : tid; idx < ntp * 16; idx += WW ? 64 : PREP_MFMA_THREADS) {
    const int tp = idx >> 4, r = idx & 15;
    if (r >= R) continue;
    typedef float f32x16_t __attribute__((ext_vector_type(16)));
    typedef float f32x32_t __attribute__((ext_vector_type(32)));
    typedef uint32_t u32x6_t __attribute__((ext_vector_type(6)));
    const bool is_sign = tp == ntp - 1;
    float coef = 1.0f;
    if (tp < mb) {
      coef = 0.0f;
      for (int t = 0; t < ly.n_terms; ++t)
        if (ly.term_mask[t] == (1 << (mb - 1 - tp))) coef = ly.term_coef[t];
    } else if (!is_sign) {
      coef = 0.0f;
      int seen = 0;
      for (int t = 0; t < ly.n_terms; ++t) {
        if (__builtin_popcount(ly.term_mask[t]) > 1) {
          if (seen == tp - mb) coef = ly.term_coef[t];
          ++seen;
        }
      }
    }
    const int gi = r / G, hg = r - gi * G;
    const float base = 4.0f * (is_sign ? stat[r * 2 + 1] : coef * stat[r * 2 + 0]);
    const prep_f32x4* src = (const prep_f32x4*)((is_sign ? s_sk : s_rot) + r * PREP_MFMA_LD);
    float x[32];
#pragma unroll
    for (int k4 = 0; k4 < 8; ++k4) {
      const prep_f32x4 v4 = src[k4];
      x[4 * k4] = v4[0]; x[4 * k4 + 1] = v4[1]; x[4 * k4 + 2] = v4[2]; x[4 * k4 + 3] = v4[3];
    }
    f32x16_t va, vb;
#pragma unroll
    for (int kloc = 0; kloc < 32; ++kloc) {
      const int c = 4 * (kloc & 7) + (kloc >> 3), t4 = kloc >> 3;
      const float v = x[c] * (base * (t4 == 1 ? 0.5f : (t4 == 2 ? 0.25f : 1.0f)));
      if (kloc & 1) vb[kloc >> 1] = v;
      else va[kloc >> 1] = v;
    }
    uint32_t* dst = qa_pack + (group0 + gi) * (int64_t)(ntp * wpl * 2 * 64 * 8);
    const float one = 1.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      u32x6_t code;
      asm volatile("v_cvt_scalef32_2xpk16_fp6_f32 %0, %1, %2, %3" : "=&v"(code) : "v"(va), "v"(vb), "v"(one));
      uint32_t* o = dst + (((tp * wpl + chunk) * 2 + (t >> 1)) * 64 + 2 * hg + (t & 1) + 16 * kw) * 8;
      // (whole 32-byte slots, the two unused dwords included: full sectors reach memory without a merge)
      *(uint4*)o = make_uint4(code[0], code[1], code[2], code[3]);
      *(uint4*)(o + 4) = make_uint4(code[4], code[5], 0u, 0u);
      for (int ha = hg + G; ha < head_rows; ha += G) {               // operand rows of heads the group does not have
        uint32_t* z = o + (2 * (ha - hg)) * 8;
        *(uint4*)z = make_uint4(0u, 0u, 0u, 0u);
        *(uint4*)(z + 4) = make_uint4(0u, 0u, 0u, 0u);
      }
      if (t < 3) {
        f32x32_t rr;
        asm volatile("v_cvt_scalef32_pk32_f32_fp6 %0, %1, %2" : "=&v"(rr) : "v"(code), "v"(one));
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          va[k] = (va[k] - rr[2 * k]) * 32.0f;
          vb[k] = (vb[k] - rr[2 * k + 1]) * 32.0f;
        }
      }
    }
  }
  }
}

// LDS bytes of a preparation workgroup
static inline size_t prep_smem_bytes(int RG, int d) {       // RG: query rows of a workgroup
  return (size_t)(RG * d + 2 * PREP_SLICES * RG * PREP_COLS + 2 * RG * PREP_COLS + 4 * ROT_MAX_ROWS + 32) * sizeof(float);
}

}  // namespace tq
