// Read-side kernels on the reference's flat tensor layouts: query rotation /
// sketch, the asymmetric score estimator, and key / value de-quantisation.

#include "tq_common.h"
#include "tq_prep.h"
#include "tq_options.h"
#include "tq_decode_mfma.h"

namespace tq {

// q_rot = q Pi^T, q_sk = q S^T for `rows` query vectors (triton_kernels.py:527-528), fp32.
// A workgroup handles R consecutive rows (the query heads of one KV head when
// called from the decode path) and a slice of ROT_COLS output columns with
// ROT_COLS x ROT_SLICES threads: thread (j, s) sums slice s of the contraction for
// its column of every row, so each matrix element is read once per workgroup; the
// slices meet in LDS.
constexpr int ROT_SLICES = 8;      // (ROT_COLS = 32 output columns per workgroup: tq_prep.h)

// sq[0 .. tot) = elements off .. off + have of q as fp32, zeros behind them (off, have and tot multiples of 8):
// 16-byte loads, all of a thread's in flight together, when q allows them
__device__ __forceinline__ void rows_to_lds(const void* __restrict__ q, int dtype, int64_t off, int have, int tot,
                                            float* __restrict__ sq, int tid, int n_threads) {
  if ((((uintptr_t)q) & 15) == 0 && dtype != TQ_F32) {
    const uint4* src = (const uint4*)((const uint16_t*)q + off);
    const bool bf = dtype == TQ_BF16;
#pragma unroll 4
    for (int c = tid; c < tot / 8; c += n_threads) {
      const uint4 w = 8 * c < have ? src[c] : make_uint4(0u, 0u, 0u, 0u);
      const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
      float v[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[2 * k] = bf ? __uint_as_float(ws[k] << 16) : f16_bits_to_f32((uint16_t)(ws[k] & 0xffffu));
        v[2 * k + 1] = bf ? __uint_as_float(ws[k] & 0xffff0000u) : f16_bits_to_f32((uint16_t)(ws[k] >> 16));
      }
      *(float4*)(sq + 8 * c) = make_float4(v[0], v[1], v[2], v[3]);
      *(float4*)(sq + 8 * c + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
  } else if ((((uintptr_t)q) & 15) == 0) {
    const float4* src = (const float4*)((const float*)q + off);
#pragma unroll 4
    for (int c = tid; c < tot / 4; c += n_threads)
      *(float4*)(sq + 4 * c) = 4 * c < have ? src[c] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  } else {
    for (int o = tid; o < tot; o += n_threads) sq[o] = o < have ? load_as_f32(q, off + o, dtype) : 0.0f;
  }
}

// BATCH: matrix rows of both matrices requested before the first is used (8, 16 or 24, a divisor of the d / 8 rows a
// thread contracts): the kernel is a chain of memory latencies, one per batch (head_dim 576: 9 -> 3; the sums add in
// the same order whatever the batch).
// HALVES (1 or 2): a workgroup of HALVES x 256 threads takes HALVES x 8 rows; the halves run the same loads a
// moment apart, so the second finds the matrix lines in the compute unit's cache: with many rows half the traffic
// from L2 for the same work per thread (128 rows at head_dim 576: 42 -> 21 MB).
// PACK (a decode step at a head size of the wide-head page kernel): the workgroup also turns its 32 columns - one
// plane word - of every row into the kernel's fp6 query operands (four terms per value, as prep_query_body packs them
// for the other head sizes) and writes them where the page-kernel workgroups of the row's head group fetch them,
// and the workgroups of the first word write the rows' statistics.  The operands are normalised by bounds every
// workgroup can compute from the raw query: |q_rot_j| <= ||q|| (Pi is orthogonal) and |q_sk_j| <= ||q|| max_j ||S_j||;
// the sums over all coordinates the scores need are q . colsum(Pi), q . colsum(S).
template <int BATCH, int HALVES, bool PACK>
__global__ void __launch_bounds__(ROT_COLS * ROT_SLICES * HALVES)
rotate_query_kernel(const void* __restrict__ q, int dtype, int64_t rows, int R, tq_layer ly, float* __restrict__ q_rot,
                    float* __restrict__ q_sk, WidePack wp) {
  extern __shared__ __align__(16) float sm[];
  constexpr int T1 = ROT_COLS * ROT_SLICES;
  const int d = ly.d, tid = threadIdx.x, half = tid / T1, t1 = tid - half * T1, jl = t1 % ROT_COLS, sl = t1 / ROT_COLS;
  const int j = blockIdx.y * ROT_COLS + jl;
  float* sq = sm;                                  // [R][d] inputs (R rows per workgroup: up to 8 per half)
  float* pa = sq + R * d;                          // [ROT_SLICES][R][ROT_COLS] partial sums
  float* pb = pa + ROT_SLICES * R * ROT_COLS;
  const int64_t row0 = (int64_t)blockIdx.x * R;
  const int nr = (int)((rows - row0) < R ? (rows - row0) : R);
  // the first batch of matrix rows (and, below, the column sums) is requested before the queries: neither depends on them
  const int per = d / ROT_SLICES, i0 = sl * per;
  float mp[BATCH], ms[BATCH];
#pragma unroll
  for (int k = 0; k < BATCH; ++k) {
    mp[k] = ly.PiT[(int64_t)(i0 + k) * d + j];
    ms[k] = ly.ST[(int64_t)(i0 + k) * d + j];
  }
  constexpr int CS = PACK ? 12 : 1;                // column sums of a lane (PACK; d <= 768)
  float cs1[CS], cs2[CS];
  if constexpr (PACK) {
#pragma unroll
    for (int k = 0; k < CS; ++k) {
      const int c = min((tid & 63) + 64 * k, d - 1);
      cs1[k] = ly.Pi_colsum[c];
      cs2[k] = ly.S_colsum[c];
    }
  }
  rows_to_lds(q, dtype, row0 * d, nr * d, R * d, sq, tid, (int)blockDim.x);
  __syncthreads();
  float* s_rot = pb + ROT_SLICES * R * ROT_COLS;   // PACK: [R][ROT_COLS] this word's rotated values, then the sketched ones
  float* s_sk = s_rot + R * ROT_COLS;
  float* s_rs = s_sk + R * ROT_COLS;               // PACK: [R][2] multipliers of q_rot / q_sk
  float* s_cf = s_rs + 2 * R;                      // PACK: [16] coefficient of each term plane
  if constexpr (PACK) {
    // row statistics, a wavefront per row (every workgroup of the rows computes the same ones)
    const int lane = tid & 63, wv = tid >> 6, n_wv = (int)blockDim.x >> 6;
    float cmax = 0.0f;
    for (int t = 0; t < ly.n_terms; ++t) cmax = fmaxf(cmax, fabsf(ly.term_coef[t]));
    for (int r = wv; r < nr; r += n_wv) {
      float ss = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int k = 0; k < CS; ++k) {
        const int c = lane + 64 * k;
        const float x = c < d ? sq[r * d + c] : 0.0f;
        ss = fmaf(x, x, ss);
        s1 = fmaf(x, cs1[k], s1);
        s2 = fmaf(x, cs2[k], s2);
      }
      ss = wave_sum_fast(ss); s1 = wave_sum_fast(s1); s2 = wave_sum_fast(s2);
      if (lane == 0) {
        const float nq = sqrtf(ss), k = wp.sm_scale * 1.4426950408889634f;
        // bound < 2^e: e = exponent field - 126, kept within +-100
        const int e1 = min(max((int)((__float_as_uint(fabsf(k) * nq * cmax) >> 23) & 255u) - 126, -100), 100);
        const int e2 = min(max((int)((__float_as_uint(2.0f * fabsf(k * ly.qjl_scale) * nq * ly.S_rownorm_max) >> 23) & 255u) - 126, -100), 100);
        s_rs[2 * r] = k * __uint_as_float((uint32_t)(127 - e1) << 23);
        s_rs[2 * r + 1] = 2.0f * k * ly.qjl_scale * __uint_as_float((uint32_t)(127 - e2) << 23);
        if (blockIdx.y == 0) {
          float* st = wp.q_stat + (row0 + r) * 4;
          st[0] = (float)e1; st[1] = (float)e2; st[2] = k * ly.term_const * s1; st[3] = -k * ly.qjl_scale * s2;
        }
      }
    }
    if (tid < 16) s_cf[tid] = wide_term_plane_coef(ly, wp.ntp, tid);
  }
  const int r0 = half * ROT_MAX_ROWS, RH = min(R - r0, ROT_MAX_ROWS);      // this half's rows: r0 .. r0 + RH - 1
  float a[ROT_MAX_ROWS], b[ROT_MAX_ROWS];
#pragma unroll
  for (int r = 0; r < ROT_MAX_ROWS; ++r) a[r] = b[r] = 0.0f;
  // BATCH matrix rows at a time: all their loads are in flight before the first use
  for (int ib = i0; ib < i0 + per; ib += BATCH) {
    if (ib > i0) {                                         // (the same for every thread)
#pragma unroll
      for (int k = 0; k < BATCH; ++k) {
        mp[k] = ly.PiT[(int64_t)(ib + k) * d + j];
        ms[k] = ly.ST[(int64_t)(ib + k) * d + j];
      }
    }
#pragma unroll
    for (int r = 0; r < ROT_MAX_ROWS; ++r) {
      if (r < RH) {
#pragma unroll
        for (int k4 = 0; k4 < BATCH / 4; ++k4) {
          const float4 x4 = *(const float4*)(sq + (r0 + r) * d + ib + 4 * k4);      // (ib and d are multiples of 8)
          const float xs[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            a[r] = fmaf(xs[k], mp[4 * k4 + k], a[r]);
            b[r] = fmaf(xs[k], ms[4 * k4 + k], b[r]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < ROT_MAX_ROWS; ++r) {
    if (r < RH) {
      pa[(sl * R + r0 + r) * ROT_COLS + jl] = a[r];
      pb[(sl * R + r0 + r) * ROT_COLS + jl] = b[r];
    }
  }
  __syncthreads();
  for (int o = tid; o < nr * ROT_COLS; o += blockDim.x) {
    const int r = o / ROT_COLS, c = o - r * ROT_COLS;
    float ra = 0.0f, rb = 0.0f;
    for (int k = 0; k < ROT_SLICES; ++k) { ra += pa[(k * R + r) * ROT_COLS + c]; rb += pb[(k * R + r) * ROT_COLS + c]; }
    q_rot[(row0 + r) * d + blockIdx.y * ROT_COLS + c] = ra;
    q_sk[(row0 + r) * d + blockIdx.y * ROT_COLS + c] = rb;
    if constexpr (PACK) {
      s_rot[o] = ra;
      s_sk[o] = rb;
    }
  }
  if constexpr (PACK) {
    __syncthreads();
    wide_pack_word(wp, d, nr, (int)row0, (int)blockIdx.y, s_rot, s_sk, s_rs, s_cf, tid, (int)blockDim.x, 0, wp.ntp);
  }
}

// the rotation on the matrix cores (rotate_mfma_body, tq_prep.h) as a launch of its own
template <int KPW, bool F16Q>
__global__ void __launch_bounds__(ROTM_THREADS)
rotate_mfma_kernel(const uint16_t* __restrict__ q, int64_t rows, int n_tiles, tq_layer ly, float* __restrict__ q_rot,
                   float* __restrict__ q_sk, WidePack wp) {
  extern __shared__ __align__(16) float sm[];
  rotate_mfma_body<KPW, F16Q>(q, rows, n_tiles, ly, q_rot, q_sk, wp, (int)blockIdx.x, sm);
}

template <int KPW>
__global__ void __launch_bounds__(ROTM_THREADS)
rotate_mfma_tiles_kernel(const uint16_t* __restrict__ q, int64_t rows, int n_tiles, int tpw, tq_layer ly,
                         float* __restrict__ q_rot, float* __restrict__ q_sk, WidePack wp) {
  extern __shared__ __align__(16) float sm[];
  rotate_mfma_tiles_body<KPW>(q, rows, n_tiles, tpw, ly, q_rot, q_sk, wp, (int)blockIdx.x, sm);
}

template <int PER, int DT, bool PACKED>
__global__ void __launch_bounds__(PREP_COLS * PREP_SLICES)
prep_query_kernel(const void* __restrict__ q, int G, int gpw, int64_t n_rows, int g_tot, tq_layer ly, float sm_scale,
                  float* __restrict__ q_rot, float* __restrict__ q_sk, float* __restrict__ q_stat,
                  uint32_t* __restrict__ qa_pack, unsigned long long* __restrict__ arrivals, int head_rows, int n_units,
                  int n_prep, PagePrefetch pf) {
  extern __shared__ __align__(16) float sm[];
  // the preparation workgroups first (unit fastest, as a two-dimensional grid would order them), then the
  // workgroups that read the page kernel's first pages ahead of it
  const int id = blockIdx.x;
  if (id < n_prep)
    prep_query_body<PER, DT, PACKED>(q, G, gpw, n_rows, g_tot, ly, sm_scale, q_rot, q_sk, q_stat, qa_pack, arrivals, head_rows,
                                     id % n_units, id / n_units, sm);
  else
    prefetch_pages_body<PREP_COLS * PREP_SLICES>(pf, id - n_prep);
}

// The preparation on the matrix cores (bf16 queries, head_dim 128 / 256): a workgroup per (tile of up to 16 query
// rows, plane word), then the page-prefetch workgroups.
// WW: a workgroup per tile, its wavefronts each taking a plane word at a time.
template <int D, bool WW>
__global__ void __launch_bounds__(PREP_MFMA_THREADS)
prep_mfma_kernel(const uint16_t* __restrict__ q, int G, int64_t n_rows, tq_layer ly, float sm_scale,
                 float* __restrict__ q_stat, uint32_t* __restrict__ qa_pack, unsigned long long* __restrict__ arrivals,
                 int head_rows, int n_tiles, int n_prep, PagePrefetch pf) {
  extern __shared__ __align__(16) float sm[];
  const int id = blockIdx.x;
  if (id < n_prep)
    prep_mfma_body<D, WW>(q, G, n_rows, ly, sm_scale, q_stat, qa_pack, arrivals, head_rows, id % n_tiles, id / n_tiles, sm);
  else
    prefetch_pages_body<PREP_MFMA_THREADS>(pf, id - n_prep);
}

// scores[b, i, k] for a tile of QT queries and one key per thread.  The rotated and sketched queries sit
// in LDS as [coordinate][QT] rows, so a 16-byte broadcast read feeds four queries; a thread reads its key's
// packed codes 32 coordinates (eff index words, one sign word) at a time.  NQ = 4 serves tiles of at most four
// queries with half the work.  Each (query, key) sum runs over the coordinates in ascending order.
constexpr int QT = 8;

template <int NQ>
__device__ __forceinline__ void score_accumulate(const float* s_rot, const float* s_sk, const float* s_cent, int d,
                                                 int eff, const uint32_t* ip, const uint32_t* sp, float (&am)[QT],
                                                 float (&aq)[QT]) {
  const unsigned mask = (1u << eff) - 1u;
  for (int c0 = 0; c0 < d; c0 += 32) {
    uint32_t iw[4] = {0, 0, 0, 0};
    const uint32_t* w = ip + (c0 >> 5) * eff;
    iw[0] = w[0];
    if (eff >= 2) iw[1] = w[1];
    if (eff == 4) { iw[2] = w[2]; iw[3] = w[3]; }
    const uint32_t sb = sp[c0 >> 5];
#pragma unroll
    for (int j = 0; j < 4; ++j) {                    // index word j of this run: 32 / eff coordinates
      const int per_w = 32 / eff;
      if (j * per_w >= 32) break;
      for (int s = 0; s < per_w; ++s) {
        const int cl = j * per_w + s, c = c0 + cl;
        const float cv = s_cent[(iw[j] >> (eff * s)) & mask];
        const float sg = ((sb >> cl) & 1u) ? 1.0f : -1.0f;
#pragma unroll
        for (int i4 = 0; i4 < NQ / 4; ++i4) {
          const float4 r = *reinterpret_cast<const float4*>(s_rot + c * QT + 4 * i4);
          const float4 k = *reinterpret_cast<const float4*>(s_sk + c * QT + 4 * i4);
          am[4 * i4 + 0] = fmaf(r.x, cv, am[4 * i4 + 0]);
          am[4 * i4 + 1] = fmaf(r.y, cv, am[4 * i4 + 1]);
          am[4 * i4 + 2] = fmaf(r.z, cv, am[4 * i4 + 2]);
          am[4 * i4 + 3] = fmaf(r.w, cv, am[4 * i4 + 3]);
          aq[4 * i4 + 0] = fmaf(k.x, sg, aq[4 * i4 + 0]);
          aq[4 * i4 + 1] = fmaf(k.y, sg, aq[4 * i4 + 1]);
          aq[4 * i4 + 2] = fmaf(k.z, sg, aq[4 * i4 + 2]);
          aq[4 * i4 + 3] = fmaf(k.w, sg, aq[4 * i4 + 3]);
        }
      }
    }
  }
}

__global__ void __launch_bounds__(256)
score_kernel(const float* __restrict__ q_rot, const float* __restrict__ q_sk, int64_t n_q,
             const uint8_t* __restrict__ idx, const uint8_t* __restrict__ signs, const void* __restrict__ norms,
             int norm_dtype, const float* __restrict__ rnorms, int64_t n_k, tq_layer ly, float* __restrict__ scores) {
  extern __shared__ __align__(16) float sm[];
  const int d = ly.d, mb = ly.mse_bits;
  float* s_rot = sm;              // [d][QT]
  float* s_sk = sm + QT * d;      // [d][QT]
  float* s_cent = s_sk + QT * d;  // [16]
  const int64_t b = blockIdx.z;
  const int64_t q0 = (int64_t)blockIdx.y * QT;
  const int nq = (int)((n_q - q0) < QT ? (n_q - q0) : QT);
  for (int o = threadIdx.x; o < QT * d; o += blockDim.x) {
    int i = o / d, c = o - i * d;
    bool ok = i < nq;
    s_rot[c * QT + i] = ok ? q_rot[(b * n_q + q0) * d + o] : 0.0f;
    s_sk[c * QT + i] = ok ? q_sk[(b * n_q + q0) * d + o] : 0.0f;
  }
  if (threadIdx.x < (1 << mb)) s_cent[threadIdx.x] = ly.centroids[threadIdx.x];
  __syncthreads();
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= n_k) return;
  const int eff = eff_bits(mb), row = idx_row_bytes(d, mb), srow = d >> 3;
  const uint32_t* ip = (const uint32_t*)(idx + (b * n_k + k) * row);
  const uint32_t* sp = (const uint32_t*)(signs + (b * n_k + k) * srow);
  float am[QT], aq[QT];
#pragma unroll
  for (int i = 0; i < QT; ++i) am[i] = aq[i] = 0.0f;
  if (nq <= 4) score_accumulate<4>(s_rot, s_sk, s_cent, d, eff, ip, sp, am, aq);
  else score_accumulate<8>(s_rot, s_sk, s_cent, d, eff, ip, sp, am, aq);
  const float nk = load_as_f32(norms, b * n_k + k, norm_dtype);
  const float rk = __fmul_rn(ly.qjl_scale, rnorms[b * n_k + k]);
  for (int i = 0; i < nq; ++i) scores[(b * n_q + q0 + i) * n_k + k] = __fadd_rn(__fmul_rn(am[i], nk), __fmul_rn(aq[i], rk));
}

// the same sums with byte loads, for index / sign rows that are not 4-byte aligned
__global__ void __launch_bounds__(256)
score_bytes_kernel(const float* __restrict__ q_rot, const float* __restrict__ q_sk, int64_t n_q,
                   const uint8_t* __restrict__ idx, const uint8_t* __restrict__ signs, const void* __restrict__ norms,
                   int norm_dtype, const float* __restrict__ rnorms, int64_t n_k, tq_layer ly,
                   float* __restrict__ scores) {
  extern __shared__ float sm[];
  const int d = ly.d, mb = ly.mse_bits;
  float* s_rot = sm;              // [QT][d]
  float* s_sk = sm + QT * d;      // [QT][d]
  float* s_cent = s_sk + QT * d;  // [16]
  const int64_t b = blockIdx.z;
  const int64_t q0 = (int64_t)blockIdx.y * QT;
  const int nq = (int)((n_q - q0) < QT ? (n_q - q0) : QT);
  for (int o = threadIdx.x; o < QT * d; o += blockDim.x) {
    int i = o / d;
    bool ok = i < nq;
    s_rot[o] = ok ? q_rot[(b * n_q + q0) * d + o] : 0.0f;
    s_sk[o] = ok ? q_sk[(b * n_q + q0) * d + o] : 0.0f;
  }
  if (threadIdx.x < (1 << mb)) s_cent[threadIdx.x] = ly.centroids[threadIdx.x];
  __syncthreads();
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= n_k) return;
  const int eff = eff_bits(mb), per = 8 / eff, row = idx_row_bytes(d, mb), srow = d >> 3;
  const unsigned mask = (1u << eff) - 1u;
  const uint8_t* ip = idx + (b * n_k + k) * row;
  const uint8_t* sp = signs + (b * n_k + k) * srow;
  float am[QT], aq[QT];
#pragma unroll
  for (int i = 0; i < QT; ++i) am[i] = aq[i] = 0.0f;
  for (int c0 = 0; c0 < d; c0 += 8) {
    unsigned sb = sp[c0 >> 3];
    for (int s = 0; s < 8; ++s) {
      int c = c0 + s;
      unsigned byte = ip[c / per];
      float cv = s_cent[(byte >> (eff * (c % per))) & mask];
      float sg = ((sb >> s) & 1u) ? 1.0f : -1.0f;
#pragma unroll
      for (int i = 0; i < QT; ++i) {
        am[i] = fmaf(s_rot[i * d + c], cv, am[i]);
        aq[i] = fmaf(s_sk[i * d + c], sg, aq[i]);
      }
    }
  }
  const float nk = load_as_f32(norms, b * n_k + k, norm_dtype);
  const float rk = __fmul_rn(ly.qjl_scale, rnorms[b * n_k + k]);
  for (int i = 0; i < nq; ++i) scores[(b * n_q + q0 + i) * n_k + k] = __fadd_rn(__fmul_rn(am[i], nk), __fmul_rn(aq[i], rk));
}

// x_hat for a tile of TILE vectors: (c[idx] Pi) * norm + (sigma S) * (qjl_scale * rnorm)
// (quantizer.py:151-165, 259-272).  d threads, thread i owns output coordinate i and
// sums over j in ascending order.  The tile's centroid and sign values sit in LDS as
// [j][TILE] rows (padded by 4 floats) so one 16-byte broadcast read feeds four FMAs.
template <int TILE, bool QJL>
__global__ void __launch_bounds__(1024)
dequant_keys_kernel(const uint8_t* __restrict__ idx, const uint8_t* __restrict__ signs, const void* __restrict__ norms,
                    int norm_dtype, const float* __restrict__ rnorms, int64_t n_vec, tq_layer ly,
                    float* __restrict__ out) {
  constexpr int LD = TILE + 4;
  extern __shared__ float sm[];
  const int d = ly.d, mb = ly.mse_bits, i = threadIdx.x;
  float* sc = sm;             // [d][LD] centroid values
  float* ss = sm + LD * d;    // [d][LD] +-1
  const int eff = eff_bits(mb), per = 8 / eff, row = idx_row_bytes(d, mb), srow = d >> 3;
  const unsigned mask = (1u << eff) - 1u;
  const int64_t v0 = (int64_t)blockIdx.x * TILE;
  for (int t = 0; t < TILE; ++t) {
    int64_t v = v0 + t;
    float cv = 0.0f, sg = 0.0f;
    if (v < n_vec) {
      unsigned byte = idx[v * row + i / per];
      cv = ly.centroids[(byte >> (eff * (i % per))) & mask];
      if (QJL) sg = ((signs[v * srow + (i >> 3)] >> (i & 7)) & 1u) ? 1.0f : -1.0f;
    }
    sc[i * LD + t] = cv;
    if (QJL) ss[i * LD + t] = sg;
  }
  __syncthreads();
  float a[TILE], b[QJL ? TILE : 1];
#pragma unroll
  for (int t = 0; t < TILE; ++t) a[t] = 0.0f;
#pragma unroll
  for (int t = 0; t < (QJL ? TILE : 1); ++t) b[t] = 0.0f;
#pragma unroll 2
  for (int j = 0; j < d; ++j) {
    const float pv = ly.Pi[(int64_t)j * d + i];
    const float sv = QJL ? ly.S[(int64_t)j * d + i] : 0.0f;
#pragma unroll
    for (int t4 = 0; t4 < TILE / 4; ++t4) {
      const float4 c = *reinterpret_cast<const float4*>(sc + j * LD + 4 * t4);
      a[4 * t4 + 0] = fmaf(c.x, pv, a[4 * t4 + 0]);
      a[4 * t4 + 1] = fmaf(c.y, pv, a[4 * t4 + 1]);
      a[4 * t4 + 2] = fmaf(c.z, pv, a[4 * t4 + 2]);
      a[4 * t4 + 3] = fmaf(c.w, pv, a[4 * t4 + 3]);
      if (QJL) {
        const float4 g = *reinterpret_cast<const float4*>(ss + j * LD + 4 * t4);
        b[4 * t4 + 0] = fmaf(g.x, sv, b[4 * t4 + 0]);
        b[4 * t4 + 1] = fmaf(g.y, sv, b[4 * t4 + 1]);
        b[4 * t4 + 2] = fmaf(g.z, sv, b[4 * t4 + 2]);
        b[4 * t4 + 3] = fmaf(g.w, sv, b[4 * t4 + 3]);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TILE; ++t) {
    int64_t v = v0 + t;
    if (v < n_vec) {
      float r = __fmul_rn(a[t], load_as_f32(norms, v, norm_dtype));
      if (QJL) r = __fadd_rn(r, __fmul_rn(b[t], __fmul_rn(ly.qjl_scale, rnorms[v])));
      out[v * d + i] = r;
    }
  }
}

template <int TILE, bool QJL>
static int launch_dequant_keys(const uint8_t* idx, const uint8_t* signs, const void* norms, int norm_dtype,
                               const float* rnorms, int64_t n_vec, const tq_layer* layer, float* out, hipStream_t st) {
  const int d = layer->d;
  const size_t smem = (size_t)(QJL ? 2 : 1) * (TILE + 4) * d * sizeof(float);
  auto kern = dequant_keys_kernel<TILE, QJL>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return (int)e;
  }
  kern<<<dim3((unsigned)((n_vec + TILE - 1) / TILE)), dim3(d), smem, st>>>(idx, signs, norms, norm_dtype, rnorms, n_vec,
                                                                            *layer, out);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

// fp32(code) * scale + zero with separately rounded multiply and add (kv_cache.py:101-116)
__global__ void dequant_values_kernel(const uint8_t* __restrict__ data, const void* __restrict__ scales,
                                      const void* __restrict__ zeros, int dtype, int64_t n_vec, int d, int gs, int bits,
                                      float* __restrict__ out) {
  int64_t gid = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (gid >= n_vec * d) return;
  int64_t v = gid / d;
  int c = (int)(gid - v * d);
  const int per = 8 / bits, ng = d / gs;
  unsigned byte = data[v * (d / per) + c / per];
  float code = (float)((byte >> (bits * (c % per))) & ((1u << bits) - 1u));
  float s = load_as_f32(scales, v * ng + c / gs, dtype);
  float z = load_as_f32(zeros, v * ng + c / gs, dtype);
  out[gid] = __fadd_rn(__fmul_rn(code, s), z);
}

// The same arithmetic, a thread per 8 consecutive channels (they share a group when the group size is a
// multiple of 8): one load of the packed codes, scale and zero read once, two 16-byte stores.
template <int BITS>
__global__ void dequant_values8_kernel(const uint8_t* __restrict__ data, const void* __restrict__ scales,
                                       const void* __restrict__ zeros, int dtype, int64_t n_vec, int d, int gs,
                                       float* __restrict__ out) {
  const int64_t gid = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;      // chunk of 8 channels
  const int cpv = d >> 3;
  if (gid >= n_vec * cpv) return;
  const int64_t v = gid / cpv;
  const int c0 = (int)(gid - v * cpv) * 8;
  const int ng = d / gs;
  const uint8_t* src = data + v * (d * BITS / 8) + c0 * BITS / 8;
  uint64_t bits64;
  if (BITS == 2) bits64 = *(const uint16_t*)src;
  else if (BITS == 4) bits64 = *(const uint32_t*)src;
  else bits64 = *(const uint64_t*)src;
  const float sc = load_as_f32(scales, v * ng + c0 / gs, dtype);
  const float z = load_as_f32(zeros, v * ng + c0 / gs, dtype);
  float r[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float code = (float)(uint32_t)((bits64 >> (BITS * i)) & ((1u << BITS) - 1u));
    r[i] = __fadd_rn(__fmul_rn(code, sc), z);
  }
  float4* dst = (float4*)(out + v * d + c0);
  dst[0] = make_float4(r[0], r[1], r[2], r[3]);
  dst[1] = make_float4(r[4], r[5], r[6], r[7]);
}

}  // namespace tq

using namespace tq;

static int check_layer_rd(const tq_layer* ly, bool need_sketch) {
  if (!ly) return TQ_ENULL;
  if (ly->d < 64 || ly->d > 768 || (ly->d & 63)) return TQ_EUNSUPPORTED;
  if (ly->mse_bits < 1 || ly->mse_bits > 4) return TQ_EUNSUPPORTED;
  if (!ly->Pi || !ly->PiT || !ly->centroids) return TQ_ENULL;
  if (need_sketch && (!ly->S || !ly->ST)) return TQ_ENULL;
  return TQ_OK;
}

namespace tq {
// matrix-core de-quantiser (tq_quantize_mfma.hip); TQ_EUNSUPPORTED = use the vector-ALU kernel
int launch_dequant_mfma(const uint8_t* idx, const uint8_t* signs, const void* norms, int norm_dtype, const float* rnorms,
                        int64_t n_vec, const tq_layer& ly, float* out, hipStream_t st);

// Whether launch_rotate_query prepares these rows on the matrix cores (bf16 queries at head_dim 128 / 256 with the
// split matrices at hand; whole groups of G heads; operands only).
// (head_dim 256 with few rows keeps the vector-ALU kernel: 64 rows - 32 workgroups here, each pulling 96 KB of
// matrix terms - measured 1 us slower per step; from 64 workgroups on the two are level or this one ahead:
// 16 x 8192 at 32 q heads 35.0 -> 34.5 us per step, 64 x 2048 40.2 -> 36.4, 256 x 1024 107.6 -> 86.2)
bool prep_on_matrix_cores(const void* q, int dtype, int64_t rows, const tq_layer* layer, int G, int g_tot) {
  const int d = layer->d;
  if (g_tot > 0 && g_tot % G == 0) g_tot = 0;
  const int rows_tile = (16 / G) * G;
  const int64_t n_mprep = ((rows + rows_tile - 1) / rows_tile) * (d / 32);
  const int mfma_opt = opt_prep_mfma.load(std::memory_order_relaxed);
  return dtype == TQ_BF16 && (d == 128 || d == 256) && layer->Pi_split && layer->S_split && layer->Pi_colsum &&
         layer->S_colsum && g_tot == 0 && G <= ROT_MAX_ROWS && rows % G == 0 && (((uintptr_t)q) & 15) == 0 &&
         mfma_opt != 0 && (d == 128 || n_mprep >= 64 || mfma_opt > 1);
}

// Whether the rotation launch of a decode step also packs the wide-head page kernel's query operands ...
static bool rotate_packs(int64_t rows, const tq_layer* layer, const WidePack* wide) {
  return wide != nullptr && wide->qa != nullptr && wide->q_stat != nullptr && layer->Pi_colsum && layer->S_colsum &&
         wide->ntp >= 2 && wide->ntp <= 9 && rows % wide->Hq == 0 && rows < (1 << 30) && layer->d <= 768;
}
// ... and whether it does so on the matrix cores (bf16 queries with the layer's split matrices)
// row tiles a rotation workgroup takes: one while the card holds all workgroups at once (two per compute unit of the
// kernel that takes several)
static int rotate_tiles_per_workgroup(int64_t rows, int d) {
  const int64_t n_tiles = (rows + 15) / 16, pair_rounds = (2 * (d / ROT_COLS) + 7) / 8;
  const int64_t slots = 2 * (int64_t)device_compute_units();
  // (workgroups of a (word, product) pair the card has room for: the tiles are shared out among that many, so that
  // the launch is one round of workgroups and not one and a bit)
  const int64_t per_pair = slots / (8 * pair_rounds) > 0 ? slots / (8 * pair_rounds) : 1;
  const int64_t tpw = (n_tiles + per_pair - 1) / per_pair;
  return (int)(tpw > ROTM_MAX_TPW ? ROTM_MAX_TPW : (tpw < 1 ? 1 : tpw));
}
// (bf16 queries; fp16 queries as two bf16 terms while a workgroup takes one row tile)
bool rotate_on_matrix_cores(const void* q, int dtype, int64_t rows, const tq_layer* layer, const WidePack* wide) {
  const int d = layer->d;
  return rotate_packs(rows, layer, wide) && layer->Pi_split && layer->S_split &&
         (((uintptr_t)q) & 15) == 0 && d % 64 == 0 && d >= 320 && d <= 704 &&
         (dtype == TQ_BF16 || (dtype == TQ_F16 && rotate_tiles_per_workgroup(rows, d) == 1)) &&
         opt_prep_mfma.load(std::memory_order_relaxed) != 0;
}

// q_rot_unused: the caller only needs the packed operands and statistics (the page kernel on the matrix
// cores), not the fp32 rotated / sketched queries
int launch_rotate_query(const void* q, int dtype, int64_t rows, const tq_layer* layer, float* q_rot, float* q_sk,
                        float* q_stat, uint32_t* qa_pack, int G, float sm_scale, hipStream_t st, bool q_rot_unused,
                        unsigned long long* arrivals, const PagePrefetch* prefetch, int g_tot, const WidePack* wide) {
  const int d = layer->d;
  if (qa_pack) {       // operands of the matrix-core decode kernel wanted
    // g_tot: query heads per KV head when its groups of G are unequal (0: the rows are whole groups of G)
    if (g_tot > 0 && g_tot % G == 0) g_tot = 0;
    if (!q_stat || !layer->Pi_colsum || !layer->S_colsum || G > ROT_MAX_ROWS || (g_tot > 0 ? rows % g_tot : rows % G) ||
        (d != 64 && d != 128 && d != 256))
      return TQ_EUNSUPPORTED;
    const int head_rows = decode_mfma_head_rows(d, G);      // rows of a group's operands the page kernel reads
    if (q_rot_unused && prep_on_matrix_cores(q, dtype, rows, layer, G, g_tot)) {
      const int rows_tile = (16 / G) * G;
      const int n_tiles = (int)((rows + rows_tile - 1) / rows_tile);
      // (several tiles per workgroup - in turn, or their products first and then all four wavefronts packing - measured
      // slower at every size: 256 x 1024 tokens 83.0 -> 83.9 us per step with four, 64 x 2048 33.8 -> 38.6)
      // Head_dim 128 with more (tile, word) pairs than the card holds workgroups of this kernel at once (four per compute
      // unit): a workgroup per tile, its wavefronts taking a plane word each (256 x 1024 tokens, 32 q / 8 KV heads:
      // preparation 16.5 -> 12.3 us; smaller ones lose 1 - 2 us, and at head_dim 256, where a wavefront takes two words in
      // turn, 128 x 2048 at 16 q / 2 KV heads goes from 44.6 to 54.5 us per step).
      const int opt_ww = opt_prep_words.load(std::memory_order_relaxed);
      const bool ww = opt_ww < 0 ? d == 128 && (int64_t)n_tiles * (d / 32) > (int64_t)4 * device_compute_units() : opt_ww != 0;
      const int n_mprep = ww ? n_tiles : n_tiles * (d / 32);
      PagePrefetch pf;
      if (prefetch && prefetch->blocks > 0 && prefetch->n_wg > 0 && n_mprep <= 2 * device_compute_units()) pf = *prefetch;
      pf.front = n_mprep;
      const dim3 grid((unsigned)(n_mprep + (pf.blocks > 0 ? pf.n_wg : 0))), block(PREP_MFMA_THREADS);
      const size_t smem = (size_t)prep_mfma_smem_floats() * sizeof(float) * (ww ? 4 : 1);
      if (d == 128 && ww)
        prep_mfma_kernel<128, true><<<grid, block, smem, st>>>((const uint16_t*)q, G, rows, *layer, sm_scale, q_stat, qa_pack,
                                                               arrivals, head_rows, n_tiles, n_mprep, pf);
      else if (d == 128)
        prep_mfma_kernel<128, false><<<grid, block, smem, st>>>((const uint16_t*)q, G, rows, *layer, sm_scale, q_stat, qa_pack,
                                                                arrivals, head_rows, n_tiles, n_mprep, pf);
      else if (ww)
        prep_mfma_kernel<256, true><<<grid, block, smem, st>>>((const uint16_t*)q, G, rows, *layer, sm_scale, q_stat, qa_pack,
                                                               arrivals, head_rows, n_tiles, n_mprep, pf);
      else
        prep_mfma_kernel<256, false><<<grid, block, smem, st>>>((const uint16_t*)q, G, rows, *layer, sm_scale, q_stat, qa_pack,
                                                                arrivals, head_rows, n_tiles, n_mprep, pf);
      hipError_t e = hipGetLastError();
      return e == hipSuccess ? TQ_OK : (int)e;
    }
    // one group of heads per workgroup while the card holds all of them at once (three workgroups of 74 registers
    // per lane on each compute unit); beyond that, as many whole groups as fit a workgroup's eight rows
    // (64 x 2048 tokens at 32 q / 8 KV heads: 45.9 -> 42.2 us per step, 256 x 1024: 134 -> 121)
    const int gpw = g_tot > 0 ? 1 : prep_groups_per_workgroup(G, (rows / G) * (d / PREP_COLS), 3 * (int64_t)device_compute_units());
    const int64_t rows_per_wg = (int64_t)G * gpw;
    size_t smem = prep_smem_bytes(G * gpw, d);
    const int n_units = g_tot > 0 ? (int)(rows / g_tot) * ((g_tot + G - 1) / G) : (int)((rows + rows_per_wg - 1) / rows_per_wg);
    const int n_prep = n_units * (d / PREP_COLS);
    PagePrefetch pf;
    // (a preparation that already fills the card - hundreds of sequences - gains nothing from more workgroups:
    // 64 x 2048 tokens at 32 q / 8 KV heads measured 44.6 -> 46.3 us per step with them)
    if (prefetch && prefetch->blocks > 0 && prefetch->n_wg > 0 && n_prep <= 2 * device_compute_units()) pf = *prefetch;
    pf.front = n_prep;
    const dim3 grid((unsigned)(n_prep + (pf.blocks > 0 ? pf.n_wg : 0))), block(PREP_COLS * PREP_SLICES);
#define TQ_PREP(PER, DT)                                                                                               \
  {                                                                                                                    \
    if (gpw > 1)                                                                                                       \
      prep_query_kernel<PER, DT, true><<<grid, block, smem, st>>>(q, G, gpw, rows, g_tot, *layer, sm_scale, q_rot, q_sk, q_stat, \
                                                                  qa_pack, arrivals, head_rows, n_units, n_prep, pf);              \
    else                                                                                                               \
      prep_query_kernel<PER, DT, false><<<grid, block, smem, st>>>(q, G, gpw, rows, g_tot, *layer, sm_scale, q_rot, q_sk, q_stat, \
                                                                   qa_pack, arrivals, head_rows, n_units, n_prep, pf);             \
  }
#define TQ_PREP_DT(PER)                              \
  {                                                  \
    if (dtype == TQ_BF16) TQ_PREP(PER, TQ_BF16)      \
    else if (dtype == TQ_F16) TQ_PREP(PER, TQ_F16)   \
    else if (dtype == TQ_F32) TQ_PREP(PER, TQ_F32)   \
    else return TQ_EINVAL;                           \
  }
    if (d == 64) TQ_PREP_DT(4)
    else if (d == 128) TQ_PREP_DT(8)
    else TQ_PREP_DT(16)
#undef TQ_PREP_DT
#undef TQ_PREP
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TQ_OK : (int)e;
  }
  // rows per workgroup: 8, or 16 (two halves of 256 threads) when that still leaves a workgroup for half the compute units
  const bool wide_rows = rows >= 32 && ((rows + 15) / 16) * (d / ROT_COLS) >= device_compute_units() / 2;
  const int max_r = wide_rows ? 16 : ROT_MAX_ROWS;
  const int R = (int)(rows < max_r ? rows : max_r);
  if (R < 1 || d % ROT_COLS || d % (8 * ROT_SLICES)) return TQ_EUNSUPPORTED;
  const bool pack = rotate_packs(rows, layer, wide);
  const WidePack wp = pack ? *wide : WidePack{};
  // bf16 queries with the layer's split matrices: rotation and packing on the matrix cores
  if (rotate_on_matrix_cores(q, dtype, rows, layer, wide)) {
    const int n_tiles = (int)((rows + 15) / 16), pair_rounds = (2 * (d / ROT_COLS) + 7) / 8;
    // more workgroups than the card holds at once (two per compute unit of the kernel below): several row tiles per workgroup
    const int tpw = rotate_tiles_per_workgroup(rows, d);
    if (tpw > 1) {
      const int n_tg = (n_tiles + tpw - 1) / tpw;
      const dim3 tgrid((unsigned)(8 * pair_rounds * n_tg));
      const size_t tsm = (size_t)rotate_mfma_tiles_smem_floats(tpw) * sizeof(float);
#define TQ_ROTT(KPW) \
  case KPW: rotate_mfma_tiles_kernel<KPW><<<tgrid, dim3(ROTM_THREADS), tsm, st>>>((const uint16_t*)q, rows, n_tiles, tpw, *layer, q_rot, q_sk, wp); break;
      switch (d / 64) {
        TQ_ROTT(5) TQ_ROTT(6) TQ_ROTT(7) TQ_ROTT(8) TQ_ROTT(9) TQ_ROTT(10) TQ_ROTT(11)
      }
#undef TQ_ROTT
      hipError_t e = hipGetLastError();
      return e == hipSuccess ? TQ_OK : (int)e;
    }
    const dim3 mgrid((unsigned)(8 * pair_rounds * n_tiles)), mblock(ROTM_THREADS);
    const size_t msm = (size_t)rotate_mfma_smem_floats() * sizeof(float);
#define TQ_ROTM(KPW) \
  case KPW:                                                                                                            \
    if (dtype == TQ_F16) rotate_mfma_kernel<KPW, true><<<mgrid, mblock, msm, st>>>((const uint16_t*)q, rows, n_tiles, *layer, q_rot, q_sk, wp); \
    else rotate_mfma_kernel<KPW, false><<<mgrid, mblock, msm, st>>>((const uint16_t*)q, rows, n_tiles, *layer, q_rot, q_sk, wp);               \
    break;
    switch (d / 64) {
      TQ_ROTM(5) TQ_ROTM(6) TQ_ROTM(7) TQ_ROTM(8) TQ_ROTM(9) TQ_ROTM(10) TQ_ROTM(11)
    }
#undef TQ_ROTM
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TQ_OK : (int)e;
  }
  size_t smem = (size_t)(R * d + 2 * ROT_SLICES * R * ROT_COLS + (pack ? 2 * R * ROT_COLS + 2 * R + 16 : 0)) * sizeof(float);
  const dim3 rgrid((unsigned)((rows + R - 1) / R), d / ROT_COLS), rblock(ROT_COLS * ROT_SLICES * (wide_rows ? 2 : 1));
  const int per = d / ROT_SLICES;
#define TQ_ROTATE(BATCH, MAXR)                                                                                         \
  {                                                                                                                    \
    auto kern = pack ? rotate_query_kernel<BATCH, MAXR, true> : rotate_query_kernel<BATCH, MAXR, false>;             \
    if (smem > 48 * 1024) {                                                                                            \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);    \
      if (e != hipSuccess) return (int)e;                                                                              \
    }                                                                                                                  \
    kern<<<rgrid, rblock, smem, st>>>(q, dtype, rows, R, *layer, q_rot, q_sk, wp);                                     \
  }
#define TQ_ROTATE_R(BATCH)                 \
  {                                        \
    if (wide_rows) TQ_ROTATE(BATCH, 2)     \
    else TQ_ROTATE(BATCH, 1)               \
  }
  if (per % 24 == 0) TQ_ROTATE_R(24)
  else if (per % 16 == 0) TQ_ROTATE_R(16)
  else TQ_ROTATE_R(8)
#undef TQ_ROTATE_R
#undef TQ_ROTATE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  return TQ_OK;
}
}  // namespace tq

extern "C" int tq_rotate_query(const void* q, int dtype, int64_t rows, const tq_layer* layer, float* q_rot,
                               float* q_sk, void* stream) {
  int rc = check_layer_rd(layer, true);
  if (rc) return rc;
  if (!q || !q_rot || !q_sk) return TQ_ENULL;
  if (rows < 0 || dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  if (rows == 0) return TQ_OK;
  return launch_rotate_query(q, dtype, rows, layer, q_rot, q_sk, nullptr, nullptr, 1, 0.0f, (hipStream_t)stream, false, nullptr, nullptr, 0, nullptr);
}

extern "C" int tq_score(const void* q, int dtype, int64_t batch, int64_t n_q, const uint8_t* idx, const uint8_t* signs,
                        const void* norms, int norm_dtype, const float* rnorms, int64_t n_k, const tq_layer* layer,
                        float* scores, float* work, void* stream) {
  int rc = check_layer_rd(layer, true);
  if (rc) return rc;
  if (!q || !idx || !signs || !norms || !rnorms || !scores || !work) return TQ_ENULL;
  if (batch < 0 || n_q < 0 || n_k < 0 || norm_dtype < TQ_F32 || norm_dtype > TQ_BF16) return TQ_EINVAL;
  if (batch > 65535) return TQ_EUNSUPPORTED;
  if (batch == 0 || n_q == 0 || n_k == 0) return TQ_OK;
  const int d = layer->d;
  float* q_rot = work;
  float* q_sk = work + batch * n_q * d;
  rc = tq_rotate_query(q, dtype, batch * n_q, layer, q_rot, q_sk, stream);
  if (rc) return rc;
  dim3 grid((unsigned)((n_k + 255) / 256), (unsigned)((n_q + QT - 1) / QT), (unsigned)batch);
  size_t smem = (2 * QT * d + 16) * sizeof(float);
  if ((uintptr_t)idx % 4 == 0 && (uintptr_t)signs % 4 == 0)
    score_kernel<<<grid, dim3(256), smem, (hipStream_t)stream>>>(q_rot, q_sk, n_q, idx, signs, norms, norm_dtype,
                                                                rnorms, n_k, *layer, scores);
  else
    score_bytes_kernel<<<grid, dim3(256), smem, (hipStream_t)stream>>>(q_rot, q_sk, n_q, idx, signs, norms,
                                                                      norm_dtype, rnorms, n_k, *layer, scores);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

extern "C" int tq_dequant_keys(const uint8_t* idx, const uint8_t* signs, const void* norms, int norm_dtype,
                               const float* rnorms, int64_t n_vec, const tq_layer* layer, float* out, void* stream) {
  int rc = check_layer_rd(layer, signs != nullptr);
  if (rc) return rc;
  if (!idx || !norms || !out) return TQ_ENULL;
  if (signs && !rnorms) return TQ_ENULL;
  if (n_vec < 0 || norm_dtype < TQ_F32 || norm_dtype > TQ_BF16) return TQ_EINVAL;
  if (n_vec == 0) return TQ_OK;
  hipStream_t st = (hipStream_t)stream;
  rc = tq::launch_dequant_mfma(idx, signs, norms, norm_dtype, rnorms, n_vec, *layer, out, st);
  if (rc != TQ_EUNSUPPORTED) return rc;
  // vector-ALU kernel: 32 vectors per workgroup while both LDS tiles fit (d <= 512), else 16
  const bool wide = layer->d <= 512;
  if (signs)
    return wide ? launch_dequant_keys<32, true>(idx, signs, norms, norm_dtype, rnorms, n_vec, layer, out, st)
                : launch_dequant_keys<16, true>(idx, signs, norms, norm_dtype, rnorms, n_vec, layer, out, st);
  return wide ? launch_dequant_keys<32, false>(idx, signs, norms, norm_dtype, rnorms, n_vec, layer, out, st)
              : launch_dequant_keys<16, false>(idx, signs, norms, norm_dtype, rnorms, n_vec, layer, out, st);
}

extern "C" int tq_dequant_values(const uint8_t* data, const void* scales, const void* zeros, int dtype, int64_t n_vec,
                                 int d, int group_size, int bits, float* out, void* stream) {
  if (!data || !scales || !zeros || !out) return TQ_ENULL;
  if (bits != 2 && bits != 4 && bits != 8) return TQ_EUNSUPPORTED;
  if (d <= 0 || group_size <= 0 || d % group_size || (d * bits) % 8 || n_vec < 0) return TQ_EINVAL;
  if (dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  if (n_vec == 0) return TQ_OK;
  hipStream_t st = (hipStream_t)stream;
  // chunks of 8 channels when they stay inside a group and the accesses are aligned
  const int cb = bits;                                          // bytes of codes per chunk
  if (d % 8 == 0 && group_size % 8 == 0 && (uintptr_t)data % cb == 0 && (uintptr_t)out % 16 == 0) {
    const int64_t chunks = n_vec * (d / 8);
    const dim3 grid((unsigned)((chunks + 255) / 256)), block(256);
    if (bits == 2) dequant_values8_kernel<2><<<grid, block, 0, st>>>(data, scales, zeros, dtype, n_vec, d, group_size, out);
    else if (bits == 4) dequant_values8_kernel<4><<<grid, block, 0, st>>>(data, scales, zeros, dtype, n_vec, d, group_size, out);
    else dequant_values8_kernel<8><<<grid, block, 0, st>>>(data, scales, zeros, dtype, n_vec, d, group_size, out);
    TQ_CHECK_LAUNCH();
    return TQ_OK;
  }
  int64_t total = n_vec * d;
  dequant_values_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
      data, scales, zeros, dtype, n_vec, d, group_size, bits, out);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}
