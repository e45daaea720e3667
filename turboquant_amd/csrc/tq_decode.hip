// Fused decode attention over the paged compressed store.
//
//   stage 0  rotate_query (tq_score.hip): q_rot = q Pi^T, q_sk = q S^T
//   stage 1  decode_pages_kernel: one workgroup per (split, KV head, sequence)
//            walks its share of the sequence's pages; all G query heads of the
//            group are scored from one read of the page; online softmax and the
//            value accumulation stay in registers; result = partial (m, l, acc)
//            exact_tail_words_kernel / exact_tail_kernel: the same partial for the exact recent tokens
//            (prep_tail_kernel: stage 0 and the exact tail in one launch, for small grids)
//   stage 2  merge_kernel: log-sum-exp merge of the partials, cast to q's dtype
//
// Score of a token (triton_kernels.py:49-53,138):
//   s = sm_scale * ( norm * sum_j q_rot[j] c[idx_j] + qjl_scale * rnorm * sum_j q_sk[j] sigma_j )

#include <atomic>

#include <chrono>
#include <cstring>
#include <type_traits>

#include <hip/hip_ext.h>

#include "tq_common.h"
#include "tq_prep.h"
#include "tq_decode_mfma.h"
#include "tq_options.h"

// Device memory of the entry point that allocates nothing (tq_decode_attn_paged_noalloc): the split partials,
// the rotated queries and the packed query operands of one decode call.  One copy per GPU the library's code
// is loaded on, held until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress; kernels receive the address that call returned.
static __device__ __align__(256) unsigned char scratch[TQ_NOALLOC_SCRATCH_BYTES];

namespace tq {

constexpr int G_MAX = 16;      // query heads per KV head handled by one workgroup of the general page kernel
constexpr int G_LIMIT = 128;   // ... and per KV head in all: the matrix-core kernels serve them in groups of at most 8
constexpr float NEG_BIG = -1.0e30f;

// General page kernel (vector ALU) for the shapes without a matrix-core kernel: any head_dim that is a
// multiple of 64, 1..4-bit indices, 2/4-bit values, fp16 / bf16 / fp32 pools, up to G_MAX query heads per
// KV head.  A workgroup of 256 threads walks its pages in chunks of 256 tokens (16 pages):
//   scores   a thread per token: the key's plane words are read a word at a time, the rotated / sketched
//            queries sit in LDS as [coordinate][GP] rows (GP = query heads rounded up to 4) so that one
//            16-byte broadcast read feeds four heads;
//   softmax  online over chunks: the chunk maxima per head come from a [16 heads][16 lanes] reduction;
//   values   a thread per channel (and per slice of the chunk's tokens while head_dim < 256): codes from the
//            channel's field, scale / zero per (group, token), weights from LDS, four heads per read.
constexpr int GEN_THREADS = 256, GEN_CHUNK = 256;

// 16 consecutive elements of the pool's dtype (a 16-byte aligned row) as fp32
__device__ __forceinline__ void load_row16(const uint8_t* p, int dtype, float (&out)[16]) {
  if (dtype == TQ_F32) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 v = reinterpret_cast<const float4*>(p)[q];
      out[4 * q] = v.x; out[4 * q + 1] = v.y; out[4 * q + 2] = v.z; out[4 * q + 3] = v.w;
    }
  } else {
    const uint4 a = reinterpret_cast<const uint4*>(p)[0], b = reinterpret_cast<const uint4*>(p)[1];
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      out[2 * q] = dtype == TQ_BF16 ? __uint_as_float(w[q] << 16) : f16_bits_to_f32((uint16_t)(w[q] & 0xffffu));
      out[2 * q + 1] = dtype == TQ_BF16 ? __uint_as_float(w[q] & 0xffff0000u) : f16_bits_to_f32((uint16_t)(w[q] >> 16));
    }
  }
}

template <int VB, int GP4>      // GP4 = GP / 4
__global__ void __launch_bounds__(GEN_THREADS)
decode_pages_kernel(const float* __restrict__ q_rot, const float* __restrict__ q_sk, int Hq, int Hkv,
                    const uint8_t* __restrict__ pool, const int32_t* __restrict__ block_table, int bt_stride,
                    const int32_t* __restrict__ seq_lens, float sm_scale, tq_layer ly, tq_page_layout L,
                    float* __restrict__ parts, int n_parts, int n_split, int len_sub, int max_pages, int num_pages,
                    int head_groups) {
  constexpr int GP = 4 * GP4;
  const int d = ly.d, mb = ly.mse_bits, words = d >> 5;
  // the query heads of a KV head in head_groups groups of at most G_MAX (workgroups blockIdx.y = KV head x groups + group)
  const int g_all = Hq / Hkv, g_per = (g_all + head_groups - 1) / head_groups;
  const int split = blockIdx.x, h = (int)blockIdx.y / head_groups, b = blockIdx.z;
  const int g0 = ((int)blockIdx.y - h * head_groups) * g_per, G = min(g_per, g_all - g0);
  const int tid = threadIdx.x;

  extern __shared__ __align__(16) float smem[];
  float* s_rot = smem;                       // [d][GP]
  float* s_sk = s_rot + d * GP;              // [d][GP]
  float* s_m = s_sk + d * GP;                // [16] chunk maxima
  float* s_cent = s_m + 16;                  // [16]
  float* s_p = s_cent + 16;                  // [GEN_CHUNK][GP] scores, then softmax weights
  float* s_red = s_p;                        // after the loop: [TG][GP][d] partial accumulators
  float* s_ml = s_rot;                       // after the loop: [TG][GP] weight sums, then [GP] maxima

  for (int o = tid; o < d * GP; o += GEN_THREADS) {
    const int c = o / GP, g = o - c * GP;
    const int64_t row = (int64_t)b * Hq + h * g_all + g0 + (g < G ? g : 0);
    s_rot[o] = g < G ? q_rot[row * d + c] : 0.0f;
    s_sk[o] = g < G ? q_sk[row * d + c] : 0.0f;
  }
  if (tid < 16) s_cent[tid] = tid < (1 << mb) ? ly.centroids[tid] : 0.0f;
  __syncthreads();

  // len_sub: newest tokens that are attended to exactly.  A length beyond the block table is cut to the table.
  const int seq_len = max(min(seq_lens[b], max_pages * TQ_PAGE_TOKENS) - len_sub, 0);
  const int n_pages = (seq_len + TQ_PAGE_TOKENS - 1) / TQ_PAGE_TOKENS;
  const int per_split = (n_pages + n_split - 1) / n_split;
  const int pg_begin = split * per_split;
  const int pg_end = min(n_pages, pg_begin + per_split);
  const int32_t* bt = block_table + (int64_t)b * bt_stride;
  const int64_t head_off = (int64_t)h * L.page_bytes, page_stride = (int64_t)Hkv * L.page_bytes;

  // value stage geometry: TG slices of the chunk's tokens while head_dim < 256, else several channels a thread
  const int TG = d < GEN_THREADS ? GEN_THREADS / d : 1;          // 4 (d = 64), 2 (d = 128), 1
  const int vch = tid % (d < GEN_THREADS ? d : GEN_THREADS), vtg = d < GEN_THREADS ? tid / d : 0;
  const bool vactive = vtg < TG;                                  // d = 192: 64 threads have no slice
  const int NCH = (d + GEN_THREADS - 1) / GEN_THREADS;            // channels per thread: 1, or up to 3 (d = 768)
  constexpr int MAXCH = 3;
  const int tok_per_tg = GEN_CHUNK / TG;
  const int es = L.dtype == TQ_F32 ? 4 : 2;

  float m_run[GP], l_run[GP], acc[MAXCH][GP];
#pragma unroll
  for (int g = 0; g < GP; ++g) {
    m_run[g] = NEG_BIG;
    l_run[g] = 0.0f;
#pragma unroll
    for (int k = 0; k < MAXCH; ++k) acc[k][g] = 0.0f;
  }

  for (int pc = pg_begin; pc < pg_end; pc += GEN_CHUNK / TQ_PAGE_TOKENS) {
    // ---- scores: thread = token pc * 16 + tid
    {
      const int pi = pc + (tid >> 4), n = tid & 15;
      // a table entry outside the pool (stale or poisoned) is read as page 0 and its tokens get no weight
      const int raw = bt[pi < pg_end ? pi : pg_begin];
      const bool in_pool = (unsigned)raw < (unsigned)num_pages;
      const bool valid = pi < pg_end && pi * TQ_PAGE_TOKENS + n < seq_len && in_pool;
      const uint8_t* pg = pool + (int64_t)(in_pool ? raw : 0) * page_stride + head_off;
      float pm[GP], pq[GP];
#pragma unroll
      for (int g = 0; g < GP; ++g) pm[g] = pq[g] = 0.0f;
      for (int w = 0; w < words; ++w) {
        uint32_t pw[5] = {0, 0, 0, 0, 0};
        for (int p = 0; p <= mb; ++p) pw[p] = *(const uint32_t*)(pg + key_word_off(L, p, w, n));
        const uint32_t sgw = pw[mb];
        for (int i = 0; i < 32; ++i) {
          unsigned id = 0;
          for (int p = 0; p < mb; ++p) id = (id << 1) | ((pw[p] >> i) & 1u);
          const float cv = s_cent[id];
          const float sg = ((sgw >> i) & 1u) ? 1.0f : -1.0f;
          const float4* qr = reinterpret_cast<const float4*>(s_rot + (w * 32 + i) * GP);
          const float4* qs = reinterpret_cast<const float4*>(s_sk + (w * 32 + i) * GP);
#pragma unroll
          for (int g4 = 0; g4 < GP4; ++g4) {
            const float4 r = qr[g4], k = qs[g4];
            pm[4 * g4 + 0] = fmaf(r.x, cv, pm[4 * g4 + 0]);
            pm[4 * g4 + 1] = fmaf(r.y, cv, pm[4 * g4 + 1]);
            pm[4 * g4 + 2] = fmaf(r.z, cv, pm[4 * g4 + 2]);
            pm[4 * g4 + 3] = fmaf(r.w, cv, pm[4 * g4 + 3]);
            pq[4 * g4 + 0] = fmaf(k.x, sg, pq[4 * g4 + 0]);
            pq[4 * g4 + 1] = fmaf(k.y, sg, pq[4 * g4 + 1]);
            pq[4 * g4 + 2] = fmaf(k.z, sg, pq[4 * g4 + 2]);
            pq[4 * g4 + 3] = fmaf(k.w, sg, pq[4 * g4 + 3]);
          }
        }
      }
      const float nk = ((const float*)(pg + L.off_meta))[2 * n];
      const float rk = ly.qjl_scale * ((const float*)(pg + L.off_meta))[2 * n + 1];
#pragma unroll
      for (int g = 0; g < GP; ++g) s_p[tid * GP + g] = valid ? sm_scale * (nk * pm[g] + rk * pq[g]) : NEG_BIG;
    }
    __syncthreads();
    // ---- chunk maxima: thread (g, j) scans tokens j, j + 16, ... of head g, then the 16 lanes of a head combine
    {
      const int g = tid >> 4, j = tid & 15;
      float mx = NEG_BIG;
      if (g < GP)
        for (int t = j; t < GEN_CHUNK; t += 16) mx = fmaxf(mx, s_p[t * GP + g]);
      mx = lanes_max_dpp<16>(mx);
      if (j == 0) s_m[g] = mx;
    }
    __syncthreads();
    // ---- weights of the chunk against the new running maxima; the accumulators follow the maxima
    {
      float alpha[GP];
#pragma unroll
      for (int g = 0; g < GP; ++g) {
        const float m_new = fmaxf(m_run[g], s_m[g]);
        alpha[g] = __expf(m_run[g] - m_new);
        m_run[g] = m_new;
        l_run[g] *= alpha[g];
#pragma unroll
        for (int k = 0; k < MAXCH; ++k) acc[k][g] *= alpha[g];
      }
      const int pi = pc + (tid >> 4), n = tid & 15;
      const bool valid = pi < pg_end && pi * TQ_PAGE_TOKENS + n < seq_len &&
                         (unsigned)bt[pi < pg_end ? pi : pg_begin] < (unsigned)num_pages;
#pragma unroll
      for (int g = 0; g < GP; ++g) {
        const float sc = s_p[tid * GP + g];
        s_p[tid * GP + g] = valid ? __expf(sc - m_run[g]) : 0.0f;
      }
    }
    __syncthreads();
    // ---- values: thread = channel (x slice of the chunk's tokens)
    if (vactive) {
      const int t_begin = vtg * tok_per_tg, t_end = t_begin + tok_per_tg;
      for (int t0 = t_begin; t0 < t_end; t0 += TQ_PAGE_TOKENS) {
        const int pi = pc + (t0 >> 4);
        if (pi >= pg_end) break;
        if ((unsigned)bt[pi] >= (unsigned)num_pages) continue;        // its tokens have weight 0
        const uint8_t* pg = pool + (int64_t)bt[pi] * page_stride + head_off;
        const int n_valid = min(TQ_PAGE_TOKENS, seq_len - pi * TQ_PAGE_TOKENS);
#pragma unroll
        for (int k = 0; k < MAXCH; ++k) {
          if (k < NCH) {
            const int ch = vch + GEN_THREADS * k;
            if (ch < d) {
              const int grp = ch / L.group_size;
              const uint32_t* field = (const uint32_t*)(pg + vfield_off(L, ch));
              const uint32_t f0 = field[0], f1 = (VB >= 4) ? field[1] : 0u;
              const uint32_t f2 = (VB == 8) ? field[2] : 0u, f3 = (VB == 8) ? field[3] : 0u;
              // scales and zeros of the 16 tokens of this (page, group): two rows of 16 elements
              float sc[16], zr[16];
              load_row16(pg + L.off_vscale + grp * TQ_PAGE_TOKENS * es, L.dtype, sc);
              load_row16(pg + L.off_vzero + grp * TQ_PAGE_TOKENS * es, L.dtype, zr);
#pragma unroll
              for (int t = 0; t < TQ_PAGE_TOKENS; ++t) {
                unsigned code;
                if (VB == 2) code = (f0 >> (2 * t)) & 3u;
                else if (VB == 4) code = ((t < 8 ? f0 : f1) >> (4 * (t & 7))) & 15u;
                else code = ((t < 4 ? f0 : (t < 8 ? f1 : (t < 12 ? f2 : f3))) >> (8 * (t & 3))) & 255u;
                // slots past the end of the sequence may hold anything: they contribute an exact zero
                const float val = t < n_valid ? fmaf((float)code, sc[t], zr[t]) : 0.0f;
                const float4* pp = reinterpret_cast<const float4*>(s_p + (t0 + t) * GP);
#pragma unroll
                for (int g4 = 0; g4 < GP4; ++g4) {
                  const float4 w4 = pp[g4];
                  acc[k][4 * g4 + 0] = fmaf(w4.x, val, acc[k][4 * g4 + 0]);
                  acc[k][4 * g4 + 1] = fmaf(w4.y, val, acc[k][4 * g4 + 1]);
                  acc[k][4 * g4 + 2] = fmaf(w4.z, val, acc[k][4 * g4 + 2]);
                  acc[k][4 * g4 + 3] = fmaf(w4.w, val, acc[k][4 * g4 + 3]);
                  if (k == 0) {        // the sum of the weights rides along (the same in every thread of a slice)
                    l_run[4 * g4 + 0] += w4.x;
                    l_run[4 * g4 + 1] += w4.y;
                    l_run[4 * g4 + 2] += w4.z;
                    l_run[4 * g4 + 3] += w4.w;
                  }
                }
              }
            }
          }
        }
      }
    }
    __syncthreads();                          // s_p is rewritten by the next chunk
  }

  // ---- combine the token slices and write the partial (all threads share the same running maxima)
  if (vactive) {
#pragma unroll
    for (int k = 0; k < MAXCH; ++k) {
      if (k < NCH) {
        const int ch = vch + GEN_THREADS * k;
        if (ch < d)
#pragma unroll
          for (int g = 0; g < GP; ++g) s_red[(vtg * GP + g) * d + ch] = acc[k][g];
      }
    }
    if (vch == 0)
#pragma unroll
      for (int g = 0; g < GP; ++g) s_ml[vtg * GP + g] = l_run[g];
  }
  if (tid == 0)
#pragma unroll
    for (int g = 0; g < GP; ++g) s_ml[4 * GP + g] = m_run[g];
  __syncthreads();
  for (int o = tid; o < G * d; o += GEN_THREADS) {
    const int g = o / d, ch = o - g * d;
    float aa = 0.0f, ll = 0.0f;
    for (int t = 0; t < TG; ++t) {
      aa += s_red[(t * GP + g) * d + ch];
      ll += s_ml[t * GP + g];
    }
    float* out = parts + (((int64_t)b * Hq + h * g_all + g0 + g) * n_parts + split) * (d + 2);
    if (ch == 0) { out[0] = s_ml[4 * GP + g]; out[1] = ll; }
    out[2 + ch] = aa;
  }
}

// Partial (m, l, acc) over exact recent tokens (score.py:99-111, 138-173): one workgroup of 512 threads
// per (KV head, sequence, group of TAIL_GC query heads).  Key rows, then value rows, are staged through an
// LDS tile a chunk of tokens at a time with every load of a chunk in flight at once (the rows come from HBM:
// a loop that waits for one row per iteration costs a memory latency per token).  Scores: eight threads per
// token, each over every eighth coordinate for the group's heads at once; values: a thread per channel and
// slice of the chunk's tokens.
constexpr int TAIL_MAX_CHUNKS = 4;      // workgroups that may share the exact tokens of one (sequence, head group)
constexpr int TAIL_THREADS = 512, TAIL_WAVES = TAIL_THREADS / 64, TAIL_GC = 4, TAIL_TILE_FLOATS = 64 * 260;

static size_t tail_smem(int d, int recent_rows) {
  return ((size_t)TAIL_GC * d + (size_t)TAIL_GC * recent_rows + 2 * TAIL_GC + TAIL_TILE_FLOATS) * sizeof(float);
}

// (the element type is a template parameter: a run-time switch inside the load would put every load of
// the staging loop under a branch and serialise them)
template <int DT>
__global__ void __launch_bounds__(TAIL_THREADS)
exact_tail_kernel(const void* __restrict__ q, int Hq, int Hkv, int d, const void* __restrict__ rk,
                  const void* __restrict__ rv, int recent_rows, int64_t rs_b, int64_t rs_r, int64_t rs_h,
                  const int32_t* __restrict__ recent_len, float sm_scale, float* __restrict__ parts, int n_parts,
                  int part_index) {
  constexpr int GC = TAIL_GC;
  const int G = Hq / Hkv, h = blockIdx.x, b = blockIdx.y, g0 = blockIdx.z * GC, tid = threadIdx.x;
  const int Gc = min(GC, G - g0);                                   // query heads of this workgroup
  const int lane = tid & 63, wave = tid >> 6;
  const int R = recent_len ? min(recent_len[b], recent_rows) : recent_rows;
  extern __shared__ __align__(16) float sm[];
  float* sq = sm;                      // [d][GC]
  float* ss = sq + GC * d;             // [recent_rows][GC] scores, then softmax weights
  float* sml = ss + GC * recent_rows;  // [GC][2]
  float* tile = sml + 2 * GC;          // [CH][d + 1] rows of the current chunk; at the end [TS][GC][d] partials
  const int ld = d + 1;
  const int CH = min(TAIL_TILE_FLOATS / ld, 32 * (d < TAIL_THREADS ? TAIL_THREADS / d : 1));   // 21 tokens (d = 768) .. 252 (d = 64)
  // thread = column x row slice (rows ts, ts + TS, ...) for staging and for the value sums; a head
  // dimension above 512 gives a thread two columns
  const int TS = d < TAIL_THREADS ? TAIL_THREADS / d : 1;
  const int ch0 = d < TAIL_THREADS ? tid % d : tid, ts = d < TAIL_THREADS ? tid / d : 0;
  const bool active = ts < TS;
  const int64_t base0 = b * rs_b + h * rs_h;
  auto stage = [&](const void* src, int c0, int n) {                // rows c0 .. c0 + n - 1 -> tile
    if (active) {
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int ch = ch0 + TAIL_THREADS * k;
        if (ch < d) {
          // a thread has at most 32 rows of a chunk (CH / TS): all of its loads are issued before the first store
          float v[32];
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            const int t = ts + i * TS;
            v[i] = Elem<DT>::load(src, base0 + (int64_t)(c0 + (t < n ? t : 0)) * rs_r + ch);
          }
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            const int t = ts + i * TS;
            if (t < n) tile[t * ld + ch] = v[i];
          }
        }
      }
    }
  };
  for (int o = tid; o < GC * d; o += TAIL_THREADS) {
    const int g = o / d, c = o - g * d;
    sq[c * GC + g] = g < Gc ? Elem<DT>::load(q, ((int64_t)b * Hq + h * G + g0) * d + o) : 0.0f;
  }
  // scores
  for (int c0 = 0; c0 < R; c0 += CH) {
    const int n = min(CH, R - c0);
    stage(rk, c0, n);
    __syncthreads();
    const int seg = tid & 7;
    for (int t0 = 0; t0 < n; t0 += TAIL_THREADS / 8) {              // uniform trip count: the shuffles need every lane
      const int t = t0 + (tid >> 3);
      const float* row = tile + (t < n ? t : 0) * ld;
      float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
      for (int c = seg; c < d; c += 8) {
        const float kx = row[c];
        const float4 q4 = *reinterpret_cast<const float4*>(sq + c * GC);
        a0 = fmaf(kx, q4.x, a0);
        a1 = fmaf(kx, q4.y, a1);
        a2 = fmaf(kx, q4.z, a2);
        a3 = fmaf(kx, q4.w, a3);
      }
      a0 = lanes_sum_dpp<8>(a0);
      a1 = lanes_sum_dpp<8>(a1);
      a2 = lanes_sum_dpp<8>(a2);
      a3 = lanes_sum_dpp<8>(a3);
      if (seg == 0 && t < n)
        *reinterpret_cast<float4*>(ss + (c0 + t) * GC) = make_float4(a0 * sm_scale, a1 * sm_scale, a2 * sm_scale, a3 * sm_scale);
    }
    __syncthreads();
  }
  // softmax statistics and weights, a wavefront per query head
  for (int g = wave; g < GC; g += TAIL_WAVES) {
    float mx = NEG_BIG;
    for (int t = lane; t < R; t += 64) mx = fmaxf(mx, ss[t * GC + g]);
    mx = wave_max_fast(mx);
    float sum = 0.0f;
    for (int t = lane; t < R; t += 64) {
      float p = __expf(ss[t * GC + g] - mx);
      ss[t * GC + g] = p;
      sum += p;
    }
    sum = wave_sum_fast(sum);
    if (lane == 0) { sml[g * 2] = mx; sml[g * 2 + 1] = sum; }
  }
  __syncthreads();
  // values
  float acc[2][GC];
#pragma unroll
  for (int k = 0; k < 2; ++k)
#pragma unroll
    for (int g = 0; g < GC; ++g) acc[k][g] = 0.0f;
  for (int c0 = 0; c0 < R; c0 += CH) {
    const int n = min(CH, R - c0);
    stage(rv, c0, n);
    __syncthreads();
    if (active) {
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int ch = ch0 + TAIL_THREADS * k;
        if (ch < d) {
          for (int t = ts; t < n; t += TS) {
            const float v = tile[t * ld + ch];
            const float4 w4 = *reinterpret_cast<const float4*>(ss + (c0 + t) * GC);
            acc[k][0] = fmaf(w4.x, v, acc[k][0]);
            acc[k][1] = fmaf(w4.y, v, acc[k][1]);
            acc[k][2] = fmaf(w4.z, v, acc[k][2]);
            acc[k][3] = fmaf(w4.w, v, acc[k][3]);
          }
        }
      }
    }
    __syncthreads();
  }
  if (active) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int ch = ch0 + TAIL_THREADS * k;
      if (ch < d)
#pragma unroll
        for (int g = 0; g < GC; ++g) tile[(ts * GC + g) * d + ch] = acc[k][g];
    }
  }
  __syncthreads();
  for (int o = tid; o < Gc * d; o += TAIL_THREADS) {
    const int g = o / d, ch = o - g * d;
    float a = 0.0f;
    for (int s2 = 0; s2 < TS; ++s2) a += tile[(s2 * GC + g) * d + ch];
    float* out = parts + (((int64_t)b * Hq + h * G + g0 + g) * n_parts + part_index) * (d + 2);
    if (ch == 0) { out[0] = sml[g * 2]; out[1] = sml[g * 2 + 1]; }
    out[2 + ch] = a;
  }
}

// The same partial with the rows staged as 32-bit words (two 16-bit channels, or one fp32 channel, per
// word): the key rows AND the value rows of the first chunk are requested before anything waits, so a
// tail that fits one chunk (128 tokens at head size 256, 16-bit) costs a single memory latency.  Both
// tiles stay in LDS in the cache's own element type and are converted where they are read.  Needs word
// alignment: 16-bit rows whose strides are even and whose base is 4-byte aligned.
constexpr int TAIL_TILE_WORDS = 128 * 136, TAIL_RPT = 32;     // words per tile (keys, values); rows per thread
constexpr int TAIL_WIDE_LOADS = 8;                            // 16-byte loads a thread has in flight per tile

template <int DT> struct TailWord;
template <> struct TailWord<TQ_F32> {
  static constexpr int EPW = 1;
  static __device__ __forceinline__ void unpack(uint32_t w, float (&x)[2]) { x[0] = __uint_as_float(w); x[1] = 0.0f; }
};
template <> struct TailWord<TQ_BF16> {
  static constexpr int EPW = 2;
  static __device__ __forceinline__ void unpack(uint32_t w, float (&x)[2]) {
    x[0] = __uint_as_float(w << 16);
    x[1] = __uint_as_float(w & 0xffff0000u);
  }
};
template <> struct TailWord<TQ_F16> {
  static constexpr int EPW = 2;
  static __device__ __forceinline__ void unpack(uint32_t w, float (&x)[2]) {
    x[0] = f16_bits_to_f32((uint16_t)(w & 0xffffu));
    x[1] = f16_bits_to_f32((uint16_t)(w >> 16));
  }
};

// words of one row tile (keys, values): room for every exact row when that is less than the largest tile
// (W words per row: d for fp32 rows, d / 2 for 16-bit rows)
static int tail_tile_words(int W, int recent_rows, bool wide) {
  const int64_t ldw = wide ? W + 8 : W + 1;
  // (at least 4096 words: at the end the key tile holds the row slices' partial sums, [<= 8][4 heads][d])
  int64_t need = ((recent_rows + 15) / 16 * 16) * ldw;
  if (need < 4096) need = 4096;
  return (int)(need < TAIL_TILE_WORDS ? (need + 3) / 4 * 4 : TAIL_TILE_WORDS);
}
static size_t tail_words_smem(int d, int recent_rows, int tile_words) {
  return ((size_t)TAIL_GC * d + (size_t)TAIL_GC * recent_rows + 2 * TAIL_GC + 2 * (size_t)tile_words) * sizeof(float);
}

// KC = word columns per thread (2 only for fp32 rows of more than 512 channels).
// PAGED: the exact tokens are the newest min(seq_len, recent_rows) tokens of the sequence in a paged
// exact cache of 16-token blocks (rk / rv its base, ws_blk / ws_r / ws_h its block, token and head
// strides in words); token p of sequence b sits in slot p % 16 of block block_table[b][p / 16].
// Otherwise rk / rv are (B, recent_rows, H, d) rows with strides ws_b / ws_r / ws_h and recent_len valid rows.
struct TailArgs {
  const void* q;
  int Hq, Hkv, d;
  const uint32_t *rk, *rv;
  int recent_rows;
  int64_t ws_b, ws_r, ws_h;
  const int32_t* recent_len;
  const int32_t* block_table;
  int bt_stride;
  int max_pages, num_blocks;       // entries of a block-table row; blocks of the paged exact cache
  const int32_t* seq_lens;
  int64_t ws_blk;
  int wide;                        // rows and strides are 16-byte aligned: four words per load
  int tile_words;                  // LDS words of one row tile (tail_tile_words)
  float sm_scale;
  float* parts;
  int n_parts, part_index;
  int t_chunks;                    // workgroups that share the exact tokens of a (sequence, head group); chunk c writes part part_index + c
};

// (a device function: the stand-alone kernel and the launch that shares its grid with the query
// preparation both run it; h / b are the workgroup's KV head and sequence, gz = head group + number of head
// groups x token chunk, `sm` its LDS)
template <int DT, int KC, bool PAGED, bool WIDE>
__device__ __forceinline__ void exact_tail_words_body(const TailArgs& A, int h, int b, int gz, float* sm) {
  const void* __restrict__ q = A.q;
  const int Hq = A.Hq, Hkv = A.Hkv, d = A.d, recent_rows = A.recent_rows, bt_stride = A.bt_stride;
  const uint32_t* __restrict__ rk = A.rk;
  const uint32_t* __restrict__ rv = A.rv;
  const int64_t ws_b = A.ws_b, ws_r = A.ws_r, ws_h = A.ws_h, ws_blk = A.ws_blk;
  const int32_t* __restrict__ recent_len = A.recent_len;
  const int32_t* __restrict__ block_table = A.block_table;
  const int32_t* __restrict__ seq_lens = A.seq_lens;
  const float sm_scale = A.sm_scale;
  float* __restrict__ parts = A.parts;
  const int n_parts = A.n_parts;
  constexpr int GC = TAIL_GC, EPW = TailWord<DT>::EPW, RPT = TAIL_RPT / KC;
  const int G = Hq / Hkv, tid = threadIdx.x;
  const int n_gz = (G + GC - 1) / GC, chunk = gz / n_gz, g0 = (gz - chunk * n_gz) * GC;
  const int part_index = A.part_index + chunk;
  const int Gc = min(GC, G - g0);
  const int lane = tid & 63, wave = tid >> 6;
  const int seq = PAGED ? min(seq_lens[b], A.max_pages * TQ_PAGE_TOKENS) : 0;     // cut to the block table
  const int num_blocks = A.num_blocks;
  const int R_all = PAGED ? max(min(seq, recent_rows), 0) : (recent_len ? min(recent_len[b], recent_rows) : recent_rows);
  // this workgroup's share of the exact tokens (all of them with one chunk); it may be empty
  const int r_lo = (int)((int64_t)R_all * chunk / A.t_chunks), R = (int)((int64_t)R_all * (chunk + 1) / A.t_chunks) - r_lo;
  const int first = (PAGED ? seq - R_all : 0) + r_lo;   // position (row, when not paged) of the first exact token of the share
  const int32_t* bt = block_table + (PAGED ? (int64_t)b * bt_stride : 0);
  float* sq = sm;                                   // [d][GC]
  float* ss = sq + GC * d;                          // [recent_rows][GC] scores, then softmax weights
  float* sml = ss + GC * recent_rows;               // [GC][2]
  uint32_t* ktile = (uint32_t*)(sml + 2 * GC);      // [CH][W + 1] key rows of the chunk; at the end [TS][GC][d] partials
  uint32_t* vtile = ktile + A.tile_words;           // [CH][W + 1] value rows
  // words per row (a multiple of 32); leading dimension: odd, or (16-byte loads) W + 8, which keeps rows
  // 16-byte aligned and spreads the 8 tokens x 8 segments a wavefront reads in the score stage over all banks
  constexpr bool wide = WIDE;
  const int W = d / EPW, ldw = wide ? W + 8 : W + 1;
  const int TS = W < TAIL_THREADS ? TAIL_THREADS / W : 1;          // row slices
  const int QW = W >> 2, RP = TAIL_THREADS / QW;                   // wide: 4-word pieces per row, rows per round of loads
  const int wq = tid % QW, wr = tid / QW;                          // wide: this thread's piece and row slot
  const int CH = wide ? min(A.tile_words / ldw, TAIL_WIDE_LOADS * RP)
                      : min(A.tile_words / ldw, TS * RPT);         // rows per chunk
  const int cw0 = W < TAIL_THREADS ? tid % W : tid, ts = W < TAIL_THREADS ? tid / W : 0;
  const bool active = ts < TS;
  const int64_t base0 = (PAGED ? 0 : b * ws_b) + h * ws_h;
  // word offset of exact row `row` (< R) of this (sequence, head)
  auto row_base = [&](int row) -> int64_t {
    if (PAGED) {
      const int p = first + row;
      const int raw = bt[p >> 4];                       // an entry outside the cache is read as block 0
      return base0 + (int64_t)((unsigned)raw < (unsigned)num_blocks ? raw : 0) * ws_blk + (int64_t)(p & 15) * ws_r;
    }
    return base0 + (int64_t)(first + row) * ws_r;
  };
  // loads of rows c0 + ts, c0 + ts + TS, ... of this thread's columns, all issued before anything waits
  // (n >= 1: callers skip empty chunks, so the clamped row exists)
  auto request = [&](const uint32_t* src, int c0, int n, uint32_t (&reg)[KC][RPT]) {
    int64_t rb[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int t = ts + i * TS;
      rb[i] = row_base(c0 + (t < n ? t : 0));
    }
#pragma unroll
    for (int k = 0; k < KC; ++k) {
      const int cw = min(cw0 + TAIL_THREADS * k, W - 1);
#pragma unroll
      for (int i = 0; i < RPT; ++i) reg[k][i] = src[rb[i] + cw];
    }
  };
  auto deposit = [&](uint32_t* tile, int n, const uint32_t (&reg)[KC][RPT]) {
#pragma unroll
    for (int k = 0; k < KC; ++k) {
      const int cw = cw0 + TAIL_THREADS * k;
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        const int t = ts + i * TS;
        if (t < n && cw < W) tile[t * ldw + cw] = reg[k][i];
      }
    }
  };
  // the query first (it is the oldest request, so it can go to LDS while the rows are still on their way)
  constexpr int QPT = (GC * 768 + TAIL_THREADS - 1) / TAIL_THREADS;      // query elements per thread, d <= 768
  float qreg[QPT];
#pragma unroll
  for (int i = 0; i < QPT; ++i) {
    const int o = tid + i * TAIL_THREADS;
    qreg[i] = Elem<DT>::load(q, ((int64_t)b * Hq + h * G + g0) * d + min(o, Gc * d - 1));
  }
  auto deposit_query = [&]() {
#pragma unroll
    for (int i = 0; i < QPT; ++i) {
      const int o = tid + i * TAIL_THREADS;
      if (o < GC * d) {
        const int g = o / d, c = o - g * d;
        sq[c * GC + g] = g < Gc ? qreg[i] : 0.0f;
      }
    }
  };
  // the same with 16-byte pieces: round i takes rows wr + i RP; a round none of whose rows exists is skipped
  // (uniformly), a row that does not exist inside a live round re-reads the chunk's first row
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  // (the row offsets first, all of them - they hold the block-table loads of a paged cache -, and once for
  // keys and values: a table load between two row loads would have to wait for the row load before it)
  auto row_bases4 = [&](int c0, int n, int64_t (&rb)[TAIL_WIDE_LOADS]) {
#pragma unroll
    for (int i = 0; i < TAIL_WIDE_LOADS; ++i) {
      const int t = wr + i * RP;
      rb[i] = row_base(c0 + (t < n ? t : 0)) + 4 * wq;
    }
  };
  auto request4 = [&](const uint32_t* src, const int64_t (&rb)[TAIL_WIDE_LOADS], int n, u32x4_t (&reg)[TAIL_WIDE_LOADS]) {
#pragma unroll
    for (int i = 0; i < TAIL_WIDE_LOADS; ++i)
      if (i * RP < n) reg[i] = *(const u32x4_t*)(src + rb[i]);
  };
  auto deposit4 = [&](uint32_t* tile, int n, const u32x4_t (&reg)[TAIL_WIDE_LOADS]) {
#pragma unroll
    for (int i = 0; i < TAIL_WIDE_LOADS; ++i) {
      const int t = wr + i * RP;
      if (i * RP < n && t < n) *(u32x4_t*)(tile + t * ldw + 4 * wq) = reg[i];
    }
  };
  const int n_first = min(CH, R);
  if constexpr (wide) {
    if (wr < RP && n_first > 0) {
      u32x4_t kreg[TAIL_WIDE_LOADS], vreg[TAIL_WIDE_LOADS];
      int64_t rb[TAIL_WIDE_LOADS];
      row_bases4(0, n_first, rb);
      request4(rk, rb, n_first, kreg);
      request4(rv, rb, n_first, vreg);
      deposit_query();
      deposit4(ktile, n_first, kreg);
      deposit4(vtile, n_first, vreg);
    } else {
      deposit_query();
    }
  } else {
    if (active && n_first > 0) {
      uint32_t kreg[KC][RPT], vreg[KC][RPT];
      request(rk, 0, n_first, kreg);
      request(rv, 0, n_first, vreg);
      deposit_query();
      deposit(ktile, n_first, kreg);
      deposit(vtile, n_first, vreg);
    } else {
      deposit_query();
    }
  }
  __syncthreads();
  // scores: eight threads per token, each over every eighth word of the row, for the group's heads at once
  for (int c0 = 0; c0 < R; c0 += CH) {
    const int n = min(CH, R - c0);
    if (c0 > 0) {
      __syncthreads();
      if constexpr (wide) {
        if (wr < RP) {
          u32x4_t kreg[TAIL_WIDE_LOADS];
          int64_t rb[TAIL_WIDE_LOADS];
          row_bases4(c0, n, rb);
          request4(rk, rb, n, kreg);
          deposit4(ktile, n, kreg);
        }
      } else {
        if (active) {
          uint32_t kreg[KC][RPT];
          request(rk, c0, n, kreg);
          deposit(ktile, n, kreg);
        }
      }
      __syncthreads();
    }
    // (a thread takes two tokens per trip, 64 apart, against one read of the query values; one when the chunk
    // has no second token for anybody: the share of a workgroup that splits the exact tokens with others)
    const int seg = tid & 7;
    constexpr int TPT = TAIL_THREADS / 8;
    auto score_trip = [&](int t0, auto nt_tag) __attribute__((always_inline)) {
      constexpr int NT = decltype(nt_tag)::value;
      int t[NT];
      const uint32_t* row[NT];
      float a[NT][4];
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        t[u] = t0 + (tid >> 3) + u * TPT;
        row[u] = ktile + (t[u] < n ? t[u] : 0) * ldw;
        a[u][0] = a[u][1] = a[u][2] = a[u][3] = 0.0f;
      }
      for (int cw = seg; cw < W; cw += 8) {
        float x[NT][2];
#pragma unroll
        for (int u = 0; u < NT; ++u) TailWord<DT>::unpack(row[u][cw], x[u]);
#pragma unroll
        for (int e = 0; e < EPW; ++e) {
          const float4 q4 = *reinterpret_cast<const float4*>(sq + (cw * EPW + e) * GC);
#pragma unroll
          for (int u = 0; u < NT; ++u) {
            a[u][0] = fmaf(x[u][e], q4.x, a[u][0]);
            a[u][1] = fmaf(x[u][e], q4.y, a[u][1]);
            a[u][2] = fmaf(x[u][e], q4.z, a[u][2]);
            a[u][3] = fmaf(x[u][e], q4.w, a[u][3]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < NT; ++u) {
#pragma unroll
        for (int g = 0; g < 4; ++g) a[u][g] = lanes_sum_dpp<8>(a[u][g]);
        if (seg == 0 && t[u] < n)
          *reinterpret_cast<float4*>(ss + (c0 + t[u]) * GC) =
              make_float4(a[u][0] * sm_scale, a[u][1] * sm_scale, a[u][2] * sm_scale, a[u][3] * sm_scale);
      }
    };
    for (int t0 = 0; t0 < n; t0 += 2 * TPT) {                        // uniform trip count: the lane exchanges need every lane
      if (t0 + TPT < n) score_trip(t0, std::integral_constant<int, 2>{});
      else score_trip(t0, std::integral_constant<int, 1>{});
    }
  }
  __syncthreads();
  // softmax statistics and weights, a wavefront per query head
  for (int g = wave; g < GC; g += TAIL_WAVES) {
    float mx = NEG_BIG;
    for (int t = lane; t < R; t += 64) mx = fmaxf(mx, ss[t * GC + g]);
    mx = wave_max_fast(mx);
    float sum = 0.0f;
    for (int t = lane; t < R; t += 64) {
      float p = __expf(ss[t * GC + g] - mx);
      ss[t * GC + g] = p;
      sum += p;
    }
    sum = wave_sum_fast(sum);
    if (lane == 0) { sml[g * 2] = mx; sml[g * 2 + 1] = sum; }
  }
  __syncthreads();
  // values: a thread per word column and row slice
  float acc[KC][2][GC];
#pragma unroll
  for (int k = 0; k < KC; ++k)
#pragma unroll
    for (int e = 0; e < 2; ++e)
#pragma unroll
      for (int g = 0; g < GC; ++g) acc[k][e][g] = 0.0f;
  for (int c0 = 0; c0 < R; c0 += CH) {
    const int n = min(CH, R - c0);
    if (c0 > 0) {
      __syncthreads();
      if constexpr (wide) {
        if (wr < RP) {
          u32x4_t vreg[TAIL_WIDE_LOADS];
          int64_t rb[TAIL_WIDE_LOADS];
          row_bases4(c0, n, rb);
          request4(rv, rb, n, vreg);
          deposit4(vtile, n, vreg);
        }
      } else {
        if (active) {
          uint32_t vreg[KC][RPT];
          request(rv, c0, n, vreg);
          deposit(vtile, n, vreg);
        }
      }
      __syncthreads();
    }
    if (active) {
#pragma unroll
      for (int k = 0; k < KC; ++k) {
        const int cw = cw0 + TAIL_THREADS * k;
        if (cw < W) {
          for (int t = ts; t < n; t += TS) {
            float x[2];
            TailWord<DT>::unpack(vtile[t * ldw + cw], x);
            const float4 w4 = *reinterpret_cast<const float4*>(ss + (c0 + t) * GC);
#pragma unroll
            for (int e = 0; e < EPW; ++e) {
              acc[k][e][0] = fmaf(w4.x, x[e], acc[k][e][0]);
              acc[k][e][1] = fmaf(w4.y, x[e], acc[k][e][1]);
              acc[k][e][2] = fmaf(w4.z, x[e], acc[k][e][2]);
              acc[k][e][3] = fmaf(w4.w, x[e], acc[k][e][3]);
            }
          }
        }
      }
    }
  }
  float* ptile = (float*)ktile;                     // [TS][GC][d]: the key tile is no longer needed
  if (active) {
#pragma unroll
    for (int k = 0; k < KC; ++k) {
      const int cw = cw0 + TAIL_THREADS * k;
      if (cw < W)
#pragma unroll
        for (int e = 0; e < EPW; ++e)
#pragma unroll
          for (int g = 0; g < GC; ++g) ptile[(ts * GC + g) * d + cw * EPW + e] = acc[k][e][g];
    }
  }
  __syncthreads();
  for (int o = tid; o < Gc * d; o += TAIL_THREADS) {
    const int g = o / d, ch = o - g * d;
    float a = 0.0f;
    for (int s2 = 0; s2 < TS; ++s2) a += ptile[(s2 * GC + g) * d + ch];
    float* out = parts + (((int64_t)b * Hq + h * G + g0 + g) * n_parts + part_index) * (d + 2);
    if (ch == 0) { out[0] = sml[g * 2]; out[1] = sml[g * 2 + 1]; }
    out[2 + ch] = a;
  }
}

template <int DT, int KC, bool PAGED, bool WIDE>
__global__ void __launch_bounds__(TAIL_THREADS)
exact_tail_words_kernel(TailArgs A) {
  extern __shared__ __align__(16) float sm[];
  exact_tail_words_body<DT, KC, PAGED, WIDE>(A, blockIdx.x, blockIdx.y, blockIdx.z, sm);
}

// One launch for the two things a hybrid step does before its page kernel: the exact-tail workgroups
// (the first n_tail, so that the longer-running ones start first) and the query preparation of the
// matrix-core kernel.  They are independent of each other, both have 512 lanes, and together they are
// far fewer workgroups than the card has compute units, so the launch takes as long as the slower of
// the two instead of their sum plus a dispatch gap.
static_assert(TAIL_THREADS == PREP_COLS * PREP_SLICES, "the two roles share a workgroup size");
template <int PER, int DT, bool PAGED, bool PACKED>
__global__ void __launch_bounds__(TAIL_THREADS, 4)
prep_tail_kernel(TailArgs A, int n_tail, int B, int Gq, tq_layer ly, float* __restrict__ q_rot, float* __restrict__ q_sk,
                 float* __restrict__ q_stat, uint32_t* __restrict__ qa_pack, unsigned long long* __restrict__ arrivals,
                 int prep_gpw, int n_front, PagePrefetch pf, int g_tot, int head_rows) {
  extern __shared__ __align__(16) float sm[];
  const int id = blockIdx.x;
  if (id < n_tail) {
    const int per_z = A.Hkv * B;
    exact_tail_words_body<DT, 1, PAGED, true>(A, id % A.Hkv, (id / A.Hkv) % B, id / per_z, sm);
  } else if (id >= n_front) {      // behind the tail and the preparation: the page kernel's first pages, read ahead of it
    prefetch_pages_body<TAIL_THREADS>(pf, id - n_front);
  } else {
    const int words = ly.d / PREP_COLS, p = id - n_tail;
    // (arrivals: the arrival counters of the groups of query heads, zeroed for a page kernel that merges its splits itself)
    prep_query_body<PER, DT, PACKED>(A.q, Gq, prep_gpw, (int64_t)B * A.Hq, g_tot, ly, A.sm_scale, q_rot, q_sk, q_stat, qa_pack,
                                     arrivals, head_rows, p / words, p % words, sm);
  }
}

// The same for the head sizes of the wide-head page kernel with bf16 queries: the exact-tail workgroups and the rotation /
// operand packing on the matrix cores (rotate_mfma_body: the first 256 threads of its workgroups) in one launch.
template <int KPW, bool PAGED>
__global__ void __launch_bounds__(TAIL_THREADS)
rotate_tail_kernel(TailArgs A, int n_tail, int B, int n_tiles, tq_layer ly, float* __restrict__ q_rot,
                   float* __restrict__ q_sk, WidePack wp) {
  extern __shared__ __align__(16) float sm[];
  const int id = blockIdx.x;
  if (id < n_tail) {
    const int per_z = A.Hkv * B;
    exact_tail_words_body<TQ_BF16, 1, PAGED, true>(A, id % A.Hkv, (id / A.Hkv) % B, id / per_z, sm);
  } else if (threadIdx.x < ROTM_THREADS) {
    rotate_mfma_body<KPW>((const uint16_t*)A.q, (int64_t)B * A.Hq, n_tiles, ly, q_rot, q_sk, wp, id - n_tail, sm);
  }
}

// n_parts partials are merged per row; consecutive rows are part_stride partials apart.
// gridDim.y workgroups per row, each with an equal share of the row's channels (all of them repeat the
// small weight computation).  A thread owns a pair of channels and every S-th part (S = 256 / pairs
// subsets share the parts when a workgroup has fewer than 256 channel pairs); its first MERGE_CHUNK
// accumulator loads are issued before anything else, so that the (m, l) loads, the weights
// exp(m_s - M) and their reductions all run under one memory latency.
constexpr int MERGE_CHUNK = 16;
// Workgroups per row.  With few rows a workgroup's share of the partials (n_parts x d floats, written by
// compute units all over the card) arrives no faster than one compute unit can pull it in: 64 rows of
// 64 parts x 256 channels are merged 0.9 us sooner by four workgroups each (1.6 us with 65 parts).  The shares stay
// at 32 channel pairs or more, and no wider than there are parts to share among the subsets.
static int merge_row_groups(int64_t rows, int n_parts, int d) {
  const int np = d >> 1;
  int ny = 1;
  if ((np & (np - 1)) != 0 || np > 256 || opt_merge_row_groups.load(std::memory_order_relaxed) == 0) return 1;
  while (rows * ny * 2 <= 256 && np / (ny * 2) >= 32 && 256 / (np / (ny * 2)) <= n_parts) ny *= 2;
  return ny;
}
static size_t merge_smem(int n_parts, int d, int ny) {
  const int np = (d >> 1) / ny, S = np >= 256 ? 1 : 256 / np;
  return ((size_t)3 * n_parts + 8 + (size_t)S * (d / ny)) * sizeof(float);
}

__global__ void __launch_bounds__(256)
merge_kernel(const float* __restrict__ parts, int n_parts, int part_stride, int d, int dtype, void* __restrict__ out,
             int row_groups) {
  extern __shared__ float s_w[];                 // [n_parts] weights, [n_parts] m, [n_parts] l, [8] scratch, [S][dw] sums
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // (row_groups = gridDim.y, as an argument: it arrives with the others instead of through one more scalar load
  // of the launch's implicit data in front of the first accumulator loads)
  const int dw = d / row_groups, c0 = (int)blockIdx.y * dw;       // this workgroup's channels: c0 .. c0 + dw - 1
  const float* p = parts + row * part_stride * (int64_t)(d + 2);
  float* s_m = s_w + n_parts;
  float* s_l = s_m + n_parts;
  float* scratch = s_l + n_parts;
  float* s_sum = scratch + 8;
  const int np = dw >> 1;                                       // channel pairs of this workgroup
  const int S = np >= 256 ? 1 : 256 / np;                       // subsets of parts (dw is a multiple of 64)
  const int tps = 256 / S;                                      // threads per subset
  const int sub = tid / tps, pr = tid - sub * tps;
  typedef float f2 __attribute__((ext_vector_type(2)));
  // first chunk of this thread's accumulator loads (pair pr; parts sub, sub + S, ...), clamped in range
  f2 v[MERGE_CHUNK];
#pragma unroll
  for (int k = 0; k < MERGE_CHUNK; ++k) {
    const int sp = min(sub + k * S, n_parts - 1);
    v[k] = *(const f2*)(p + (int64_t)sp * (d + 2) + 2 + c0 + 2 * min(pr, np - 1));
  }
  float mm = NEG_BIG;
  for (int sp = tid; sp < n_parts; sp += blockDim.x) {
    const f2 ml = *(const f2*)(p + (int64_t)sp * (d + 2));
    s_m[sp] = ml[0];
    s_l[sp] = ml[1];
    if (ml[1] > 0.0f) mm = fmaxf(mm, ml[0]);
  }
  mm = wave_max_fast(mm);
  if (lane == 0) scratch[wave] = mm;
  __syncthreads();
  mm = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
  float ll = 0.0f;
  for (int sp = tid; sp < n_parts; sp += blockDim.x) {
    const float w = s_l[sp] > 0.0f ? __expf(s_m[sp] - mm) : 0.0f;
    s_w[sp] = w;
    ll += w * s_l[sp];
  }
  ll = wave_sum_fast(ll);
  if (lane == 0) scratch[4 + wave] = ll;
  __syncthreads();
  ll = scratch[4] + scratch[5] + scratch[6] + scratch[7];
  const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;
  // every part was written by its producer (empty ones as zeros), so the loads need no guard
  for (int p0 = pr; p0 < np; p0 += tps) {
    f2 acc = {0.0f, 0.0f};
    for (int k0 = 0; sub + k0 * S < n_parts; k0 += MERGE_CHUNK) {
      if (k0 > 0 || p0 != pr) {
#pragma unroll
        for (int k = 0; k < MERGE_CHUNK; ++k) {
          const int sp = min(sub + (k0 + k) * S, n_parts - 1);
          v[k] = *(const f2*)(p + (int64_t)sp * (d + 2) + 2 + c0 + 2 * p0);
        }
      }
#pragma unroll
      for (int k = 0; k < MERGE_CHUNK; ++k) {
        const int sp = sub + (k0 + k) * S;
        const float w = sp < n_parts ? s_w[sp] : 0.0f;
        acc[0] = fmaf(w, v[k][0], acc[0]);
        acc[1] = fmaf(w, v[k][1], acc[1]);
      }
    }
    s_sum[sub * dw + 2 * p0] = acc[0];
    s_sum[sub * dw + 2 * p0 + 1] = acc[1];
  }
  __syncthreads();
  for (int ch = tid; ch < dw; ch += blockDim.x) {
    float aa = 0.0f;
    for (int q = 0; q < S; ++q) aa += s_sum[q * dw + ch];
    store_from_f32(out, row * d + c0 + ch, aa * inv, dtype);
  }
}

}  // namespace tq

using namespace tq;

namespace tq {
int launch_rotate_query(const void* q, int dtype, int64_t rows, const tq_layer* layer, float* q_rot, float* q_sk,
                        float* q_stat, uint32_t* qa_pack, int G, float sm_scale, hipStream_t st, bool q_rot_unused,
                        unsigned long long* arrivals, const PagePrefetch* prefetch, int g_tot, const WidePack* wide);
bool prep_on_matrix_cores(const void* q, int dtype, int64_t rows, const tq_layer* layer, int G, int g_tot);
bool rotate_on_matrix_cores(const void* q, int dtype, int64_t rows, const tq_layer* layer, const WidePack* wide);
}  // namespace tq

static size_t parts_floats(int B, int Hq, int d, int n_parts) { return (size_t)B * Hq * n_parts * (d + 2); }
// arrival counters of the in-launch merge: one 64-bit word per group of query heads, at most B * Hq groups
static size_t counter_words(int B, int Hq) { return (size_t)B * Hq; }

// ---- knobs (tq_set_option) -----------------------------------------------------------------------------
namespace tq {
std::atomic<int> opt_append_parts{3};
std::atomic<int> opt_fp6_centroids{1};
std::atomic<int> opt_merge_in_kernel{1};
std::atomic<int> opt_page_pairs{1};
std::atomic<int> opt_narrow_rows{1};
std::atomic<int> opt_wide_workgroups{1};
std::atomic<int> opt_split_skew{1};
std::atomic<int> opt_merge_row_groups{1};
std::atomic<int> opt_tail_chunks{1};
std::atomic<int> opt_prefetch_trips{-1};
std::atomic<int> opt_prep_mfma{1};
std::atomic<int> opt_sequence_walkers{-1};
std::atomic<int> opt_prep_words{-1};
std::atomic<int> opt_append_small{-1};
std::atomic<int> opt_wide_heads{1};
std::atomic<int> opt_wide_prepack{1};
}  // namespace tq

extern "C" int tq_set_option(const char* name, int64_t value) {
  if (!name) return TQ_ENULL;
  if (!std::strcmp(name, "wide_workgroups")) { opt_wide_workgroups.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "split_skew")) {
    if (value < 0 || value > 8) return TQ_EINVAL;
    opt_split_skew.store((int)value);
    return TQ_OK;
  }
  if (!std::strcmp(name, "prefetch_trips")) {
    if (value < -1 || value > 64) return TQ_EINVAL;
    opt_prefetch_trips.store((int)value);
    return TQ_OK;
  }
  if (!std::strcmp(name, "prep_mfma")) {
    if (value < 0 || value > 2) return TQ_EINVAL;
    opt_prep_mfma.store((int)value);
    return TQ_OK;
  }
  if (!std::strcmp(name, "tail_chunks")) { opt_tail_chunks.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "merge_row_groups")) { opt_merge_row_groups.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "wide_prepack")) { opt_wide_prepack.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "wide_heads")) {
    if (value < 0 || value > 2) return TQ_EINVAL;
    opt_wide_heads.store((int)value);
    return TQ_OK;
  }
  if (!std::strcmp(name, "append_small")) {
    if (value < -1 || value > (1 << 24)) return TQ_EINVAL;
    opt_append_small.store((int)value);
    return TQ_OK;
  }
  if (!std::strcmp(name, "prep_words")) {
    if (value < -1 || value > 1) return TQ_EINVAL;
    opt_prep_words.store((int)value);
    return TQ_OK;
  }
  if (!std::strcmp(name, "sequence_walkers")) {
    if (value != -1 && value != 1 && value != 2 && value != 4) return TQ_EINVAL;
    opt_sequence_walkers.store((int)value);
    return TQ_OK;
  }
  if (!std::strcmp(name, "narrow_rows")) { opt_narrow_rows.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "page_pairs")) { opt_page_pairs.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "merge_in_kernel")) { opt_merge_in_kernel.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "fp6_centroids")) { opt_fp6_centroids.store(value != 0); return TQ_OK; }
  if (!std::strcmp(name, "append_parts")) {
    if (value < 1 || value > 3) return TQ_EINVAL;
    opt_append_parts.store((int)value);
    return TQ_OK;
  }
  return TQ_EINVAL;
}

extern "C" int tq_decode_page_kernel(const tq_layer* layer, const tq_page_layout* layout) {
  if (!layer || !layout) return TQ_ENULL;
  if (layer->Pi_colsum && layer->S_colsum && decode_mfma_has_kernel(*layer, *layout)) return 1;
  return decode_wide_has_kernel(*layer, *layout) ? 2 : 0;
}

extern "C" size_t tq_decode_workspace_bytes(int B, int Hq, int d, int n_split) {
  if (B <= 0 || Hq <= 0 || d <= 0 || n_split <= 0) return 0;
  // partials for n_split history splits + up to TAIL_MAX_CHUNKS of the exact tail, then q_rot, q_sk, 4 statistics per query row and
  // the packed query operands of the matrix-core kernel (sized for the largest kernel: 9 term planes, 8 heads)
  return (parts_floats(B, Hq, d, n_split + TAIL_MAX_CHUNKS) + (size_t)2 * B * Hq * d + (size_t)4 * B * Hq) * sizeof(float) +
         counter_words(B, Hq) * sizeof(unsigned long long) + decode_mfma_pack_words(B, Hq, d) * sizeof(uint32_t);
}

extern "C" int tq_decode_merge(const float* parts, int64_t rows, int n_parts, int d, int dtype, void* out,
                               void* stream) {
  if (!parts || !out) return TQ_ENULL;
  if (rows < 0 || n_parts <= 0 || d <= 0 || dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  if (rows == 0) return TQ_OK;
  const int ny = merge_row_groups(rows, n_parts, d);
  merge_kernel<<<dim3((unsigned)rows, ny), dim3(256), merge_smem(n_parts, d, ny), (hipStream_t)stream>>>(
      parts, n_parts, n_parts, d, dtype, out, ny);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

namespace {
// The exact tokens of a step.  Rows: (B, rows, H, d) tensors with element strides s_b / s_r / s_h and `len`
// valid rows per sequence.  Paged: the newest min(seq_len, rows) tokens of every sequence, read in place
// from a paged exact cache (block stride s_blk, token stride s_r, head stride s_h) through the step's
// block table; the compressed pages then cover the tokens before them.
struct TailSpec {
  const void* k = nullptr;
  const void* v = nullptr;
  int rows = 0;
  int64_t s_b = 0, s_r = 0, s_h = 0, s_blk = 0;
  const int32_t* len = nullptr;
  bool paged = false;
};
}  // namespace

static int decode_stages(const void* q, int dtype, int B, int Hq, int Hkv, const uint8_t* pool, int64_t num_pages,
                         const int32_t* block_table, int bt_stride, const int32_t* seq_lens, float sm_scale,
                         const tq_layer* layer, const tq_page_layout* layout, const TailSpec& ts, void* out,
                         void* workspace, int n_split, int stages, void* stream) {
  const void *recent_k = ts.k, *recent_v = ts.v;
  const int recent_rows = ts.rows;
  const int64_t rs_b = ts.s_b, rs_r = ts.s_r, rs_h = ts.s_h;
  const int32_t* recent_len = ts.len;
  if (!q || !pool || !block_table || !seq_lens || !layer || !layout || !out || !workspace) return TQ_ENULL;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || n_split <= 0 || num_pages <= 0) return TQ_EINVAL;
  if (B > 65535 || Hkv > 65535) return TQ_EUNSUPPORTED;
  // bt_stride > 0: a table row per sequence, that many entries; 0: one row shared by all sequences, length
  // unknown; < 0: one shared row of -bt_stride entries.  Lengths beyond the row are cut to it in the kernels.
  const int k_max_rows = 0x7fffffff / TQ_PAGE_TOKENS;
  const int max_pages = bt_stride == 0 ? k_max_rows : (bt_stride > 0 ? bt_stride : -bt_stride) < k_max_rows
                                                          ? (bt_stride > 0 ? bt_stride : -bt_stride) : k_max_rows;
  if (bt_stride < 0) bt_stride = 0;
  const int pool_pages = (int)(num_pages < 0x7fffffff ? num_pages : 0x7fffffff);
  const int d = layer->d, G = Hq / Hkv;
  if (d != layout->d || layer->mse_bits != layout->mse_bits) return TQ_EINVAL;
  if (d < 64 || d > 768 || (d & 63) || G > G_LIMIT) return TQ_EUNSUPPORTED;
  if (layout->value_bits != 2 && layout->value_bits != 4 && layout->value_bits != 8) return TQ_EUNSUPPORTED;
  const bool tail = recent_k != nullptr && recent_rows > 0;
  if (tail && !recent_v) return TQ_ENULL;
  if (tail && recent_rows > 1024) return TQ_EUNSUPPORTED;
  const int len_sub = tail && ts.paged ? recent_rows : 0;       // newest tokens the pages do not cover
  hipStream_t st = (hipStream_t)stream;
  // the matrix-core kernel takes up to 8 query heads per group: a KV head with more is served by kv_div
  // groups of Gq = ceil(G / kv_div) heads, the last one of fewer when G does not divide (11 heads: 6 + 5)
  const int kv_div = (G + 7) / 8;
  const int Gq = (G + kv_div - 1) / kv_div;
  if ((int64_t)Hkv * kv_div > 65535) return TQ_EUNSUPPORTED;      // (head groups are a grid dimension)
  // (the same table the launchers dispatch over: a shape without an instantiation keeps its split count and takes
  // the general kernel's preparation, which writes the fp32 rotated / sketched queries that kernel reads)
  const bool mfma_shape = kv_div && layer->Pi_colsum && layer->S_colsum && decode_mfma_has_kernel(*layer, *layout);
  // Short contexts with at most four query heads per group run workgroups of eight wavefronts on half as many
  // splits (the same number of wavefronts): everything below - partials, merge, the workspace's carving - then
  // uses the halved count, for every stage of the step alike.
  const bool wide_wg = mfma_shape && layout->key_lane_major && decode_mfma_wide_workgroups(d, Gq, n_split, max_pages);
  if (wide_wg) n_split /= 2;
  if (dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  // the exact tail as 32-bit words: always for fp32, for 16-bit rows when they are word-aligned
  const int epw = dtype == TQ_F32 ? 1 : 2;
  const bool words = epw == 1 || (((((uintptr_t)recent_k | (uintptr_t)recent_v) & 3) == 0) &&
                                  !((rs_b | rs_r | rs_h | ts.s_blk) & 1));
  // Workgroups per (sequence, KV head, group of TAIL_GC query heads) of the exact tail, each with a share of the
  // exact tokens and a partial of its own.  One such workgroup pulls 2 x recent_rows rows into one compute unit
  // and is the longest-running part of its launch; with few of them and a merge kernel behind (many splits - the
  // in-launch merge takes exactly one partial of the tail) up to TAIL_MAX_CHUNKS share the rows
  // (4 x 131072, 16 q / 2 KV heads, 128 exact tokens: 16 -> 64 workgroups).
  int t_chunks = 1;
  if (tail && words && n_split > MERGE_IN_KERNEL_MAX_SPLITS && opt_tail_chunks.load(std::memory_order_relaxed) != 0) {
    const int64_t groups = (int64_t)Hkv * B * ((G + TAIL_GC - 1) / TAIL_GC);
    while (t_chunks < TAIL_MAX_CHUNKS && groups * t_chunks * 2 <= 128 && recent_rows / (t_chunks * 2) >= 16) t_chunks *= 2;
  }
  const int n_parts = n_split + t_chunks;
  float* parts = (float*)workspace;
  float* q_rot = parts + parts_floats(B, Hq, d, n_parts);
  float* q_sk = q_rot + (size_t)B * Hq * d;
  float* q_stat = q_sk + (size_t)B * Hq * d;
  unsigned long long* arrivals = (unsigned long long*)(q_stat + (size_t)4 * B * Hq);    // 8-byte aligned: every term above is even
  uint32_t* qa_pack = (uint32_t*)(arrivals + counter_words(B, Hq));
  // Head sizes of the wide-head page kernel: the rotation launch also packs the kernel's query operands (one copy per
  // group of heads, instead of one per page-kernel workgroup) and writes the row statistics.  All stages of a step
  // decide alike, from the layer, the layout and the options.
  WidePack wide_pre;
  if (!mfma_shape && kv_div && decode_wide_has_kernel(*layer, *layout) && layer->Pi_colsum && layer->S_colsum &&
      opt_wide_prepack.load(std::memory_order_relaxed) != 0 && decode_wide_term_planes(*layer) > 0 &&
      (size_t)B * Hkv * kv_div * decode_wide_term_planes(*layer) * 2 * wide_qa_stride(d) + 4 <= decode_mfma_pack_words(B, Hq, d)) {
    wide_pre.qa = (uint32_t*)(((uintptr_t)qa_pack + 15) & ~(uintptr_t)15);      // (16-byte pieces are fetched and stored)
    wide_pre.q_stat = q_stat;
    wide_pre.Hq = Hq; wide_pre.Hkv = Hkv; wide_pre.kv_div = kv_div; wide_pre.ntp = decode_wide_term_planes(*layer);
    wide_pre.sm_scale = sm_scale;
  }

  if (tail && ts.paged && !words) return TQ_EUNSUPPORTED;       // a paged exact cache has to be word-aligned
  TailArgs ta;
  ta.q = q; ta.Hq = Hq; ta.Hkv = Hkv; ta.d = d;
  ta.rk = (const uint32_t*)recent_k; ta.rv = (const uint32_t*)recent_v; ta.recent_rows = recent_rows;
  ta.ws_b = rs_b / epw; ta.ws_r = rs_r / epw; ta.ws_h = rs_h / epw; ta.recent_len = recent_len;
  ta.block_table = block_table; ta.bt_stride = bt_stride; ta.seq_lens = seq_lens; ta.ws_blk = ts.s_blk / epw;
  // 16-byte pieces when every row starts on a 16-byte boundary and a row's pieces fit the workgroup
  ta.wide = words && ((((uintptr_t)recent_k | (uintptr_t)recent_v) & 15) == 0) &&
            !((ta.ws_b | ta.ws_r | ta.ws_h | ta.ws_blk) & 3) && (d / epw) / 4 <= TAIL_THREADS;
  ta.tile_words = tail_tile_words(d / epw, recent_rows, ta.wide != 0);
  ta.max_pages = max_pages; ta.num_blocks = pool_pages;       // the exact cache shares the pool's block numbers
  ta.sm_scale = sm_scale; ta.parts = parts; ta.n_parts = n_parts; ta.part_index = n_split;
  ta.t_chunks = t_chunks;
  const int n_tail = Hkv * B * ((G + TAIL_GC - 1) / TAIL_GC) * t_chunks;
  bool tail_done = false;

  // A whole compressed-only step with few context splits: the workgroup that finishes last among the splits of a
  // (sequence, group of query heads) merges them inside the page kernel's launch, and no merge kernel follows
  // (with many splits that workgroup would read more than the separate launch costs).  The preparation kernel
  // zeroes the arrival counters of its groups.
  FusedMerge fm;
  if (stages == 7 && mfma_shape && n_split <= MERGE_IN_KERNEL_MAX_SPLITS && opt_merge_in_kernel.load()) {
    fm.out = out;
    fm.out_dtype = dtype;
    fm.counters = arrivals;
    fm.n_extra = tail ? 1 : 0;          // the exact tail's partial, written by an earlier launch of this step
  }
  if (stages & 1) {
    if (!layer->Pi || !layer->PiT || !layer->S || !layer->ST || !layer->centroids) return TQ_ENULL;
    // Workgroups added to the preparation launch read the first pages of every page-kernel workgroup's range
    // ahead of it (the preparation leaves most of the card idle): prefetch_trips trips of each block walker.
    PagePrefetch pf;
    // By default (-1) only at head_dim 256: there the read-ahead takes 1.5 us off the page kernel and adds 0.7 - 1.1 us to the
    // preparation launch (4 x 131072: step 54.8 -> 54.0 us); at head_dim 128 / 64 it moves as much time as it saves
    // (16 x 8192: page kernel 33.1 -> 31.4 us, step 38.1 -> 38.7 us; 64 x 2048: step 35.3 -> 36.4 us).
    const int pf_opt = opt_prefetch_trips.load(std::memory_order_relaxed);
    const int pf_trips = mfma_shape ? (pf_opt < 0 ? (d == 256 ? 1 : 0) : pf_opt) : 0;
    if (pf_trips > 0 && (int64_t)n_split * Hkv * kv_div * B <= 4096) {
      decode_mfma_plan(pf, d, B, Hkv * kv_div, kv_div, n_split, wide_wg);
      pf.pool = pool; pf.block_table = block_table; pf.seq_lens = seq_lens;
      pf.bt_stride = bt_stride; pf.max_pages = max_pages; pf.num_pages = pool_pages; pf.len_sub = len_sub;
      pf.page_bytes = (uint32_t)layout->page_bytes;
      pf.fetch_bytes = pf.page_bytes;       // (keys and norms alone, half the bytes, measured the same)
      pf.page_stride = (uint32_t)((int64_t)Hkv * layout->page_bytes);
      pf.blocks = pf_trips * pf.ngrp;
    }
    // (in the launch shared with the tail a compute unit holds two workgroups: beyond that the preparation
    // workgroups take several groups of heads each, see prep_query_body)
    // (groups of unequal size - the heads of a KV head do not divide into kv_div groups - take one workgroup each)
    const int g_tot = kv_div > 1 && G % kv_div ? G : 0;
    const int prep_gpw = g_tot ? 1 : prep_groups_per_workgroup(Gq, n_tail + (int64_t)(B * Hq / Gq) * (d / PREP_COLS),
                                                               2 * (int64_t)device_compute_units());
    const int prep_rows = Gq * prep_gpw;                          // query rows of a preparation workgroup
    const int n_prep = (g_tot ? B * Hkv * kv_div : (B * Hq + prep_rows - 1) / prep_rows) * (d / PREP_COLS);
    // Whole hybrid step on the matrix-core path: the exact tail shares the preparation's launch (the tail
    // workgroups first, so that the longer-running ones start first).  The kernel is built for 128 registers
    // per lane and the tail's LDS is sized by the rows it holds, so two workgroups fit a compute unit; with more
    // workgroups than that the rest follow as slots free up, which still measured faster than a launch each
    // (16 x 8192: 48.9 -> 45.2 us per step, 32 x 32768: 223.6 -> 221.5 us).
    size_t fsm = tail_words_smem(d, recent_rows, ta.tile_words);
    if (prep_smem_bytes(prep_rows, d) > fsm) fsm = prep_smem_bytes(prep_rows, d);
    // ... unless the tail's tiles leave room for one workgroup per compute unit only (head_dim 256 with 128 exact
    // tokens: 139 KB) and the grid is larger than the card: the preparation workgroups would queue behind that
    // LDS size too (128 x 2048, 16 q / 2 KV heads: 109.7 us per step fused, 88.1 as two launches)
    const bool one_per_unit = fsm > (size_t)80 * 1024;
    // ... or the preparation alone is more than the card holds at once and can run on the matrix cores, which the
    // shared launch (vector-ALU preparation body) cannot: then a launch each
    const bool mfma_prep_ahead = mfma_shape && n_prep > 2 * device_compute_units() &&
                                 prep_on_matrix_cores(q, dtype, (int64_t)B * Hq, layer, Gq, g_tot);
    if (tail && ta.wide && mfma_shape && stages == 7 && !mfma_prep_ahead &&
        !(one_per_unit && n_tail + n_prep > device_compute_units())) {
#define TQ_LAUNCH_PT(PER, DT, PAGED)                                                                                 \
  {                                                                                                                  \
    auto kern = prep_gpw > 1 ? prep_tail_kernel<PER, DT, PAGED, true> : prep_tail_kernel<PER, DT, PAGED, false>;     \
    if (fsm > 48 * 1024) {                                                                                           \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)fsm);   \
      if (e != hipSuccess) return (int)e;                                                                            \
    }                                                                                                                \
    pf.front = n_tail + n_prep;                                                                                      \
    if (pf.front > 2 * device_compute_units()) pf.blocks = 0;                                                        \
    kern<<<dim3((unsigned)(n_tail + n_prep + (pf.blocks > 0 ? pf.n_wg : 0))), dim3(TAIL_THREADS), fsm, st>>>(        \
        ta, n_tail, B, Gq, *layer, q_rot, q_sk, q_stat, qa_pack, fm.counters, prep_gpw, n_tail + n_prep, pf, g_tot, \
        decode_mfma_head_rows(d, Gq));                                                                               \
  }
#define TQ_LAUNCH_PT_DT(PER, PAGED)                                \
  {                                                                \
    if (dtype == TQ_BF16) TQ_LAUNCH_PT(PER, TQ_BF16, PAGED)        \
    else if (dtype == TQ_F16) TQ_LAUNCH_PT(PER, TQ_F16, PAGED)     \
    else TQ_LAUNCH_PT(PER, TQ_F32, PAGED)                          \
  }
      if (d == 64) {
        if (ts.paged) TQ_LAUNCH_PT_DT(4, true)
        else TQ_LAUNCH_PT_DT(4, false)
      } else if (d == 128) {
        if (ts.paged) TQ_LAUNCH_PT_DT(8, true)
        else TQ_LAUNCH_PT_DT(8, false)
      } else {
        if (ts.paged) TQ_LAUNCH_PT_DT(16, true)
        else TQ_LAUNCH_PT_DT(16, false)
      }
#undef TQ_LAUNCH_PT_DT
#undef TQ_LAUNCH_PT
      TQ_CHECK_LAUNCH();
      tail_done = true;
    } else if (tail && ta.wide && stages == 7 && dtype == TQ_BF16 && (d == 512 || d == 576) && static_cast<int64_t>(n_tail) <= 4 * device_compute_units() &&
               rotate_on_matrix_cores(q, dtype, (int64_t)B * Hq, layer, wide_pre.qa ? &wide_pre : nullptr)) {
      // Hybrid step at the head sizes of latent attention: the exact tail shares the launch of the rotation
      // (16 x 8192 at head_dim 576: one launch of 13 us instead of 10 + 13)
      const int n_tiles = (B * Hq + 15) / 16, pair_rounds = (2 * (d / ROT_COLS) + 7) / 8;
      size_t fsm = tail_words_smem(d, recent_rows, ta.tile_words);
      if ((size_t)rotate_mfma_smem_floats() * sizeof(float) > fsm) fsm = (size_t)rotate_mfma_smem_floats() * sizeof(float);
#define TQ_LAUNCH_RT(KPW, PAGED)                                                                                     \
  {                                                                                                                  \
    auto kern = rotate_tail_kernel<KPW, PAGED>;                                                                      \
    if (fsm > 48 * 1024) {                                                                                           \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)fsm);   \
      if (e != hipSuccess) return (int)e;                                                                            \
    }                                                                                                                \
    kern<<<dim3((unsigned)(n_tail + 8 * pair_rounds * n_tiles)), dim3(TAIL_THREADS), fsm, st>>>(                     \
        ta, n_tail, B, n_tiles, *layer, q_rot, q_sk, wide_pre);                                                      \
  }
      if (d == 576) {
        if (ts.paged) TQ_LAUNCH_RT(9, true)
        else TQ_LAUNCH_RT(9, false)
      } else {
        if (ts.paged) TQ_LAUNCH_RT(8, true)
        else TQ_LAUNCH_RT(8, false)
      }
#undef TQ_LAUNCH_RT
      TQ_CHECK_LAUNCH();
      tail_done = true;
    } else {
      int rc = launch_rotate_query(q, dtype, (int64_t)B * Hq, layer, q_rot, q_sk, q_stat,
                                   mfma_shape ? qa_pack : nullptr, mfma_shape ? Gq : G, sm_scale, st, mfma_shape,
                                   fm.counters, &pf, mfma_shape ? g_tot : 0, wide_pre.qa ? &wide_pre : nullptr);
      if (rc) return rc;
    }
  }
  if (!(stages & 6)) return TQ_OK;

  // the exact tail's partial first (it depends on nothing the page kernel does), so that a page kernel that merges
  // its splits itself finds it written
  if (tail && (stages & 2) && !tail_done) {
    const dim3 tgrid(Hkv, B, ((G + TAIL_GC - 1) / TAIL_GC) * (words ? t_chunks : 1));
    size_t tsm = words ? tail_words_smem(d, recent_rows, ta.tile_words) : tail_smem(d, recent_rows);
#define TQ_LAUNCH_TAIL(KERN, ...)                                                                                    \
  {                                                                                                                  \
    auto kern = KERN;                                                                                                \
    if (tsm > 48 * 1024) {                                                                                           \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)tsm);   \
      if (e != hipSuccess) return (int)e;                                                                            \
    }                                                                                                                \
    kern<<<tgrid, dim3(TAIL_THREADS), tsm, st>>>(__VA_ARGS__);                                                       \
  }
#define TQ_TAIL_ROWS_ARGS q, Hq, Hkv, d, recent_k, recent_v, recent_rows, rs_b, rs_r, rs_h, recent_len, sm_scale, parts, n_parts, n_split
#define TQ_TAIL_WORD_ARGS ta
#define TQ_TAIL_WORDS(PAGED, WIDE)                                                                                   \
  {                                                                                                                  \
    if (dtype == TQ_BF16) TQ_LAUNCH_TAIL((exact_tail_words_kernel<TQ_BF16, 1, PAGED, WIDE>), TQ_TAIL_WORD_ARGS)      \
    else if (dtype == TQ_F16) TQ_LAUNCH_TAIL((exact_tail_words_kernel<TQ_F16, 1, PAGED, WIDE>), TQ_TAIL_WORD_ARGS)   \
    else if (d <= TAIL_THREADS) TQ_LAUNCH_TAIL((exact_tail_words_kernel<TQ_F32, 1, PAGED, WIDE>), TQ_TAIL_WORD_ARGS) \
    else TQ_LAUNCH_TAIL((exact_tail_words_kernel<TQ_F32, 2, PAGED, WIDE>), TQ_TAIL_WORD_ARGS)                        \
  }
    if (words) {
      if (ts.paged) {
        if (ta.wide) TQ_TAIL_WORDS(true, true)
        else TQ_TAIL_WORDS(true, false)
      } else {
        if (ta.wide) TQ_TAIL_WORDS(false, true)
        else TQ_TAIL_WORDS(false, false)
      }
    } else {      // 16-bit rows that are not word-aligned
      if (dtype == TQ_BF16) TQ_LAUNCH_TAIL(exact_tail_kernel<TQ_BF16>, TQ_TAIL_ROWS_ARGS)
      else TQ_LAUNCH_TAIL(exact_tail_kernel<TQ_F16>, TQ_TAIL_ROWS_ARGS)
    }
#undef TQ_TAIL_WORDS
#undef TQ_TAIL_WORD_ARGS
#undef TQ_TAIL_ROWS_ARGS
#undef TQ_LAUNCH_TAIL
    TQ_CHECK_LAUNCH();
  }
  int mf = TQ_EUNSUPPORTED;
  if (stages & 2)
    mf = mfma_shape ? launch_decode_mfma(qa_pack, q_stat, B, Hq, Hkv * kv_div, kv_div, pool, block_table, bt_stride,
                                         seq_lens, sm_scale, *layer, *layout, parts, n_parts, n_split, len_sub,
                                         max_pages, pool_pages, fm, wide_wg, st)
                    : TQ_EUNSUPPORTED;
  if (mf > 0) return mf;
  if (mf == TQ_OK && fm.out != nullptr) return TQ_OK;         // merged in the launch
  // head sizes above 256: the matrix-core kernel that works on a block per workgroup
  if ((stages & 2) && mf == TQ_EUNSUPPORTED) {
    mf = launch_decode_wide(q_rot, q_sk, B, Hq, Hkv, pool, block_table, bt_stride, seq_lens, sm_scale, *layer, *layout,
                            parts, n_parts, n_split, len_sub, max_pages, pool_pages, wide_pre, st);
    if (mf > 0) return mf;
  }
  if ((stages & 2) && mf == TQ_EUNSUPPORTED) {      // no matrix-core kernel for this shape: general kernel
    if (dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
    // (more than G_MAX query heads per KV head: groups of equal size, a workgroup each)
    const int head_groups = (G + G_MAX - 1) / G_MAX, g_per = (G + head_groups - 1) / head_groups;
    if ((int64_t)Hkv * head_groups > 65535) return TQ_EUNSUPPORTED;
    const int gp4 = (g_per + 3) / 4, gp = 4 * gp4;      // query heads rounded up to a multiple of 4
    const int tg = d < GEN_THREADS ? GEN_THREADS / d : 1;
    const size_t work = (size_t)gp * (GEN_CHUNK > tg * d ? GEN_CHUNK : tg * d);    // weights, then slice partials
    const size_t smem = ((size_t)2 * d * gp + 32 + work) * sizeof(float);
    dim3 grid(n_split, Hkv * head_groups, B), block(GEN_THREADS);
    // an armed pair of timing events goes to this kernel's dispatch as it would to the matrix-core kernel's
    hipEvent_t t_start = nullptr, t_stop = nullptr;
    const bool timed = take_time_hook(0, t_start, t_stop);
#define TQ_LAUNCH_DEC(VB, GP4)                                                                            \
  {                                                                                                       \
    auto kern = decode_pages_kernel<VB, GP4>;                                                             \
    if (smem > 48 * 1024) {                                                                               \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
      if (e != hipSuccess) return (int)e;                                                                 \
    }                                                                                                     \
    if (timed)                                                                                            \
      hipExtLaunchKernelGGL(kern, grid, block, smem, st, t_start, t_stop, 0, q_rot, q_sk, Hq, Hkv, pool, block_table,  \
                            bt_stride, seq_lens, sm_scale, *layer, *layout, parts, n_parts, n_split, len_sub,          \
                            max_pages, pool_pages, head_groups);                                                         \
    else                                                                                                  \
      kern<<<grid, block, smem, st>>>(q_rot, q_sk, Hq, Hkv, pool, block_table, bt_stride, seq_lens, sm_scale, *layer,  \
                                      *layout, parts, n_parts, n_split, len_sub, max_pages, pool_pages, head_groups); \
  }
#define TQ_LAUNCH_DEC_G(VB)                                                      \
  {                                                                              \
    if (gp4 == 1) TQ_LAUNCH_DEC(VB, 1)                                           \
    else if (gp4 == 2) TQ_LAUNCH_DEC(VB, 2)                                      \
    else if (gp4 == 3) TQ_LAUNCH_DEC(VB, 3)                                      \
    else TQ_LAUNCH_DEC(VB, 4)                                                    \
  }
    if (layout->value_bits == 2) TQ_LAUNCH_DEC_G(2)
    else if (layout->value_bits == 4) TQ_LAUNCH_DEC_G(4)
    else TQ_LAUNCH_DEC_G(8)
#undef TQ_LAUNCH_DEC_G
#undef TQ_LAUNCH_DEC
  TQ_CHECK_LAUNCH();
  }

  if (!(stages & 4)) return TQ_OK;
  // without a tail the merge simply reads one part fewer
  const int merged = tail ? n_parts : n_split, ny = merge_row_groups((int64_t)B * Hq, merged, d);
  merge_kernel<<<dim3((unsigned)(B * Hq), ny), dim3(256), merge_smem(n_parts, d, ny), st>>>(
      parts, merged, n_parts, d, dtype, out, ny);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

extern "C" int tq_decode_attn_paged_stages(const void* q, int dtype, int B, int Hq, int Hkv, const uint8_t* pool,
                                           int64_t num_pages, const int32_t* block_table, int bt_stride,
                                           const int32_t* seq_lens, float sm_scale, const tq_layer* layer,
                                           const tq_page_layout* layout, const void* recent_k, const void* recent_v,
                                           int recent_rows, int64_t rs_b, int64_t rs_r, int64_t rs_h,
                                           const int32_t* recent_len, void* out, void* workspace, int n_split,
                                           int stages, void* stream) {
  TailSpec ts;
  ts.k = recent_k; ts.v = recent_v; ts.rows = recent_rows;
  ts.s_b = rs_b; ts.s_r = rs_r; ts.s_h = rs_h; ts.len = recent_len;
  return decode_stages(q, dtype, B, Hq, Hkv, pool, num_pages, block_table, bt_stride, seq_lens, sm_scale, layer, layout,
                       ts, out, workspace, n_split, stages, stream);
}

extern "C" int tq_decode_attn_paged_ring(const void* q, int dtype, int B, int Hq, int Hkv, const uint8_t* pool,
                                         int64_t num_pages, const int32_t* block_table, int bt_stride,
                                         const int32_t* seq_lens, float sm_scale, const tq_layer* layer,
                                         const tq_page_layout* layout, const void* k_cache, const void* v_cache,
                                         int64_t cs_blk, int64_t cs_t, int64_t cs_h, int ring_rows, void* out,
                                         void* workspace, int n_split, void* stream) {
  if (!k_cache || !v_cache) return TQ_ENULL;
  if (ring_rows <= 0 || cs_blk <= 0 || cs_t <= 0 || cs_h <= 0) return TQ_EINVAL;
  TailSpec ts;
  ts.k = k_cache; ts.v = v_cache; ts.rows = ring_rows;
  ts.s_blk = cs_blk; ts.s_r = cs_t; ts.s_h = cs_h; ts.paged = true;
  return decode_stages(q, dtype, B, Hq, Hkv, pool, num_pages, block_table, bt_stride, seq_lens, sm_scale, layer, layout,
                       ts, out, workspace, n_split, 7, stream);
}

extern "C" int tq_decode_attn_paged(const void* q, int dtype, int B, int Hq, int Hkv, const uint8_t* pool,
                                    int64_t num_pages, const int32_t* block_table, int bt_stride,
                                    const int32_t* seq_lens, float sm_scale, const tq_layer* layer,
                                    const tq_page_layout* layout, const void* recent_k, const void* recent_v,
                                    int recent_rows, int64_t rs_b, int64_t rs_r, int64_t rs_h,
                                    const int32_t* recent_len, void* out, void* workspace, int n_split, void* stream) {
  return tq_decode_attn_paged_stages(q, dtype, B, Hq, Hkv, pool, num_pages, block_table, bt_stride, seq_lens, sm_scale,
                                     layer, layout, recent_k, recent_v, recent_rows, rs_b, rs_r, rs_h, recent_len, out,
                                     workspace, n_split, 7, stream);
}

// ---- the entry point that allocates nothing -----------------------------------------------------------
namespace {
constexpr int SCRATCH_MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[SCRATCH_MAX_DEVICES];      // device address of `scratch`, per device

// Address of the current device's copy of `scratch` (looked up once per device; two threads that race
// here ask for the same address).
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= SCRATCH_MAX_DEVICES) return TQ_EUNSUPPORTED;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return TQ_EINVAL;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return TQ_OK;
}

// Bytes of workspace decode_stages really touches for this call (tq_decode_workspace_bytes reserves
// room for the largest operand set instead): partials, rotated / sketched queries, statistics, and the
// packed operands of the matrix-core kernel, (index planes + multi-bit terms + sign plane) x d/128 KiB-words
// per group of query heads.
size_t decode_scratch_need(int B, int Hq, int Hkv, int n_split, const tq_layer& ly) {
  const int d = ly.d, G = Hq / Hkv;
  const int kv_div = (G + 7) / 8;
  size_t floats = parts_floats(B, Hq, d, n_split + TAIL_MAX_CHUNKS) + (size_t)2 * B * Hq * d + (size_t)4 * B * Hq +
                  2 * counter_words(B, Hq);
  size_t words = 0;
  if (kv_div && (d == 64 || d == 128 || d == 256)) {
    int planes = ly.mse_bits + 1;
    for (int t = 0; t < ly.n_terms; ++t)
      if (__builtin_popcount(ly.term_mask[t]) > 1) ++planes;
    words = (size_t)B * Hkv * kv_div * planes * (d >= 128 ? d / 128 : 1) * 2 * 64 * 8;
  } else if (kv_div && d > 256 && decode_wide_term_planes(ly) > 0) {
    words = (size_t)B * Hkv * kv_div * decode_wide_term_planes(ly) * 2 * wide_qa_stride(d) + 4;
  }
  return (floats + words) * 4;
}
}  // namespace

extern "C" size_t tq_decode_noalloc_bytes(int B, int Hq, int Hkv, int n_split, const tq_layer* layer) {
  if (!layer || B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || n_split <= 0 || layer->d <= 0 || layer->n_terms < 0 ||
      layer->n_terms > TQ_MAX_TERMS)
    return 0;
  return decode_scratch_need(B, Hq, Hkv, n_split, *layer);
}

extern "C" int tq_noalloc_init(void) {
  void* ws = nullptr;
  return scratch_address(&ws);
}

extern "C" int tq_decode_attn_paged_noalloc(const void* q, int dtype, int B, int Hq, int Hkv, const uint8_t* pool,
                                            int64_t num_pages, const int32_t* block_table, int bt_stride,
                                            const int32_t* seq_lens, float sm_scale, const tq_layer* layer,
                                            const tq_page_layout* layout, const void* recent_k, const void* recent_v,
                                            int recent_rows, int64_t rs_b, int64_t rs_r, int64_t rs_h,
                                            const int32_t* recent_len, void* out, int n_split, void* stream) {
  if (!layer) return TQ_ENULL;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || n_split <= 0 || layer->d <= 0 || layer->n_terms < 0 ||
      layer->n_terms > TQ_MAX_TERMS)
    return TQ_EINVAL;
  if (decode_scratch_need(B, Hq, Hkv, n_split, *layer) > (size_t)TQ_NOALLOC_SCRATCH_BYTES) return TQ_ETOOBIG;
  void* ws = nullptr;
  const int rc = scratch_address(&ws);
  if (rc) return rc;
  // Every byte of the scratch area that a stage reads was written by an earlier stage of the same call,
  // so nothing has to be cleared between calls.
  return tq_decode_attn_paged_stages(q, dtype, B, Hq, Hkv, pool, num_pages, block_table, bt_stride, seq_lens, sm_scale,
                                     layer, layout, recent_k, recent_v, recent_rows, rs_b, rs_r, rs_h, recent_len, out,
                                     ws, n_split, 7, stream);
}
