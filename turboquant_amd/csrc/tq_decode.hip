// Fused decode attention over the paged compressed store.
//
//   stage 0  rotate_query (tq_score.hip): q_rot = q Pi^T, q_sk = q S^T
//   stage 1  decode_pages_kernel: one workgroup per (split, KV head, sequence)
//            walks its share of the sequence's pages; all G query heads of the
//            group are scored from one read of the page; online softmax and the
//            value accumulation stay in registers; result = partial (m, l, acc)
//            exact_tail_kernel: the same partial for the exact recent tokens
//   stage 2  merge_kernel: log-sum-exp merge of the partials, cast to q's dtype
//
// Score of a token (triton_kernels.py:49-53,138):
//   s = sm_scale * ( norm * sum_j q_rot[j] c[idx_j] + qjl_scale * rnorm * sum_j q_sk[j] sigma_j )

#include "tq_common.h"

namespace tq {

constexpr int G_MAX = 16;      // query heads per KV head handled by one workgroup
constexpr int DEC_WAVES = 4;
constexpr float NEG_BIG = -1.0e30f;

// index of coordinate c in the LDS query tile [d][G] with a 4-float skew per 32
// coordinates so that the four coordinate quarters of a wave hit distinct banks
__device__ __forceinline__ int qoff(int c, int G) { return c * G + (c >> 5) * 4; }

template <int VB>
__global__ void __launch_bounds__(DEC_WAVES * 64)
decode_pages_kernel(const float* __restrict__ q_rot, const float* __restrict__ q_sk, int Hq, int Hkv,
                    const uint8_t* __restrict__ pool, const int32_t* __restrict__ block_table, int bt_stride,
                    const int32_t* __restrict__ seq_lens, float sm_scale, tq_layer ly, tq_page_layout L,
                    float* __restrict__ parts, int n_parts, int n_split) {
  const int d = ly.d, mb = ly.mse_bits, G = Hq / Hkv, words = d >> 5;
  const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, kb = lane >> 4;
  const int cpl = d >> 6;   // channels per lane in the value stage

  extern __shared__ __align__(16) float smem[];
  const int qsz = d * G + (d >> 5) * 4;
  float* s_rot = smem;                  // [d][G] skewed
  float* s_sk = s_rot + qsz;
  float* s_cent = s_sk + qsz;           // [16]
  float* s_p = s_cent + 16;             // [DEC_WAVES][G][16] softmax weights of the current page
  float* s_red = s_p + DEC_WAVES * G * 16;   // cross-wave reduction: [DEC_WAVES][G][d + 2]

  for (int o = tid; o < d * G; o += blockDim.x) {
    int g = o / d, c = o - g * d;
    int64_t row = (int64_t)b * Hq + h * G + g;
    s_rot[qoff(c, G) + g] = q_rot[row * d + c];
    s_sk[qoff(c, G) + g] = q_sk[row * d + c];
  }
  if (tid < (1 << mb)) s_cent[tid] = ly.centroids[tid];
  __syncthreads();

  const int seq_len = seq_lens[b];
  const int n_pages = (seq_len + TQ_PAGE_TOKENS - 1) / TQ_PAGE_TOKENS;
  const int per_split = (n_pages + n_split - 1) / n_split;
  const int pg_begin = split * per_split;
  const int pg_end = min(n_pages, pg_begin + per_split);

  float m[G_MAX], l[G_MAX], acc[G_MAX][12];
#pragma unroll
  for (int g = 0; g < G_MAX; ++g) {
    m[g] = NEG_BIG;
    l[g] = 0.0f;
#pragma unroll
    for (int c = 0; c < 12; ++c) acc[g][c] = 0.0f;
  }

  const int32_t* bt = block_table + (int64_t)b * bt_stride;
  float* my_p = s_p + wave * G * 16;

  for (int pi = pg_begin + wave; pi < pg_end; pi += DEC_WAVES) {
    const uint8_t* pg = pool + ((int64_t)bt[pi] * Hkv + h) * (int64_t)L.page_bytes;
    const int n_valid = min(TQ_PAGE_TOKENS, seq_len - pi * TQ_PAGE_TOKENS);

    // ---- scores: lane (n, kb) covers coordinate words kb, kb+4, ... of token n
    float pm[G_MAX], pq[G_MAX];
#pragma unroll
    for (int g = 0; g < G_MAX; ++g) pm[g] = pq[g] = 0.0f;
    for (int w = kb; w < words; w += 4) {
      uint32_t pw[5];
      for (int p = 0; p <= mb; ++p) pw[p] = *(const uint32_t*)(pg + key_word_off(L, p, w, n));
      for (int i = 0; i < 32; ++i) {
        unsigned id = 0;
        for (int p = 0; p < mb; ++p) id = (id << 1) | ((pw[p] >> i) & 1u);
        float cv = s_cent[id];
        float sg = ((pw[mb] >> i) & 1u) ? 1.0f : -1.0f;
        const float* qr = s_rot + qoff(w * 32 + i, G);
        const float* qs = s_sk + qoff(w * 32 + i, G);
#pragma unroll
        for (int g = 0; g < G_MAX; ++g) {
          if (g < G) {
            pm[g] = fmaf(qr[g], cv, pm[g]);
            pq[g] = fmaf(qs[g], sg, pq[g]);
          }
        }
      }
    }
    const float nk = (n < n_valid) ? ((const float*)(pg + L.off_meta))[2 * n] : 0.0f;
    const float rk = (n < n_valid) ? ly.qjl_scale * ((const float*)(pg + L.off_meta))[2 * n + 1] : 0.0f;
#pragma unroll
    for (int g = 0; g < G_MAX; ++g) {
      if (g < G) {
        float a = pm[g], c = pq[g];
        a += __shfl_xor(a, 16, 64); a += __shfl_xor(a, 32, 64);
        c += __shfl_xor(c, 16, 64); c += __shfl_xor(c, 32, 64);
        float s = (n < n_valid) ? sm_scale * (nk * a + rk * c) : NEG_BIG;
        // online softmax over the 16 tokens of the page (all 64 lanes hold a copy)
        float tmax = s;
        for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
        float m_new = fmaxf(m[g], tmax);
        float alpha = __expf(m[g] - m_new);
        float p = (n < n_valid) ? __expf(s - m_new) : 0.0f;
        float psum = p;
        for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, 64);
        l[g] = l[g] * alpha + psum;
        m[g] = m_new;
#pragma unroll
        for (int c2 = 0; c2 < 12; ++c2) acc[g][c2] *= alpha;
        if (kb == 0) my_p[g * 16 + n] = p;
      }
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();

    // ---- values: lane owns channels lane, lane+64, ...
#pragma unroll
    for (int c2 = 0; c2 < 12; ++c2) {
      if (c2 < cpl) {
        const int ch = lane + 64 * c2, grp = ch / L.group_size;
        const uint32_t* field = (const uint32_t*)(pg + vfield_off(L, ch));
        uint32_t f0 = field[0], f1 = (VB == 4) ? field[1] : 0u;
        const int es = L.dtype == TQ_F32 ? 4 : 2;
        const uint8_t* sc_p = pg + L.off_vscale + grp * TQ_PAGE_TOKENS * es;
        const uint8_t* zr_p = pg + L.off_vzero + grp * TQ_PAGE_TOKENS * es;
        for (int t = 0; t < n_valid; ++t) {
          unsigned code;
          if (VB == 2) code = (f0 >> (2 * t)) & 3u;
          else code = ((t < 8 ? f0 : f1) >> (4 * (t & 7))) & 15u;
          float val = fmaf((float)code, load_as_f32(sc_p, t, L.dtype), load_as_f32(zr_p, t, L.dtype));
#pragma unroll
          for (int g = 0; g < G_MAX; ++g)
            if (g < G) acc[g][c2] = fmaf(my_p[g * 16 + t], val, acc[g][c2]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // ---- merge the four waves of the workgroup, then write the partial
  for (int g = 0; g < G; ++g) {
    float* r = s_red + ((wave * G) + g) * (d + 2);
    if (lane == 0) { r[0] = m[g]; r[1] = l[g]; }
    for (int c2 = 0; c2 < cpl; ++c2) r[2 + lane + 64 * c2] = acc[g][c2];
  }
  __syncthreads();
  for (int o = tid; o < G * d; o += blockDim.x) {
    int g = o / d, ch = o - g * d;
    float mm = NEG_BIG;
    for (int w = 0; w < DEC_WAVES; ++w) mm = fmaxf(mm, s_red[((w * G) + g) * (d + 2)]);
    float ll = 0.0f, aa = 0.0f;
    for (int w = 0; w < DEC_WAVES; ++w) {
      const float* r = s_red + ((w * G) + g) * (d + 2);
      float wgt = __expf(r[0] - mm);
      ll += wgt * r[1];
      aa += wgt * r[2 + ch];
    }
    float* out = parts + (((int64_t)b * Hq + h * G + g) * n_parts + split) * (d + 2);
    if (ch == 0) { out[0] = mm; out[1] = ll; }
    out[2 + ch] = aa;
  }
}

// Partial (m, l, acc) over exact recent tokens (score.py:99-111, 138-173): one
// workgroup of 128 threads per (KV head, sequence).
__global__ void __launch_bounds__(128)
exact_tail_kernel(const void* __restrict__ q, int dtype, int Hq, int Hkv, int d, const void* __restrict__ rk,
                  const void* __restrict__ rv, int recent_rows, int64_t rs_b, int64_t rs_r, int64_t rs_h,
                  const int32_t* __restrict__ recent_len, float sm_scale, float* __restrict__ parts, int n_parts,
                  int part_index) {
  const int G = Hq / Hkv, h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int R = recent_len ? min(recent_len[b], recent_rows) : recent_rows;
  extern __shared__ float sm[];
  float* sq = sm;              // [G][d]
  float* ss = sq + G * d;      // [G][recent_rows]
  float* sml = ss + G * recent_rows;  // [G][2]
  for (int o = tid; o < G * d; o += blockDim.x) sq[o] = load_as_f32(q, ((int64_t)b * Hq + h * G) * d + o, dtype);
  __syncthreads();
  for (int t = tid; t < R; t += blockDim.x) {
    const int64_t base = b * rs_b + (int64_t)t * rs_r + h * rs_h;
    for (int g = 0; g < G; ++g) {
      float a = 0.0f;
      for (int i = 0; i < d; ++i) a = fmaf(sq[g * d + i], load_as_f32(rk, base + i, dtype), a);
      ss[g * recent_rows + t] = a * sm_scale;
    }
  }
  __syncthreads();
  const int lane = tid & 63, wave = tid >> 6;
  for (int g = wave; g < G; g += 2) {
    float mx = NEG_BIG;
    for (int t = lane; t < R; t += 64) mx = fmaxf(mx, ss[g * recent_rows + t]);
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int t = lane; t < R; t += 64) {
      float p = __expf(ss[g * recent_rows + t] - mx);
      ss[g * recent_rows + t] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    if (lane == 0) { sml[g * 2] = mx; sml[g * 2 + 1] = sum; }
  }
  __syncthreads();
  for (int o = tid; o < G * d; o += blockDim.x) {
    int g = o / d, ch = o - g * d;
    float a = 0.0f;
    for (int t = 0; t < R; ++t)
      a = fmaf(ss[g * recent_rows + t], load_as_f32(rv, b * rs_b + (int64_t)t * rs_r + h * rs_h + ch, dtype), a);
    float* out = parts + (((int64_t)b * Hq + h * G + g) * n_parts + part_index) * (d + 2);
    if (ch == 0) { out[0] = sml[g * 2]; out[1] = sml[g * 2 + 1]; }
    out[2 + ch] = a;
  }
}

// n_parts partials are merged per row; consecutive rows are part_stride partials apart.
// One workgroup per row.  A thread owns a pair of channels and every S-th part (S = 256 / (d/2)
// subsets share the parts when a row has fewer than 256 channel pairs); its first MERGE_CHUNK
// accumulator loads are issued before anything else, so that the (m, l) loads, the weights
// exp(m_s - M) and their reductions all run under one memory latency.
constexpr int MERGE_CHUNK = 16;
static size_t merge_smem(int n_parts, int d) {
  const int np = d >> 1, S = np >= 256 ? 1 : 256 / np;
  return ((size_t)3 * n_parts + 8 + (size_t)S * d) * sizeof(float);
}

__global__ void __launch_bounds__(256)
merge_kernel(const float* __restrict__ parts, int n_parts, int part_stride, int d, int dtype, void* __restrict__ out) {
  extern __shared__ float s_w[];                 // [n_parts] weights, [n_parts] m, [n_parts] l, [8] scratch, [S][d] sums
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* p = parts + row * part_stride * (int64_t)(d + 2);
  float* s_m = s_w + n_parts;
  float* s_l = s_m + n_parts;
  float* scratch = s_l + n_parts;
  float* s_sum = scratch + 8;
  const int np = d >> 1;                                        // channel pairs of a row
  const int S = np >= 256 ? 1 : 256 / np;                       // subsets of parts (d is a multiple of 64)
  const int tps = 256 / S;                                      // threads per subset
  const int sub = tid / tps, pr = tid - sub * tps;
  typedef float f2 __attribute__((ext_vector_type(2)));
  // first chunk of this thread's accumulator loads (pair pr; parts sub, sub + S, ...), clamped in range
  f2 v[MERGE_CHUNK];
#pragma unroll
  for (int k = 0; k < MERGE_CHUNK; ++k) {
    const int sp = min(sub + k * S, n_parts - 1);
    v[k] = *(const f2*)(p + (int64_t)sp * (d + 2) + 2 + 2 * min(pr, np - 1));
  }
  float mm = NEG_BIG;
  for (int sp = tid; sp < n_parts; sp += blockDim.x) {
    const f2 ml = *(const f2*)(p + (int64_t)sp * (d + 2));
    s_m[sp] = ml[0];
    s_l[sp] = ml[1];
    if (ml[1] > 0.0f) mm = fmaxf(mm, ml[0]);
  }
  mm = wave_max(mm);
  if (lane == 0) scratch[wave] = mm;
  __syncthreads();
  mm = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
  float ll = 0.0f;
  for (int sp = tid; sp < n_parts; sp += blockDim.x) {
    const float w = s_l[sp] > 0.0f ? __expf(s_m[sp] - mm) : 0.0f;
    s_w[sp] = w;
    ll += w * s_l[sp];
  }
  ll = wave_sum(ll);
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
          v[k] = *(const f2*)(p + (int64_t)sp * (d + 2) + 2 + 2 * p0);
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
    s_sum[sub * d + 2 * p0] = acc[0];
    s_sum[sub * d + 2 * p0 + 1] = acc[1];
  }
  __syncthreads();
  for (int ch = tid; ch < d; ch += blockDim.x) {
    float aa = 0.0f;
    for (int q = 0; q < S; ++q) aa += s_sum[q * d + ch];
    store_from_f32(out, row * d + ch, aa * inv, dtype);
  }
}

}  // namespace tq

using namespace tq;

namespace tq {
int launch_rotate_query(const void* q, int dtype, int64_t rows, const tq_layer* layer, float* q_rot, float* q_sk,
                        float* q_stat, uint32_t* qa_pack, int G, float sm_scale, hipStream_t st);
size_t decode_mfma_pack_words(int B, int Hkv, int d);
int launch_decode_mfma(const uint32_t* qa_pack, const float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, hipStream_t st);
}  // namespace tq

static size_t parts_floats(int B, int Hq, int d, int n_parts) { return (size_t)B * Hq * n_parts * (d + 2); }

extern "C" size_t tq_decode_workspace_bytes(int B, int Hq, int d, int n_split) {
  if (B <= 0 || Hq <= 0 || d <= 0 || n_split <= 0) return 0;
  // partials for n_split history splits + 1 exact tail, then q_rot, q_sk, 4 statistics per query row and
  // the packed query operands of the matrix-core kernel (sized for the largest kernel: 9 term planes, 8 heads)
  return (parts_floats(B, Hq, d, n_split + 1) + (size_t)2 * B * Hq * d + (size_t)4 * B * Hq) * sizeof(float) +
         decode_mfma_pack_words(B, Hq, d) * sizeof(uint32_t);
}

extern "C" int tq_decode_merge(const float* parts, int64_t rows, int n_parts, int d, int dtype, void* out,
                               void* stream) {
  if (!parts || !out) return TQ_ENULL;
  if (rows < 0 || n_parts <= 0 || d <= 0 || dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  if (rows == 0) return TQ_OK;
  merge_kernel<<<dim3((unsigned)rows), dim3(256), merge_smem(n_parts, d), (hipStream_t)stream>>>(
      parts, n_parts, n_parts, d, dtype, out);
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
  if (!q || !pool || !block_table || !seq_lens || !layer || !layout || !out || !workspace) return TQ_ENULL;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || n_split <= 0 || num_pages <= 0 || bt_stride < 0) return TQ_EINVAL;
  if (B > 65535 || Hkv > 65535) return TQ_EUNSUPPORTED;
  const int d = layer->d, G = Hq / Hkv;
  if (d != layout->d || layer->mse_bits != layout->mse_bits) return TQ_EINVAL;
  if (d < 64 || d > 768 || (d & 63) || G > G_MAX) return TQ_EUNSUPPORTED;
  if (layout->value_bits != 2 && layout->value_bits != 4) return TQ_EUNSUPPORTED;
  const bool tail = recent_k != nullptr && recent_rows > 0;
  if (tail && !recent_v) return TQ_ENULL;
  if (tail && recent_rows > 1024) return TQ_EUNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const int n_parts = n_split + 1;
  float* parts = (float*)workspace;
  float* q_rot = parts + parts_floats(B, Hq, d, n_parts);
  float* q_sk = q_rot + (size_t)B * Hq * d;
  float* q_stat = q_sk + (size_t)B * Hq * d;
  uint32_t* qa_pack = (uint32_t*)(q_stat + (size_t)4 * B * Hq);
  // the matrix-core kernel takes up to 8 query heads per group: a KV head with more is served by kv_div
  // groups of G / kv_div heads (0 = no such split, e.g. 11 heads)
  int kv_div = 0;
  for (int n = 1; n <= G && !kv_div; ++n)
    if (G % n == 0 && G / n <= 8) kv_div = n;
  const int Gq = kv_div ? G / kv_div : G;
  const bool mfma_shape = kv_div && (d == 128 || d == 256) && (layout->dtype == TQ_BF16 || layout->dtype == TQ_F16) &&
                          layer->Pi_colsum &&
                          layer->S_colsum;

  if (stages & 1) {
    if (!layer->Pi || !layer->PiT || !layer->S || !layer->ST || !layer->centroids) return TQ_ENULL;
    if (dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
    int rc = launch_rotate_query(q, dtype, (int64_t)B * Hq, layer, q_rot, q_sk, q_stat, mfma_shape ? qa_pack : nullptr,
                                 mfma_shape ? Gq : G, sm_scale, st);
    if (rc) return rc;
  }
  if (!(stages & 6)) return TQ_OK;

  const int qsz = d * G + (d >> 5) * 4;
  size_t smem = (size_t)(2 * qsz + 16 + DEC_WAVES * G * 16 + DEC_WAVES * G * (d + 2)) * sizeof(float);
  dim3 grid(n_split, Hkv, B), block(DEC_WAVES * 64);
  int mf = TQ_EUNSUPPORTED;
  if (stages & 2)
    mf = mfma_shape ? launch_decode_mfma(qa_pack, q_stat, B, Hq, Hkv * kv_div, kv_div, pool, block_table, bt_stride,
                                         seq_lens, sm_scale, *layer, *layout, parts, n_parts, n_split, st)
                    : TQ_EUNSUPPORTED;
  if (mf > 0) return mf;
  if ((stages & 2) && mf == TQ_EUNSUPPORTED) {      // no matrix-core kernel for this shape: general kernel
#define TQ_LAUNCH_DEC(VB)                                                                                 \
  {                                                                                                       \
    auto kern = decode_pages_kernel<VB>;                                                                  \
    if (smem > 48 * 1024) {                                                                               \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
      if (e != hipSuccess) return (int)e;                                                                 \
    }                                                                                                     \
    kern<<<grid, block, smem, st>>>(q_rot, q_sk, Hq, Hkv, pool, block_table, bt_stride, seq_lens, sm_scale, *layer,  \
                                    *layout, parts, n_parts, n_split);                                    \
  }
  if (dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  if (layout->value_bits == 2) TQ_LAUNCH_DEC(2)
  else TQ_LAUNCH_DEC(4)
#undef TQ_LAUNCH_DEC
  TQ_CHECK_LAUNCH();
  }

  if (tail && (stages & 2)) {
    size_t tsm = (size_t)(G * d + G * recent_rows + 2 * G) * sizeof(float);
    auto kern = exact_tail_kernel;
    if (tsm > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)tsm);
      if (e != hipSuccess) return (int)e;
    }
    kern<<<dim3(Hkv, B), dim3(128), tsm, st>>>(q, dtype, Hq, Hkv, d, recent_k, recent_v, recent_rows, rs_b, rs_r, rs_h,
                                               recent_len, sm_scale, parts, n_parts, n_split);
    TQ_CHECK_LAUNCH();
  }
  if (!(stages & 4)) return TQ_OK;
  // without a tail the merge simply reads one part fewer
  merge_kernel<<<dim3((unsigned)(B * Hq)), dim3(256), merge_smem(n_parts, d), st>>>(
      parts, tail ? n_parts : n_split, n_parts, d, dtype, out);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
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
