// Read-side kernels on the reference's flat tensor layouts: query rotation /
// sketch, the asymmetric score estimator, and key / value de-quantisation.

#include "tq_common.h"

namespace tq {

// q_rot = q Pi^T, q_sk = q S^T for `rows` query vectors (triton_kernels.py:527-528), fp32.
// One workgroup per row with d x 4 threads: thread (j, s) sums slice s of the
// contraction for output column j, the four slices meet in LDS.  q_stat
// (nullable) receives per row {max|q_rot|, max|q_sk|, sum q_rot, sum q_sk}, which
// the matrix-core decode kernel uses to normalise and re-centre its operands.
__global__ void __launch_bounds__(1024)
rotate_query_kernel(const void* __restrict__ q, int dtype, tq_layer ly, float* __restrict__ q_rot,
                    float* __restrict__ q_sk, float* __restrict__ q_stat) {
  extern __shared__ float sm[];
  const int d = ly.d, tid = threadIdx.x, j = tid % d, sl = tid / d, n_sl = blockDim.x / d;
  float* sq = sm;                 // [d]
  float* pa = sm + d;             // [n_sl][d]
  float* pb = pa + n_sl * d;      // [n_sl][d]
  float* red = pb + n_sl * d;     // [4][16]
  const int64_t row = blockIdx.x;
  if (tid < d) sq[tid] = load_as_f32(q, row * d + tid, dtype);
  __syncthreads();
  const int per = d / n_sl, i0 = sl * per;
  float a = 0.0f, b = 0.0f;
  for (int i = i0; i < i0 + per; ++i) {
    const float x = sq[i];
    a = fmaf(x, ly.PiT[(int64_t)i * d + j], a);
    b = fmaf(x, ly.ST[(int64_t)i * d + j], b);
  }
  pa[sl * d + j] = a;
  pb[sl * d + j] = b;
  __syncthreads();
  float ra = 0.0f, rb = 0.0f;
  if (tid < d) {
    for (int k = 0; k < n_sl; ++k) { ra += pa[k * d + tid]; rb += pb[k * d + tid]; }
    q_rot[row * d + tid] = ra;
    q_sk[row * d + tid] = rb;
  }
  if (q_stat) {
    const int lane = tid & 63, wave = tid >> 6, n_wave = blockDim.x >> 6;
    float ma = wave_max(tid < d ? fabsf(ra) : 0.0f), mb = wave_max(tid < d ? fabsf(rb) : 0.0f);
    float sa = wave_sum(tid < d ? ra : 0.0f), sb = wave_sum(tid < d ? rb : 0.0f);
    if (lane == 0) { red[wave] = ma; red[16 + wave] = mb; red[32 + wave] = sa; red[48 + wave] = sb; }
    __syncthreads();
    if (tid == 0) {
      float m1 = 0.0f, m2 = 0.0f, s1 = 0.0f, s2 = 0.0f;
      for (int w = 0; w < n_wave; ++w) { m1 = fmaxf(m1, red[w]); m2 = fmaxf(m2, red[16 + w]); s1 += red[32 + w]; s2 += red[48 + w]; }
      q_stat[row * 4 + 0] = m1; q_stat[row * 4 + 1] = m2; q_stat[row * 4 + 2] = s1; q_stat[row * 4 + 3] = s2;
    }
  }
}

// scores[b, i, k] for a tile of QT queries and one key per thread.
constexpr int QT = 8;

__global__ void __launch_bounds__(256)
score_kernel(const float* __restrict__ q_rot, const float* __restrict__ q_sk, int64_t n_q,
             const uint8_t* __restrict__ idx, const uint8_t* __restrict__ signs, const void* __restrict__ norms,
             int norm_dtype, const float* __restrict__ rnorms, int64_t n_k, tq_layer ly, float* __restrict__ scores) {
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

// x_hat for a tile of 16 vectors: (c[idx] Pi) * norm + (sigma S) * (qjl_scale * rnorm)
// (quantizer.py:151-165, 259-272).  d threads, thread i owns output coordinate i.
__global__ void __launch_bounds__(1024)
dequant_keys_kernel(const uint8_t* __restrict__ idx, const uint8_t* __restrict__ signs, const void* __restrict__ norms,
                    int norm_dtype, const float* __restrict__ rnorms, int64_t n_vec, tq_layer ly,
                    float* __restrict__ out) {
  constexpr int TILE = 16;
  extern __shared__ float sm[];
  const int d = ly.d, mb = ly.mse_bits, i = threadIdx.x;
  float* sc = sm;               // [TILE][d] centroid values
  float* ss = sm + TILE * d;    // [TILE][d] +-1
  const int eff = eff_bits(mb), per = 8 / eff, row = idx_row_bytes(d, mb), srow = d >> 3;
  const unsigned mask = (1u << eff) - 1u;
  const int64_t v0 = (int64_t)blockIdx.x * TILE;
  for (int t = 0; t < TILE; ++t) {
    int64_t v = v0 + t;
    float cv = 0.0f, sg = 0.0f;
    if (v < n_vec) {
      unsigned byte = idx[v * row + i / per];
      cv = ly.centroids[(byte >> (eff * (i % per))) & mask];
      if (signs) sg = ((signs[v * srow + (i >> 3)] >> (i & 7)) & 1u) ? 1.0f : -1.0f;
    }
    sc[t * d + i] = cv;
    ss[t * d + i] = sg;
  }
  __syncthreads();
  float a[TILE], b[TILE];
#pragma unroll
  for (int t = 0; t < TILE; ++t) a[t] = b[t] = 0.0f;
  for (int j = 0; j < d; ++j) {
    float pv = ly.Pi[(int64_t)j * d + i];
    float sv = signs ? ly.S[(int64_t)j * d + i] : 0.0f;
#pragma unroll
    for (int t = 0; t < TILE; ++t) {
      a[t] = fmaf(sc[t * d + j], pv, a[t]);
      b[t] = fmaf(ss[t * d + j], sv, b[t]);
    }
  }
  for (int t = 0; t < TILE; ++t) {
    int64_t v = v0 + t;
    if (v >= n_vec) break;
    float r = __fmul_rn(a[t], load_as_f32(norms, v, norm_dtype));
    if (signs) r = __fadd_rn(r, __fmul_rn(b[t], __fmul_rn(ly.qjl_scale, rnorms[v])));
    out[v * d + i] = r;
  }
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
int launch_rotate_query(const void* q, int dtype, int64_t rows, const tq_layer* layer, float* q_rot, float* q_sk,
                        float* q_stat, hipStream_t st) {
  const int d = layer->d;
  int n_sl = 4;
  while (n_sl > 1 && (d * n_sl > 1024 || d % n_sl)) n_sl >>= 1;
  size_t smem = (size_t)(d + 2 * n_sl * d + 64) * sizeof(float);
  rotate_query_kernel<<<dim3((unsigned)rows), dim3(d * n_sl), smem, st>>>(q, dtype, *layer, q_rot, q_sk, q_stat);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TQ_OK : (int)e;
}
}  // namespace tq

extern "C" int tq_rotate_query(const void* q, int dtype, int64_t rows, const tq_layer* layer, float* q_rot,
                               float* q_sk, void* stream) {
  int rc = check_layer_rd(layer, true);
  if (rc) return rc;
  if (!q || !q_rot || !q_sk) return TQ_ENULL;
  if (rows < 0 || dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  if (rows == 0) return TQ_OK;
  return launch_rotate_query(q, dtype, rows, layer, q_rot, q_sk, nullptr, (hipStream_t)stream);
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
  score_kernel<<<grid, dim3(256), smem, (hipStream_t)stream>>>(q_rot, q_sk, n_q, idx, signs, norms, norm_dtype, rnorms,
                                                              n_k, *layer, scores);
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
  const int d = layer->d;
  size_t smem = (size_t)2 * 16 * d * sizeof(float);
  auto kern = dequant_keys_kernel;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return (int)e;
  }
  kern<<<dim3((unsigned)((n_vec + 15) / 16)), dim3(d), smem, (hipStream_t)stream>>>(idx, signs, norms, norm_dtype,
                                                                                    rnorms, n_vec, *layer, out);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

extern "C" int tq_dequant_values(const uint8_t* data, const void* scales, const void* zeros, int dtype, int64_t n_vec,
                                 int d, int group_size, int bits, float* out, void* stream) {
  if (!data || !scales || !zeros || !out) return TQ_ENULL;
  if (bits != 2 && bits != 4 && bits != 8) return TQ_EUNSUPPORTED;
  if (d <= 0 || group_size <= 0 || d % group_size || (d * bits) % 8 || n_vec < 0) return TQ_EINVAL;
  if (dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  if (n_vec == 0) return TQ_OK;
  int64_t total = n_vec * d;
  dequant_values_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
      data, scales, zeros, dtype, n_vec, d, group_size, bits, out);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}
