// Quantise path: key quantiser (rotation, Lloyd-Max bucketise, residual, QJL sign
// sketch), value group quantiser, and the writers for the flat (reference)
// layout and for the paged store.
//
// One workgroup handles a tile of TQ_PAGE_TOKENS (16) vectors of one head with
// d threads, thread j owning coordinate j of every vector of the tile.  The
// three d x d contractions run in fp32 on the vector ALUs with the tile staged
// in LDS; matrices are read column-coalesced from their row-major transposes.

#include "tq_quantize.h"
#include "tq_options.h"

namespace tq {

// ------------------------------------------------------------------------------------
// parity entry points: bucketise+pack and sign-pack from given fp32 tensors
// ------------------------------------------------------------------------------------

__global__ void bucketize_pack_kernel(const float* __restrict__ y, int64_t n_vec, int d, const float* __restrict__ thr,
                                      int mse_bits, uint8_t* __restrict__ out) {
  const int eff = eff_bits(mse_bits), per = 8 / eff, row = idx_row_bytes(d, mse_bits);
  const int n_thr = (1 << mse_bits) - 1;
  int64_t gid = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (gid >= n_vec * row) return;
  int64_t v = gid / row;
  int k = (int)(gid - v * row);
  unsigned byte = 0;
  for (int s = 0; s < per; ++s) {
    int c = k * per + s;
    if (c >= d) break;
    float val = y[v * d + c];
    unsigned idx = 0;
    for (int t = 0; t < n_thr; ++t) idx += !(val <= thr[t]);
    byte |= idx << (eff * s);
  }
  out[gid] = (uint8_t)byte;
}

__global__ void sign_pack_kernel(const float* __restrict__ p, int64_t n_vec, int d, uint8_t* __restrict__ out) {
  const int row = (d + 7) / 8;
  int64_t gid = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (gid >= n_vec * row) return;
  int64_t v = gid / row;
  int k = (int)(gid - v * row);
  unsigned byte = 0;
  for (int s = 0; s < 8; ++s) {
    int c = k * 8 + s;
    if (c < d && p[v * d + c] > 0.0f) byte |= 1u << s;
  }
  out[gid] = (uint8_t)byte;
}

template <int DT, class Source, class Sink>
__global__ void __launch_bounds__(1024)
key_tile_kernel(const void* __restrict__ x, Source src, tq_layer ly, Sink sink, int mse_only) {
  using E = Elem<DT>;
  const int d = ly.d, j = threadIdx.x, tile = blockIdx.x;
  const int lane = j & 63, wave = j >> 6, n_wave = d >> 6;
  const int mb = ly.mse_bits, n_thr = (1 << mb) - 1;

  extern __shared__ __align__(16) unsigned char smem[];
  float* sx = (float*)smem;                 // [TILE][d] input as fp32
  float* su = sx + TILE * d;                // [TILE][d] unit vector -> centroid values -> residual
  uint8_t* sidx = (uint8_t*)(su + TILE * d);  // [TILE][d]
  uint8_t* ssgn = sidx + TILE * d;          // [TILE][d]
  float* snorm = (float*)(ssgn + TILE * d); // [TILE] norm as fp32 (value of the input dtype)
  float* srn = snorm + TILE;                // [TILE]
  float* scent = srn + TILE;                // [16] centroids
  int* svalid = (int*)(scent + 16);         // [TILE]

  if (j < (1 << mb)) scent[j] = ly.centroids[j];
  // (1) stage the tile
  for (int t = 0; t < TILE; ++t) {
    int64_t off;
    bool ok = src.locate(tile, t, off);
    sx[t * d + j] = ok ? E::load(x, off + j) : 0.0f;
    if (j == 0) svalid[t] = ok;
  }
  __syncthreads();
  {  // nothing to do for a tile without tokens (tail tiles of the paged grid)
    int any = 0;
    for (int t = 0; t < TILE; ++t) any |= svalid[t];
    if (!any) return;
  }
  // (2) norm in the input dtype (quantizer.py:136)
  for (int t = wave; t < TILE; t += n_wave) {
    float ss = 0.0f;
    for (int i = lane; i < d; i += 64) { float a = sx[t * d + i]; ss += a * a; }
    ss = wave_sum(ss);
    if (lane == 0) snorm[t] = E::round(sqrtf(ss));
  }
  __syncthreads();
  // (3) unit vector, still in the input dtype (quantizer.py:138)
  for (int t = 0; t < TILE; ++t) {
    float den = E::round(snorm[t] + 1e-10f);
    su[t * d + j] = E::round(sx[t * d + j] / den);
  }
  __syncthreads();
  // The three contractions: a thread owns two columns (c0, c0 + d / 2) of eight tokens - the lower half of the
  // workgroup the tile's first eight tokens, the upper half the others - so an LDS read of four vector elements feeds
  // eight multiply-adds (with one column of sixteen tokens per thread the loop waited for LDS: nine wavefronts reading
  // the same sixteen rows).  Every (token, column) sum still runs over the contraction in ascending order.
  constexpr int TH = TILE / 2;
  const int hd = d >> 1, upper = j >= hd ? 1 : 0, c0 = j - upper * hd, t_lo = upper * TH;
  float acc[TH][2];
  auto contract = [&](const float* __restrict__ M) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < TH; ++t) acc[t][0] = acc[t][1] = 0.0f;
    for (int i = 0; i < d; i += 4) {
      float m[4][2];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        m[k][0] = M[(int64_t)(i + k) * d + c0];
        m[k][1] = M[(int64_t)(i + k) * d + c0 + hd];
      }
#pragma unroll
      for (int t = 0; t < TH; ++t) {
        const float4 u = *(const float4*)(su + (t_lo + t) * d + i);
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          acc[t][c] = fmaf(u.x, m[0][c], acc[t][c]); acc[t][c] = fmaf(u.y, m[1][c], acc[t][c]);
          acc[t][c] = fmaf(u.z, m[2][c], acc[t][c]); acc[t][c] = fmaf(u.w, m[3][c], acc[t][c]);
        }
      }
    }
  };
  // (4) y = u Pi^T (fp32), bucketise
  contract(ly.PiT);
  __syncthreads();   // everyone is done reading su
#pragma unroll
  for (int t = 0; t < TH; ++t) {
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int tt = t_lo + t, jc = c0 + c * hd;
      float yv = acc[t][c];
      unsigned idx = 0;
      for (int k = 0; k < n_thr; ++k) idx += !(yv <= ly.thresholds[k]);
      sidx[tt * d + jc] = (uint8_t)idx;
      su[tt * d + jc] = scent[idx];
      if constexpr (std::is_same<Sink, KeyFlatSink>::value) {
        if (sink.y_dbg && svalid[tt]) sink.y_dbg[((int64_t)tile * TILE + tt) * d + jc] = yv;
      }
    }
  }
  __syncthreads();
  if (!mse_only) {
    // (5) x_hat = (c Pi) * norm ; r = x - x_hat ; rho = ||r|| (quantizer.py:241-245)
    contract(ly.Pi);
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TH; ++t) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int tt = t_lo + t, jc = c0 + c * hd;
        su[tt * d + jc] = sx[tt * d + jc] - acc[t][c] * snorm[tt];
      }
    }
    __syncthreads();
    for (int t = wave; t < TILE; t += n_wave) {
      float ss = 0.0f;
      for (int i = lane; i < d; i += 64) { float a = su[t * d + i]; ss += a * a; }
      ss = wave_sum(ss);
      if (lane == 0) srn[t] = sqrtf(ss);
    }
    // (6) p = r S^T ; sign bits (quantizer.py:248-249)
    contract(ly.ST);
#pragma unroll
    for (int t = 0; t < TH; ++t) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int tt = t_lo + t, jc = c0 + c * hd;
        ssgn[tt * d + jc] = acc[t][c] > 0.0f;
        if constexpr (std::is_same<Sink, KeyFlatSink>::value) {
          if (sink.p_dbg && svalid[tt]) sink.p_dbg[((int64_t)tile * TILE + tt) * d + jc] = acc[t][c];
        }
      }
    }
  }
  __syncthreads();

  // (7) write
  if constexpr (std::is_same<Sink, KeyFlatSink>::value)
    write_key_tile_flat<DT>(sink, tile, d, mb, mse_only, sidx, ssgn, snorm, srn, svalid, j, d);
  else
    write_key_tile_paged(sink, src, tile, d, mb, sidx, ssgn, snorm, srn, svalid, j, d);
}

static size_t key_tile_smem(int d) { return (size_t)TILE * d * (4 + 4 + 1 + 1) + (TILE * 2 + 16) * 4 + TILE * 4; }

// ------------------------------------------------------------------------------------
// value tile (kv_cache.py:45-98)
// ------------------------------------------------------------------------------------

struct ValFlatSink {
  uint8_t* data;
  void* scale;
  void* zero;
};
struct ValPagedSink {
  uint8_t* pool;
  const int32_t* block_table;
  int max_pages;
  int num_pages;           // pages of the pool (see checked_page)
  tq_page_layout L;
};

template <int DT, class Source, class Sink>
__global__ void __launch_bounds__(1024)
value_tile_kernel(const void* __restrict__ v, Source src, int d, int gs, int bits, Sink sink) {
  using E = Elem<DT>;
  const int j = threadIdx.x, tile = blockIdx.x, ng = d / gs;
  extern __shared__ __align__(16) unsigned char smem[];
  float* sv = (float*)smem;                   // [TILE][d]
  float* sscale = sv + TILE * d;              // [TILE][ng]
  float* szero = sscale + TILE * ng;          // [TILE][ng]
  uint8_t* scode = (uint8_t*)(szero + TILE * ng);  // [TILE][d]
  int* svalid = (int*)(scode + TILE * d);     // [TILE]

  {
    // all 16 loads are issued before any is used, and none sits under a branch (slots that
    // do not exist read the first vector and are zeroed afterwards)
    const typename Source::TileRef ref = src.tile_ref(tile);
    float vals[TILE];
    unsigned okm = 0;
#pragma unroll
    for (int t = 0; t < TILE; ++t) {
      int64_t off;
      const bool ok = src.slot_off(ref, t, off);
      okm |= (unsigned)ok << t;
      vals[t] = E::load(v, (ok ? off : 0) + j);
    }
    if (!okm) return;                          // uniform: validity depends on the slot only
#pragma unroll
    for (int t = 0; t < TILE; ++t) {
      sv[t * d + j] = ((okm >> t) & 1) ? vals[t] : 0.0f;
      if (j == 0) svalid[t] = (okm >> t) & 1;
    }
  }
  __syncthreads();
  const float levels = (float)((1 << bits) - 1);
  for (int o = j; o < TILE * ng; o += d) {
    int t = o / ng, g = o - t * ng;
    const float* row = sv + t * d + g * gs;
    float lo = row[0], hi = row[0];
    bool has_nan = false;
    for (int i = 0; i < gs; ++i) {
      float a = row[(i + j) % gs];           // rotate the start to spread LDS banks
      has_nan |= (a != a);
      lo = fminf(lo, a);
      hi = fmaxf(hi, a);
    }
    if (has_nan) lo = hi = __uint_as_float(0x7fc00000u);   // torch min/max propagate NaN
    float sc = E::round(E::round(hi - lo) / levels);
    float floor_v = E::round(1e-10f);
    sc = (sc != sc) ? sc : fmaxf(sc, floor_v);
    sscale[o] = sc;
    szero[o] = lo;
  }
  __syncthreads();
  for (int t = 0; t < TILE; ++t) {
    int g = j / gs;
    float sc = sscale[t * ng + g], z = szero[t * ng + g];
    float q = E::round(E::round(sv[t * d + j] - z) / sc);
    q = rintf(q);
    q = fminf(fmaxf(q, 0.0f), levels);
    scode[t * d + j] = (q != q) ? (uint8_t)0 : (uint8_t)q;
  }
  __syncthreads();

  if constexpr (std::is_same<Sink, ValFlatSink>::value) {
    const int per = 8 / bits, row = d / per;
    for (int o = j; o < TILE * row; o += d) {
      int t = o / row, k = o - t * row;
      if (!svalid[t]) continue;
      unsigned byte = 0;
      for (int s = 0; s < per; ++s) byte |= (unsigned)scode[t * d + k * per + s] << (bits * s);
      sink.data[((int64_t)tile * TILE + t) * row + k] = (uint8_t)byte;
    }
    for (int o = j; o < TILE * ng; o += d) {
      int t = o / ng, g = o - t * ng;
      if (!svalid[t]) continue;
      int64_t at = ((int64_t)tile * TILE + t) * ng + g;
      E::store(sink.scale, at, sscale[o]);
      E::store(sink.zero, at, szero[o]);
    }
  } else {
    int b, lpage, h;
    src.decode(tile, b, lpage, h);
    const tq_page_layout& L = sink.L;
    const int64_t page = checked_page(sink.block_table, sink.max_pages, sink.num_pages, b, lpage);
    if (page < 0) return;                              // outside the table or the pool: nothing is stored
    uint8_t* pg = sink.pool + (page * src.H + h) * (int64_t)L.page_bytes;
    // channel j: a field of 16*bits bits, token n at bit bits*n; read-modify-write keeps
    // the codes of slots this call does not touch
    const int wpc = bits / 2;                         // 32-bit words per channel
    uint32_t* field = (uint32_t*)(pg + vfield_off(L, j));
    const int per_word = 32 / bits;
    for (int w = 0; w < wpc; ++w) {
      uint32_t neu = 0, mask = 0;
      for (int s = 0; s < per_word; ++s) {
        int n = w * per_word + s;
        if (svalid[n]) {
          neu |= (uint32_t)scode[n * d + j] << (bits * s);
          mask |= ((1u << bits) - 1u) << (bits * s);
        }
      }
      uint32_t old = (mask == 0xffffffffu) ? 0u : field[w];
      field[w] = (old & ~mask) | neu;
    }
    for (int o = j; o < TILE * ng; o += d) {
      int n = o % TILE, g = o / TILE;
      if (!svalid[n]) continue;
      E::store(pg + L.off_vscale, g * TILE + n, sscale[n * ng + g]);
      E::store(pg + L.off_vzero, g * TILE + n, szero[n * ng + g]);
    }
  }
}

// round to the input dtype and back with the hardware conversions (v_cvt_pk_bf16_f32 / v_cvt_f16_f32,
// round to nearest even; NaN stays NaN)
template <int DT>
__device__ __forceinline__ float round_hw(float v) {
  if constexpr (DT == TQ_BF16) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t f = {v, 0.0f};
    const bf16x2_t r = __builtin_convertvector(f, bf16x2_t);
    uint32_t u;
    __builtin_memcpy(&u, &r, 4);
    return __uint_as_float(u << 16);
  } else {
    return Elem<DT>::round(v);
  }
}

// out[i] = in[i] - sub rounded to the input dtype, i < 8; bf16 rounds two numbers per conversion instruction
template <int DT>
__device__ __forceinline__ void round_pairs(const float (&in)[8], float sub, float (&out)[8]) {
  if constexpr (DT == TQ_BF16) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f32x2_t f = {in[2 * i] - sub, in[2 * i + 1] - sub};
      const bf16x2_t r = __builtin_convertvector(f, bf16x2_t);
      uint32_t u;
      __builtin_memcpy(&u, &r, 4);
      out[2 * i] = __uint_as_float(u << 16);
      out[2 * i + 1] = __uint_as_float(u & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = round_hw<DT>(in[i] - sub);
  }
}

// Faster value kernel for 16-bit inputs, 2/4-bit codes and head_dim 64 / 128 / 256: a thread owns 8
// consecutive channels of one token (one 16-byte load), a group's minimum / maximum meet through
// cross-lane exchanges, and the codes pass through LDS only to be transposed into the page's
// per-channel fields.  Arithmetic and rounding are those of value_tile_kernel.
template <int DT, int VB, class Source, class Sink>
__global__ void __launch_bounds__(512)
value_chunk_kernel(const void* __restrict__ v, Source src, int d, int gs, Sink sink) {
  using E = Elem<DT>;
  static_assert(DT != TQ_F32, "16-bit inputs");
  const int tid = threadIdx.x, tile = blockIdx.x;
  const int cpt = d >> 3;                          // chunks (threads) per token
  const int t = tid >> (31 - __builtin_clz(cpt)), ck = tid & (cpt - 1);     // token slot, chunk (head_dim 64 / 128 / 256)
  const int tpg = gs >> 3;                         // threads per group (power of two, <= 16)
  // a thread's 8 codes are one word of 8 * VB bits; the words of a chunk's 16 tokens lie together
  // (rows padded by 16 bytes), so that the thread that assembles half a channel field reads the
  // words of its 8 tokens with one or two 16-byte loads
  using CodeWord = typename std::conditional<VB == 2, uint16_t, uint32_t>::type;
  constexpr int CROW = TILE * (int)sizeof(CodeWord) + 16;      // bytes per chunk row
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* scode = smem;                     // [d / 8] rows of CROW bytes
  int* svalid = (int*)(smem + (size_t)cpt * CROW); // [TILE]

  // where the tile's rows are and which of its slots exist: uniform, looked up through the scalar cache
  TileAddr ta;
  // page lookup issued together with the input load (clamped into the table: a tile without a
  // single existing slot may lie beyond it, and then nothing is stored anyway)
  int64_t page = 0;
  int head = 0;
  if constexpr (std::is_same<Source, PagedSource>::value) {
    PagedSource::Coord c[1] = {src.coord(tile)};
    TileAddr ta1[1];
    int lpage[1];
    src.template tile_addrs<1>(c, ta1, lpage);
    ta = ta1[0];
    head = c[0].h;
    if constexpr (!std::is_same<Sink, ValFlatSink>::value)
      page = checked_page(sink.block_table, sink.max_pages, sink.num_pages, c[0].b, lpage[0]);
  } else {
    ta = src.tile_addr(tile);
  }
  const bool ok = t >= ta.lo && t < ta.hi;
  const int64_t off = ta.base + (int64_t)t * src.slot_stride();
  const bool page_ok = page >= 0;                    // uniform over the workgroup; false: nothing is stored
  // unconditional load (slots that do not exist read the first vector)
  const uint4 raw = *(const uint4*)((const uint16_t*)v + (ok ? off : 0) + ck * 8);
  if (ck == 0) svalid[t] = ok;
  // a tile none of whose slots exists may lie beyond the block table: leave before looking it up
  const int n_ok = __syncthreads_count(ok);
  if (n_ok == 0) return;
  const bool full_tile = n_ok == (int)blockDim.x;
  float x[8];
  {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = DT == TQ_BF16 ? __uint_as_float(w[i] << 16) : f16_bits_to_f32((uint16_t)(w[i] & 0xffffu));
      x[2 * i + 1] = DT == TQ_BF16 ? __uint_as_float(w[i] & 0xffff0000u) : f16_bits_to_f32((uint16_t)(w[i] >> 16));
    }
  }
  float lo = x[0], hi = x[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    lo = fminf(lo, x[i]);
    hi = fmaxf(hi, x[i]);
  }
  // a NaN among the 8 inputs, on the packed 16-bit patterns: magnitude bits above those of infinity
  int has_nan;
  {
    typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
    u16x2_t m = __builtin_bit_cast(u16x2_t, raw.x & 0x7fff7fffu);
    m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2_t, raw.y & 0x7fff7fffu));
    m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2_t, raw.z & 0x7fff7fffu));
    m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2_t, raw.w & 0x7fff7fffu));
    constexpr uint16_t inf_bits = DT == TQ_BF16 ? 0x7f80 : 0x7c00;
    has_nan = (m[0] > inf_bits) | (m[1] > inf_bits);
  }
  // the threads of a group are neighbouring lanes inside a row of 16: DPP moves (quad swaps, then half-row and
  // row mirrors, which pair quads that already agree) instead of shuffles through the LDS
  auto reduce_step = [&](auto ctrl_c) {
    constexpr int CTRL = decltype(ctrl_c)::value;
    lo = fminf(lo, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, lo), CTRL, 0xF, 0xF, true)));
    hi = fmaxf(hi, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, hi), CTRL, 0xF, 0xF, true)));
    has_nan |= __builtin_amdgcn_update_dpp(0, has_nan, CTRL, 0xF, 0xF, true);
  };
  if (tpg >= 2) reduce_step(std::integral_constant<int, 0xB1>{});
  if (tpg >= 4) reduce_step(std::integral_constant<int, 0x4E>{});
  if (tpg >= 8) reduce_step(std::integral_constant<int, 0x141>{});
  if (tpg >= 16) reduce_step(std::integral_constant<int, 0x140>{});
  if (has_nan) lo = hi = __uint_as_float(0x7fc00000u);       // torch min/max propagate NaN
  const float levels = (float)((1 << VB) - 1);
  // (hi - lo) / levels as a product: both are numbers of at most 8 significant bits, so is the divisor of every
  // quotient below, and such a quotient is never a rounding tie of the 16-bit format and at least 2^-17
  // (relative) away from one: a product with a reciprocal good to an ulp rounds like the division (checked
  // over all pairs of significands and the three nearest reciprocals).  fp16 keeps the division.
  const float range = round_hw<DT>(hi - lo);
  float sc = round_hw<DT>(DT == TQ_BF16 ? range * (1.0f / levels) : range / levels);
  const float floor_v = round_hw<DT>(1e-10f);
  sc = (sc != sc) ? sc : fmaxf(sc, floor_v);
  const float z = lo;
  // Quotients of bf16 numbers, rounded to bf16: a * (1/s) with any reciprocal good to an ulp (see above).
  // Used when the scale is an ordinary number; everything else takes the division.
  const bool fast_div = DT == TQ_BF16 && sc > 0x1p-60f && sc < 0x1p60f;
  const float rsc = __builtin_amdgcn_rcpf(sc);
  float quo[8];
  if (fast_div) {                // every a of the group is finite and at most (levels + 1) * sc < 2^64 then
    float a[8];
    round_pairs<DT>(x, z, a);
#pragma unroll
    for (int i = 0; i < 8; ++i) quo[i] = a[i] * rsc;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) quo[i] = round_hw<DT>(x[i] - z) / sc;
  }
  // 8 codes, VB bits each, channel order.  The codes are small integers held in floats: 16 bits' worth of
  // them are put together with exact multiply-adds and converted once.
  float qr[8];
  round_pairs<DT>(quo, 0.0f, qr);
  uint32_t codes = 0;
#pragma unroll
  for (int hw = 0; hw < (VB == 2 ? 1 : 2); ++hw) {
    constexpr int PER = 16 / VB;                   // codes per 16 bits
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      // clamp to [0, levels]; a NaN becomes code 0 (the median-of-three instruction returns the minimum of
      // its operands when one of them is a NaN)
      const float q = __builtin_amdgcn_fmed3f(rintf(qr[hw * PER + i]), 0.0f, levels);
      acc = fmaf(q, (float)(1 << (VB * i)), acc);
    }
    codes |= (uint32_t)acc << (16 * hw);
  }
  if constexpr (!std::is_same<Sink, ValFlatSink>::value) *(CodeWord*)(scode + ck * CROW + t * sizeof(CodeWord)) = (CodeWord)codes;
  const int ng = d / gs, g = (ck * 8) / gs;
  const bool leader = (ck & (tpg - 1)) == 0;

  if constexpr (std::is_same<Sink, ValFlatSink>::value) {
    if (ok) {
      const int64_t vec = (int64_t)tile * TILE + t;
      uint8_t* dst = sink.data + vec * (d * VB / 8) + ck * VB;           // 8 codes = VB bytes, little-end first
      if (VB == 2) *(uint16_t*)dst = (uint16_t)codes;
      else *(uint32_t*)dst = codes;
      if (leader) {
        E::store(sink.scale, vec * ng + g, sc);
        E::store(sink.zero, vec * ng + g, z);
      }
    }
  } else {
    const tq_page_layout& L = sink.L;
    uint8_t* pg = sink.pool + (page * src.H + head) * (int64_t)L.page_bytes;
    if (ok && leader && page_ok) {
      E::store(pg + L.off_vscale, g * TILE + t, sc);
      E::store(pg + L.off_vzero, g * TILE + t, z);
    }
    __syncthreads();
    // channel c: a field of 16*VB bits, token n at bit VB*n; read-modify-write keeps the codes of
    // slots this call does not touch
    // every thread assembles half a field: 8 tokens of one channel (16 bits of 2-bit codes, 32 of 4-bit)
    {
      const int c = tid >> 1, half = tid & 1;
      uint8_t* fbytes = pg + vfield_off(L, c) + half * VB;
      const unsigned char* row = scode + (c >> 3) * CROW + half * 8 * sizeof(CodeWord);
      const int sh = (c & 7) * VB;                   // the channel's code inside a word
      uint32_t neu = 0, mask = VB == 2 ? 0xffffu : 0xffffffffu;
      if constexpr (VB == 2) {
        const uint4 w = *(const uint4*)row;          // 8 tokens, two to a dword
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const uint32_t pr = (ww[k] >> sh) & 0x00030003u;
          neu |= ((pr | (pr >> 14)) & 0xfu) << (4 * k);
        }
      } else {
        const uint4 w0 = *(const uint4*)row, w1 = *(const uint4*)(row + 16);
        const uint32_t ww[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int k = 0; k < 8; ++k) neu |= ((ww[k] >> sh) & 0xfu) << (4 * k);
      }
      if (!full_tile) {                              // uniform over the workgroup
        mask = 0;
#pragma unroll
        for (int s2 = 0; s2 < 8; ++s2) mask |= (svalid[half * 8 + s2] ? (1u << VB) - 1u : 0u) << (VB * s2);
        neu &= mask;
      }
      if (mask != 0 && page_ok) {
        if (VB == 2) {
          uint16_t* f16p = (uint16_t*)fbytes;
          const uint32_t old = (mask == 0xffffu) ? 0u : *f16p;
          *f16p = (uint16_t)((old & ~mask) | neu);
        } else {
          uint32_t* f32p = (uint32_t*)fbytes;
          const uint32_t old = (mask == 0xffffffffu) ? 0u : *f32p;
          *f32p = (old & ~mask) | neu;
        }
      }
    }
  }
}

static size_t value_tile_smem(int d, int gs) { return (size_t)TILE * d * 5 + (size_t)TILE * (d / gs) * 8 + TILE * 4; }

// ------------------------------------------------------------------------------------
// page -> flat export (store.py:92-114)
// ------------------------------------------------------------------------------------

// a table entry outside the pool (stale or poisoned) is read as page 0: the export then holds that page's
// bytes for those tokens, and nothing outside the pool is touched
__device__ __forceinline__ int export_page(int raw, int num_pages) { return (unsigned)raw < (unsigned)num_pages ? raw : 0; }

__device__ __forceinline__ void copy_elem(void* dst, int64_t di, const void* src, int64_t si, int dt) {
  if (dt == TQ_F32) ((uint32_t*)dst)[di] = ((const uint32_t*)src)[si];
  else ((uint16_t*)dst)[di] = ((const uint16_t*)src)[si];
}

// The same export a word at a time: a workgroup per (page, head); index words are assembled from the
// bit planes with bit-spreading steps, sign words are copied, value codes are gathered from the page's
// per-channel fields through LDS.  Needs 4-byte aligned outputs (rows are multiples of 4 bytes because
// head_dim is a multiple of 64).
__global__ void __launch_bounds__(256)
pool_export_words_kernel(const uint8_t* __restrict__ pool, int num_pages, int H, const int32_t* __restrict__ block_table, int n_tok,
                         tq_page_layout L, uint32_t* __restrict__ idx, uint32_t* __restrict__ signs, void* norms,
                         float* rnorms, uint32_t* __restrict__ v_data, void* v_scales, void* v_zeros) {
  extern __shared__ __align__(16) uint32_t s_fields[];          // the page's value section, d * 2 vb bytes
  const int d = L.d, mb = L.mse_bits, vb = L.value_bits, ng = d / L.group_size, W = d >> 5;
  const int lpage = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const uint8_t* pg = pool + ((int64_t)export_page(block_table[lpage], num_pages) * H + h) * (int64_t)L.page_bytes;
  const int n_valid = min(TILE, n_tok - lpage * TILE);
  const int64_t flat0 = (int64_t)h * n_tok + (int64_t)lpage * TILE;
  const int field_dw = vb >> 1;                                  // dwords per channel field (16 * vb bits)
  for (int o = tid; o < d * field_dw; o += blockDim.x) s_fields[o] = ((const uint32_t*)(pg + L.off_vdata))[o];
  // keys: dword k of a row holds 32 / eff codes, code s at bit eff * s, plane 0 the top bit of a code
  const int eff = eff_bits(mb), n_per = 32 / eff, row_dw = idx_row_bytes(d, mb) >> 2;
  for (int o = tid; o < n_valid * row_dw; o += blockDim.x) {
    const int t = o / row_dw, k = o - t * row_dw, c0 = k * n_per;
    uint32_t dw = 0;
    for (int p = 0; p < mb; ++p) {
      uint32_t x = *(const uint32_t*)(pg + key_word_off(L, p, c0 >> 5, t)) >> (c0 & 31);
      if (eff == 2) {
        x &= 0xffffu;
        x = (x | (x << 8)) & 0x00ff00ffu;
        x = (x | (x << 4)) & 0x0f0f0f0fu;
        x = (x | (x << 2)) & 0x33333333u;
        x = (x | (x << 1)) & 0x55555555u;
      } else if (eff == 4) {
        x &= 0xffu;
        x = (x | (x << 12)) & 0x000f000fu;
        x = (x | (x << 6)) & 0x03030303u;
        x = (x | (x << 3)) & 0x11111111u;
      }
      dw |= x << (mb - 1 - p);
    }
    idx[(flat0 + t) * row_dw + k] = dw;
  }
  for (int o = tid; o < n_valid * W; o += blockDim.x) {
    const int t = o / W, w = o - t * W;
    signs[(flat0 + t) * W + w] = *(const uint32_t*)(pg + key_word_off(L, mb, w, t));
  }
  for (int o = tid; o < n_valid * ng; o += blockDim.x) {
    const int t = o / ng, g = o - t * ng;
    copy_elem(v_scales, (flat0 + t) * ng + g, pg + L.off_vscale, g * TILE + t, L.dtype);
    copy_elem(v_zeros, (flat0 + t) * ng + g, pg + L.off_vzero, g * TILE + t, L.dtype);
  }
  if (tid < n_valid) {
    store_from_f32(norms, flat0 + tid, ((const float*)(pg + L.off_meta))[2 * tid], L.dtype);
    rnorms[flat0 + tid] = ((const float*)(pg + L.off_meta))[2 * tid + 1];
  }
  __syncthreads();
  // values: dword j of a token's row holds 32 / vb channels; channel c's code sits at bit vb * t of its field
  const int cpd = 32 / vb, vrow_dw = (d * vb) >> 5;
  const uint32_t vmask = vb == 8 ? 0xffu : (1u << vb) - 1u;
  for (int o = tid; o < n_valid * vrow_dw; o += blockDim.x) {
    const int t = o / vrow_dw, j = o - t * vrow_dw;
    const int bit = vb * t;
    uint32_t dw = 0;
    for (int i = 0; i < cpd; ++i) {
      const int c = j * cpd + i;
      const int f = ((c & 15) * (d >> 4) + (c >> 4)) * field_dw;             // vfield_off in dwords
      dw |= ((s_fields[f + (bit >> 5)] >> (bit & 31)) & vmask) << (vb * i);
    }
    v_data[(flat0 + t) * vrow_dw + j] = dw;
  }
}

__global__ void pool_export_kernel(const uint8_t* __restrict__ pool, int num_pages, int H, const int32_t* __restrict__ block_table,
                                   int n_tok, tq_page_layout L, uint8_t* idx, uint8_t* signs, void* norms,
                                   float* rnorms, uint8_t* v_data, void* v_scales, void* v_zeros) {
  const int d = L.d, mb = L.mse_bits, vb = L.value_bits, ng = d / L.group_size;
  const int lpage = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const uint8_t* pg = pool + ((int64_t)export_page(block_table[lpage], num_pages) * H + h) * (int64_t)L.page_bytes;
  const int eff = eff_bits(mb), per = 8 / eff, row = idx_row_bytes(d, mb), srow = d >> 3;
  const int vrow = d * vb / 8, vper = 8 / vb;
  for (int n = 0; n < TILE; ++n) {
    int tok = lpage * TILE + n;
    if (tok >= n_tok) break;
    int64_t flat = (int64_t)h * n_tok + tok;
    for (int k = j; k < row; k += blockDim.x) {
      unsigned byte = 0;
      for (int s = 0; s < per; ++s) {
        int c = k * per + s;
        if (c >= d) break;
        unsigned id = 0;
        for (int p = 0; p < mb; ++p) {
          uint32_t w = *(const uint32_t*)(pg + key_word_off(L, p, c >> 5, n));
          id = (id << 1) | ((w >> (c & 31)) & 1u);
        }
        byte |= id << (eff * s);
      }
      idx[flat * row + k] = (uint8_t)byte;
    }
    for (int k = j; k < srow; k += blockDim.x) {
      uint32_t w = *(const uint32_t*)(pg + key_word_off(L, mb, k >> 2, n));
      signs[flat * srow + k] = (uint8_t)(w >> ((k & 3) * 8));
    }
    for (int k = j; k < vrow; k += blockDim.x) {
      unsigned byte = 0;
      for (int s = 0; s < vper; ++s) {
        int c = k * vper + s;
        const uint32_t* field = (const uint32_t*)(pg + vfield_off(L, c));
        int bit = vb * n;
        byte |= ((field[bit >> 5] >> (bit & 31)) & ((1u << vb) - 1u)) << (vb * s);
      }
      v_data[flat * vrow + k] = (uint8_t)byte;
    }
    for (int g = j; g < ng; g += blockDim.x) {
      copy_elem(v_scales, flat * ng + g, pg + L.off_vscale, g * TILE + n, L.dtype);
      copy_elem(v_zeros, flat * ng + g, pg + L.off_vzero, g * TILE + n, L.dtype);
    }
    if (j == 0) {
      store_from_f32(norms, flat, ((const float*)(pg + L.off_meta))[2 * n], L.dtype);
      rnorms[flat] = ((const float*)(pg + L.off_meta))[2 * n + 1];
    }
  }
}

}  // namespace tq

// ======================================================================================
// C ABI
// ======================================================================================

using namespace tq;

static int check_layer(const tq_layer* ly, bool need_sketch) {
  if (!ly) return TQ_ENULL;
  if (ly->d < 64 || ly->d > 768 || (ly->d & 63)) return TQ_EUNSUPPORTED;
  if (ly->mse_bits < 1 || ly->mse_bits > 4) return TQ_EUNSUPPORTED;
  if (!ly->Pi || !ly->PiT || !ly->centroids || !ly->thresholds) return TQ_ENULL;
  if (need_sketch && (!ly->S || !ly->ST)) return TQ_ENULL;
  return TQ_OK;
}

extern "C" int tq_version(void) { return TQ_ABI_VERSION; }

extern "C" int tq_layer_fill_terms(tq_layer* layer, const float* c) {
  if (!layer || !c) return TQ_ENULL;
  const int mb = layer->mse_bits;
  if (mb < 1 || mb > 4) return TQ_EUNSUPPORTED;
  const int n = 1 << mb;
  double w[16], wmax = 0.0;
  for (int s = 0; s < n; ++s) {           // Walsh coefficient of bit-subset s
    double a = 0.0;
    for (int b = 0; b < n; ++b) a += (__builtin_popcount(b & s) & 1) ? -(double)c[b] : (double)c[b];
    w[s] = a / n;
    if (s && (w[s] < 0 ? -w[s] : w[s]) > wmax) wmax = w[s] < 0 ? -w[s] : w[s];
  }
  // c[idx] = sum_s w_s (-1)^{parity(idx&s)} = c[0] - 2 sum_{s>0} w_s parity(idx&s)
  layer->n_terms = 0;
  layer->term_const = c[0];
  for (int s = 1; s < n; ++s) {
    double a = w[s] < 0 ? -w[s] : w[s];
    if (a <= 1e-9 * wmax) continue;
    layer->term_mask[layer->n_terms] = s;
    layer->term_coef[layer->n_terms] = (float)(-2.0 * w[s]);
    layer->n_terms++;
  }
  return TQ_OK;
}

extern "C" int tq_page_layout_init(tq_page_layout* L, int d, int mse_bits, int value_bits, int group_size, int dtype) {
  if (!L) return TQ_ENULL;
  if (d < 64 || d > 768 || (d & 63)) return TQ_EUNSUPPORTED;
  if (mse_bits < 1 || mse_bits > 4) return TQ_EUNSUPPORTED;
  if (value_bits != 2 && value_bits != 4 && value_bits != 8) return TQ_EUNSUPPORTED;
  if (group_size < 16 || d % group_size) return TQ_EINVAL;
  if (dtype < TQ_F32 || dtype > TQ_BF16) return TQ_EINVAL;
  const int es = dtype == TQ_F32 ? 4 : 2;
  L->d = d; L->mse_bits = mse_bits; L->value_bits = value_bits; L->group_size = group_size; L->dtype = dtype;
  L->key_lane_major = (d % 128 == 0 || d == 64) ? 1 : 0;
  int off = 0;
  L->off_keys = off;   off += (mse_bits + 1) * (d / 8) * TQ_PAGE_TOKENS;
  L->off_meta = off;   off += 8 * TQ_PAGE_TOKENS;
  L->off_vdata = off;  off += d * value_bits * 2;
  L->off_vscale = off; off += (d / group_size) * TQ_PAGE_TOKENS * es;
  L->off_vzero = off;  off += (d / group_size) * TQ_PAGE_TOKENS * es;
  L->page_bytes = (off + 127) & ~127;
  return TQ_OK;
}

extern "C" int tq_bucketize_pack(const float* y, int64_t n_vec, int d, const float* thresholds, int mse_bits,
                                 uint8_t* idx_out, void* stream) {
  if (!y || !thresholds || !idx_out) return TQ_ENULL;
  if (n_vec < 0 || d <= 0 || mse_bits < 1 || mse_bits > 8) return TQ_EINVAL;
  if (n_vec == 0) return TQ_OK;
  int64_t total = n_vec * idx_row_bytes(d, mse_bits);
  bucketize_pack_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
      y, n_vec, d, thresholds, mse_bits, idx_out);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

extern "C" int tq_sign_pack(const float* p, int64_t n_vec, int d, uint8_t* sign_out, void* stream) {
  if (!p || !sign_out) return TQ_ENULL;
  if (n_vec < 0 || d <= 0) return TQ_EINVAL;
  if (n_vec == 0) return TQ_OK;
  int64_t total = n_vec * ((d + 7) / 8);
  sign_pack_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(p, n_vec, d, sign_out);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

namespace tq {
template <class Source, class Sink>
int launch_key_mfma(const void* x, int dtype, const Source& src, const tq_layer& ly, const Sink& sink, int mse_only,
                    int64_t tiles, hipStream_t st);
}

template <class Source, class Sink>
static int launch_key(const void* x, int dtype, const Source& src, const tq_layer& ly, const Sink& sink, int mse_only,
                      int64_t tiles, hipStream_t st) {
  {  // matrix-core kernel when the layer carries split matrices and head_dim is 128 / 256
    int rc = launch_key_mfma(x, dtype, src, ly, sink, mse_only, tiles, st);
    if (rc != TQ_EUNSUPPORTED) return rc;
  }
  size_t smem = key_tile_smem(ly.d);
  dim3 grid((unsigned)tiles), block(ly.d);
#define TQ_LAUNCH_KEY(DT)                                                                              \
  {                                                                                                    \
    auto kern = key_tile_kernel<DT, Source, Sink>;                                                     \
    if (smem > 48 * 1024) {                                                                            \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
      if (e != hipSuccess) return (int)e;                                                              \
    }                                                                                                  \
    kern<<<grid, block, smem, st>>>(x, src, ly, sink, mse_only);                                       \
  }
  switch (dtype) {
    case TQ_F32: TQ_LAUNCH_KEY(TQ_F32) break;
    case TQ_F16: TQ_LAUNCH_KEY(TQ_F16) break;
    case TQ_BF16: TQ_LAUNCH_KEY(TQ_BF16) break;
    default: return TQ_EINVAL;
  }
#undef TQ_LAUNCH_KEY
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

static bool value_chunks_aligned(const void* v, const FlatSource& s) {
  return (uintptr_t)v % 16 == 0 && s.row_stride % 8 == 0;
}
static bool value_chunks_aligned(const void* v, const PagedSource& s) {
  return (uintptr_t)v % 16 == 0 && s.stride_b % 8 == 0 && s.stride_t % 8 == 0 && s.stride_h % 8 == 0 &&
         s.stride_blk % 8 == 0;
}

template <class Source, class Sink>
static int launch_value(const void* v, int dtype, const Source& src, int d, int gs, int bits, const Sink& sink,
                        int64_t tiles, hipStream_t st) {
  // 16-bit inputs with 2/4-bit codes on the usual head sizes take the chunked kernel
  if (dtype != TQ_F32 && (bits == 2 || bits == 4) && (d == 64 || d == 128 || d == 256) && gs >= 16 && gs <= 128 &&
      (gs & (gs - 1)) == 0 && value_chunks_aligned(v, src)) {
    const size_t sm = (size_t)(d / 8) * (TILE * (bits == 2 ? 2 : 4) + 16) + TILE * sizeof(int);
    const dim3 g2((unsigned)tiles), b2(TILE * d / 8);
#define TQ_LAUNCH_VC(DT, VB) value_chunk_kernel<DT, VB, Source, Sink><<<g2, b2, sm, st>>>(v, src, d, gs, sink)
    if (dtype == TQ_BF16) { if (bits == 2) TQ_LAUNCH_VC(TQ_BF16, 2); else TQ_LAUNCH_VC(TQ_BF16, 4); }
    else { if (bits == 2) TQ_LAUNCH_VC(TQ_F16, 2); else TQ_LAUNCH_VC(TQ_F16, 4); }
#undef TQ_LAUNCH_VC
    TQ_CHECK_LAUNCH();
    return TQ_OK;
  }
  size_t smem = value_tile_smem(d, gs);
  dim3 grid((unsigned)tiles), block(d);
#define TQ_LAUNCH_VAL(DT)                                                                              \
  {                                                                                                    \
    auto kern = value_tile_kernel<DT, Source, Sink>;                                                   \
    if (smem > 48 * 1024) {                                                                            \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
      if (e != hipSuccess) return (int)e;                                                              \
    }                                                                                                  \
    kern<<<grid, block, smem, st>>>(v, src, d, gs, bits, sink);                                        \
  }
  switch (dtype) {
    case TQ_F32: TQ_LAUNCH_VAL(TQ_F32) break;
    case TQ_F16: TQ_LAUNCH_VAL(TQ_F16) break;
    case TQ_BF16: TQ_LAUNCH_VAL(TQ_BF16) break;
    default: return TQ_EINVAL;
  }
#undef TQ_LAUNCH_VAL
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}

extern "C" int tq_quantize_keys(const void* x, int dtype, int64_t n_vec, int64_t row_stride, const tq_layer* layer,
                                uint8_t* idx_out, uint8_t* sign_out, void* norm_out, float* rnorm_out, float* y_dbg,
                                float* p_dbg, int mse_only, void* stream) {
  int rc = check_layer(layer, !mse_only);
  if (rc) return rc;
  if (!x || !idx_out || !norm_out) return TQ_ENULL;
  if (!mse_only && (!sign_out || !rnorm_out)) return TQ_ENULL;
  if (n_vec < 0 || row_stride < layer->d) return TQ_EINVAL;
  if (n_vec == 0) return TQ_OK;
  FlatSource src{n_vec, row_stride};
  KeyFlatSink sink{idx_out, sign_out, norm_out, rnorm_out, y_dbg, p_dbg};
  return launch_key(x, dtype, src, *layer, sink, mse_only, (n_vec + TILE - 1) / TILE, (hipStream_t)stream);
}

extern "C" int tq_quantize_values(const void* v, int dtype, int64_t n_vec, int64_t row_stride, int d, int group_size,
                                  int bits, uint8_t* data_out, void* scale_out, void* zero_out, void* stream) {
  if (!v || !data_out || !scale_out || !zero_out) return TQ_ENULL;
  if (d < 64 || d > 768 || (d & 63)) return TQ_EUNSUPPORTED;
  if (bits != 2 && bits != 4 && bits != 8) return TQ_EUNSUPPORTED;
  if (group_size < 16 || d % group_size || n_vec < 0 || row_stride < d) return TQ_EINVAL;
  if (n_vec == 0) return TQ_OK;
  FlatSource src{n_vec, row_stride};
  ValFlatSink sink{data_out, scale_out, zero_out};
  return launch_value(v, dtype, src, d, group_size, bits, sink, (n_vec + TILE - 1) / TILE, (hipStream_t)stream);
}

// Side stream of the calling thread on the current device (created on first use, default priority,
// kept until the process ends), with the two events of the fork / join.  nullptr when it cannot be
// had: the caller then launches on its own stream.
namespace {
struct SideLane { hipStream_t stream = nullptr; hipEvent_t fork = nullptr, join = nullptr; bool tried = false; };
constexpr int64_t SIDE_MIN_TILES = 4096;       // below this the fork / join costs more than it hides
constexpr int SIDE_MAX_DEVICES = 16;
SideLane* side_lane() {
  static thread_local SideLane lanes[SIDE_MAX_DEVICES];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SIDE_MAX_DEVICES) return nullptr;
  SideLane& l = lanes[dev];
  if (!l.tried) {
    l.tried = true;
    if (hipStreamCreateWithFlags(&l.stream, hipStreamNonBlocking) != hipSuccess) l.stream = nullptr;
    if (l.stream && (hipEventCreateWithFlags(&l.fork, hipEventDisableTiming) != hipSuccess ||
                     hipEventCreateWithFlags(&l.join, hipEventDisableTiming) != hipSuccess))
      l.stream = nullptr;
  }
  return l.stream ? &l : nullptr;
}
}  // namespace

// keys and values of the runs described by `src` into the pages of `block_table`
static int append_runs(const void* k, const void* v, int dtype, const PagedSource& src, const int32_t* block_table,
                       int max_pages, const tq_layer* layer, const tq_page_layout* layout, uint8_t* pool,
                       int64_t num_pages, void* stream) {
  int64_t tiles = (int64_t)src.B * src.tiles_per_seq * src.H;
  const int pool_pages = (int)(num_pages < 0x7fffffff ? num_pages : 0x7fffffff);    // page numbers are int32
  KeyPagedSink ks{pool, block_table, max_pages, pool_pages, *layout};
  ValPagedSink vs{pool, block_table, max_pages, pool_pages, *layout};
  int rc;
  // Large appends run the value kernel beside the key kernel: the key kernel leaves a quarter of the
  // registers and issue slots of every SIMD free, which the small value wavefronts fill (the two
  // kernels write disjoint bytes of the pages).  The value kernel goes to a side stream that is
  // forked from and joined back into the caller's stream with events, so the call stays ordered
  // on `stream` like any other.
  // (measurement knob: one of the two kernels alone, to time it without the other beside it)
  const int parts = opt_append_parts.load();
  if (parts == 1) return launch_key(k, dtype, src, *layer, ks, 0, tiles, (hipStream_t)stream);
  if (parts == 2)
    return launch_value(v, dtype, src, layer->d, layout->group_size, layout->value_bits, vs, tiles, (hipStream_t)stream);
  if (tiles >= SIDE_MIN_TILES) {
    if (SideLane* lane = side_lane()) {
      hipStream_t st = (hipStream_t)stream;
      if (hipEventRecord(lane->fork, st) == hipSuccess && hipStreamWaitEvent(lane->stream, lane->fork, 0) == hipSuccess) {
        rc = launch_value(v, dtype, src, layer->d, layout->group_size, layout->value_bits, vs, tiles, lane->stream);
        hipError_t e1 = hipEventRecord(lane->join, lane->stream);
        int rc2 = launch_key(k, dtype, src, *layer, ks, 0, tiles, st);
        hipError_t e2 = e1 == hipSuccess ? hipStreamWaitEvent(st, lane->join, 0) : e1;
        if (rc) return rc;
        if (rc2) return rc2;
        return e2 == hipSuccess ? TQ_OK : (int)e2;
      }
    }
  }
  rc = launch_key(k, dtype, src, *layer, ks, 0, tiles, (hipStream_t)stream);
  if (rc) return rc;
  return launch_value(v, dtype, src, layer->d, layout->group_size, layout->value_bits, vs, tiles, (hipStream_t)stream);
}

extern "C" int tq_append_kv_paged(const void* k, const void* v, int dtype, int B, int T, int H, int64_t stride_b,
                                  int64_t stride_t, int64_t stride_h, const int32_t* start_pos,
                                  const int32_t* block_table, int max_pages, const tq_layer* layer,
                                  const tq_page_layout* layout, uint8_t* pool, int64_t num_pages, void* stream) {
  int rc = check_layer(layer, true);
  if (rc) return rc;
  if (!k || !v || !block_table || !layout || !pool) return TQ_ENULL;
  if (dtype != layout->dtype || layout->d != layer->d || layout->mse_bits != layer->mse_bits) return TQ_EINVAL;
  if (B < 0 || T < 0 || H <= 0 || max_pages <= 0 || num_pages <= 0) return TQ_EINVAL;
  if (B == 0 || T == 0) return TQ_OK;
  // without start positions the run is known on the host: it has to fit the block table (with start
  // positions, the kernels skip whatever falls outside the table)
  if (!start_pos && T > (int64_t)max_pages * TILE) return TQ_EINVAL;
  // a run of T tokens starting anywhere inside a page touches at most this many pages
  // (the run may begin at any of the 16 slots of its first page when start_pos is given)
  const int tiles_per_seq = start_pos ? (T + TILE - 2) / TILE + 1 : (T + TILE - 1) / TILE;
  PagedSource src{B, T, H, tiles_per_seq, stride_b, stride_t, stride_h, start_pos};
  return append_runs(k, v, dtype, src, block_table, max_pages, layer, layout, pool, num_pages, stream);
}

extern "C" int tq_append_kv_ragged(const void* k, const void* v, int dtype, int B, int T_max, int H, int64_t stride_t,
                                   int64_t stride_h, const int32_t* row0, const int32_t* run_len,
                                   const int32_t* start_pos, const int32_t* block_table, int max_pages,
                                   const tq_layer* layer, const tq_page_layout* layout, uint8_t* pool,
                                   int64_t num_pages, void* stream) {
  int rc = check_layer(layer, true);
  if (rc) return rc;
  if (!k || !v || !row0 || !run_len || !start_pos || !block_table || !layout || !pool) return TQ_ENULL;
  if (dtype != layout->dtype || layout->d != layer->d || layout->mse_bits != layer->mse_bits) return TQ_EINVAL;
  if (B < 0 || T_max < 0 || H <= 0 || max_pages <= 0 || num_pages <= 0) return TQ_EINVAL;
  if (B == 0 || T_max == 0) return TQ_OK;
  const int tiles_per_seq = (T_max + TILE - 2) / TILE + 1;      // a run may begin at any slot of its first page
  PagedSource src{B, T_max, H, tiles_per_seq, 0, stride_t, stride_h, start_pos};
  src.run_len = run_len;
  src.row0 = row0;
  return append_runs(k, v, dtype, src, block_table, max_pages, layer, layout, pool, num_pages, stream);
}

extern "C" int tq_append_kv_from_blocks(const void* k_cache, const void* v_cache, int dtype, int B, int T, int H,
                                        int64_t stride_blk, int64_t stride_t, int64_t stride_h,
                                        const int32_t* src_table, int src_stride, const int32_t* start_pos,
                                        const int32_t* run_len, const int32_t* block_table, int max_pages,
                                        const tq_layer* layer, const tq_page_layout* layout, uint8_t* pool,
                                        int64_t num_pages, void* stream) {
  int rc = check_layer(layer, true);
  if (rc) return rc;
  if (!k_cache || !v_cache || !src_table || !block_table || !layout || !pool) return TQ_ENULL;
  if (dtype != layout->dtype || layout->d != layer->d || layout->mse_bits != layer->mse_bits) return TQ_EINVAL;
  if (B < 0 || T < 0 || H <= 0 || max_pages <= 0 || num_pages <= 0 || src_stride <= 0) return TQ_EINVAL;
  if (B == 0 || T == 0) return TQ_OK;
  if (!start_pos && !run_len && T > (int64_t)max_pages * TILE) return TQ_EINVAL;
  const int tiles_per_seq = start_pos ? (T + TILE - 2) / TILE + 1 : (T + TILE - 1) / TILE;
  PagedSource src{B, T, H, tiles_per_seq, 0, stride_t, stride_h, start_pos};
  src.src_table = src_table;
  src.src_stride = src_stride;
  src.stride_blk = stride_blk;
  src.run_len = run_len;
  return append_runs(k_cache, v_cache, dtype, src, block_table, max_pages, layer, layout, pool, num_pages, stream);
}

extern "C" int tq_pool_export(const uint8_t* pool, int64_t num_pages, int H, const int32_t* block_table, int n_tok,
                              const tq_page_layout* layout, uint8_t* idx, uint8_t* signs, void* norms, float* rnorms,
                              uint8_t* v_data, void* v_scales, void* v_zeros, void* stream) {
  if (!pool || !block_table || !layout || !idx || !signs || !norms || !rnorms || !v_data || !v_scales || !v_zeros)
    return TQ_ENULL;
  if (H <= 0 || n_tok < 0 || num_pages <= 0) return TQ_EINVAL;
  if (n_tok == 0) return TQ_OK;
  const tq_page_layout& L = *layout;
  const int pool_pages = (int)(num_pages < 0x7fffffff ? num_pages : 0x7fffffff);
  if ((L.value_bits == 2 || L.value_bits == 4 || L.value_bits == 8) && L.d % 64 == 0 && L.off_vdata % 4 == 0 &&
      (uintptr_t)idx % 4 == 0 && (uintptr_t)signs % 4 == 0 && (uintptr_t)v_data % 4 == 0) {
    dim3 g2((n_tok + TILE - 1) / TILE, H), b2(256);
    const size_t sm = (size_t)L.d * 2 * L.value_bits;
    pool_export_words_kernel<<<g2, b2, sm, (hipStream_t)stream>>>(pool, pool_pages, H, block_table, n_tok, L, (uint32_t*)idx,
                                                                 (uint32_t*)signs, norms, rnorms, (uint32_t*)v_data,
                                                                 v_scales, v_zeros);
    TQ_CHECK_LAUNCH();
    return TQ_OK;
  }
  dim3 grid((n_tok + TILE - 1) / TILE, H), block(64);
  pool_export_kernel<<<grid, block, 0, (hipStream_t)stream>>>(pool, pool_pages, H, block_table, n_tok, *layout, idx, signs, norms,
                                                             rnorms, v_data, v_scales, v_zeros);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}
