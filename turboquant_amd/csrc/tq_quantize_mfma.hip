// Key quantiser on the matrix cores (gfx950, bf16 MFMA 16x16x32).
//
// The three d x d contractions of the reference (y = u Pi^T, x_hat = c[idx] Pi,
// p = r S^T; quantizer.py:141,160,248) need fp32-class accuracy, because an index
// or a sign flips whenever a result crosses a threshold.  Every fp32 number is the
// exact sum of three bf16 numbers (8 + 8 + 8 significand bits), so each operand is
// split into bf16 terms and the product is assembled from bf16 MFMAs whose partial
// products are exact; terms (a, b) with a + b > 2 are below fp32 resolution and are
// skipped.  The matrices are split once per layer on the host and stored in the order
// the MFMA operands are loaded in; inputs that already are bf16 need a single term.
//
// Workgroups (4 wavefronts) are persistent: two per compute unit (about 75 KB of LDS
// each), each looping over groups of TT = 8192/d vectors (TT/16 tiles of 16).  The next
// group's vectors are fetched into registers while the current group is worked on (the
// tile lookups behind their addresses are uniform and go through the scalar cache), and
// the matrix operand of a contraction is requested slice by slice while the previous
// contraction runs, so no global-memory latency sits on the critical path.  The vectors' operand terms sit in LDS (row
// stride padded so that the 16 rows of an MFMA operand fall into different banks);
// a wavefront owns d/64 column tiles of the output for all TT vectors, keeps the
// matrix terms of the current 32-wide slice of the contraction in registers (next
// slice prefetched), and re-reads the vector terms from LDS.  The matrix rows are
// the MFMA's row operand, so a lane ends up with four consecutive output columns
// of one vector: terms for the next contraction go back to LDS as 8-byte writes and
// the index / sign bits of a vector are gathered into 32-bit plane words with two
// lane-swap instructions.  The three contractions are separated by workgroup barriers
// because each needs complete rows of the previous result.

#include <atomic>

#include "tq_quantize.h"
#include "tq_decode_mfma.h"
#include "tq_options.h"
#include <hip/hip_ext.h>

namespace tq {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ f32x4 mfma_bf16(const u32x4& rows, const u32x4& cols, f32x4 c) {
  bf16x8 av, bv;
  __builtin_memcpy(&av, &rows, 16);
  __builtin_memcpy(&bv, &cols, 16);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, c, 0, 0, 0);
}

// fp6 (A: 16 rows x 128) x fp4 (B: 128 x 16) MFMA with per-lane power-of-two block scales (E8M0 codes); SEL
// picks the byte of scale_a that holds the code.  Only six dwords of `a` and the four of `b` are read.
template <int SEL>
__device__ __forceinline__ f32x4 mfma_fp6_fp4(const i32x8& a, const u32x4& b, f32x4 c, int scale_a, int scale_b) {
  const i32x8 bv = {(int)b[0], (int)b[1], (int)b[2], (int)b[3], 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, bv, c, 2 /*A: fp6 e2m3*/, 4 /*B: fp4*/, SEL, scale_a, 0, scale_b);
}

// two fp32 -> packed bf16 (first value in the low half), round to nearest even
__device__ __forceinline__ uint32_t cvt_pk_bf16(float a, float b) {
  f32x2 v = {a, b};
  bf16x2 r = __builtin_convertvector(v, bf16x2);
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}

// (v0, v1) = t[0] + t[1] + t[2] lane-wise, each term a packed pair of bf16: a term is
// the rounding of what the previous terms left, and every remainder is exact in fp32
__device__ __forceinline__ void split3_pk(float v0, float v1, uint32_t (&t)[3]) {
  t[0] = cvt_pk_bf16(v0, v1);
  float r0 = v0 - __uint_as_float(t[0] << 16), r1 = v1 - __uint_as_float(t[0] & 0xffff0000u);
  t[1] = cvt_pk_bf16(r0, r1);
  r0 -= __uint_as_float(t[1] << 16);
  r1 -= __uint_as_float(t[1] & 0xffff0000u);
  t[2] = cvt_pk_bf16(r0, r1);
}

// N consecutive elements of the input dtype from LDS (16-byte aligned) as fp32
template <int DT, int N>
__device__ __forceinline__ void load_run(const typename Elem<DT>::storage* p, float (&out)[N]) {
  if constexpr (DT == TQ_F32) {
#pragma unroll
    for (int c = 0; c < N; c += 4) {
      const f32x4 v = *(const f32x4*)(p + c);
      out[c] = v.x; out[c + 1] = v.y; out[c + 2] = v.z; out[c + 3] = v.w;
    }
  } else if constexpr (N % 8 == 0) {
#pragma unroll
    for (int c = 0; c < N; c += 8) {
      const u32x4 v = *(const u32x4*)(p + c);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        out[c + 2 * k] = Elem<DT>::load(&v, 2 * k);
        out[c + 2 * k + 1] = Elem<DT>::load(&v, 2 * k + 1);
      }
    }
  } else {
    static_assert(N == 4, "runs of 4 or a multiple of 8");
    const u32x2 v = *(const u32x2*)p;
#pragma unroll
    for (int k = 0; k < 4; ++k) out[k] = Elem<DT>::load(&v, k);
  }
}

template <int DT> struct InTerms;                       // bf16 terms that represent a value of the input dtype exactly
template <> struct InTerms<TQ_BF16> { static constexpr int N = 1; };
template <> struct InTerms<TQ_F16> { static constexpr int N = 2; };
template <> struct InTerms<TQ_F32> { static constexpr int N = 3; };

constexpr int KQ_WAVES = 4;
constexpr int KQ_THREADS = KQ_WAVES * 64;
constexpr int KQ_MAX_PLANES = 5;                        // 4 index bits + sign

template <int D>
struct KeyGeom {
  static constexpr int TT = 8192 / D;                   // vectors per workgroup
  static constexpr int MT = TT / 16;                    // 16-vector tiles per workgroup
  static constexpr int NPW = D / 16 / KQ_WAVES;         // output column tiles per wavefront
  static constexpr int KB = D / 32;                     // 32-wide slices of the contraction
  static constexpr int RS = D + 8;                      // LDS row stride of a term tile, in bf16
  static constexpr int W = D / 32;                      // 32-bit words per bit plane of a vector
  static constexpr int TPR = KQ_THREADS / TT;           // threads that share a vector in the norm pass
  static constexpr int SEG = D / TPR;                   // = 32 elements per thread
};

template <int DT, int D>
struct KeySmem {
  using G = KeyGeom<D>;
  using S = typename Elem<DT>::storage;
  static constexpr int XRS = D + 16 / (int)sizeof(S);                       // padded row of the input tile
  static constexpr size_t off_x = 0;
  static constexpr size_t off_terms = (size_t)G::TT * XRS * sizeof(S);      // 3 term tiles [TT][RS] bf16
  static constexpr size_t off_planes = off_terms + 3 * (size_t)G::TT * G::RS * 2;   // [plane][TT][W] words
  static constexpr size_t off_small = off_planes + (size_t)KQ_MAX_PLANES * G::TT * G::W * 4;
  // snorm[TT] srn[TT] spart[4][TT] svalid[TT] sthr[16] slut[16] (8 bytes each)
  static constexpr size_t bytes = off_small + (size_t)G::TT * (3 + KQ_WAVES) * 4 + 16 * 4 + 16 * 8;
};

// Register copy of the matrix operand: BUF slices of 32 contraction indices for the
// wavefront's column tiles.  head_dim 128 holds a whole contraction (BUF = KB); head_dim 256
// keeps a ring that runs BUF - 1 slices ahead.
template <int D>
struct MatRegs {
  static constexpr int BUF = D == 128 ? 4 : 2;
  u32x4 b[BUF][KeyGeom<D>::NPW][3];
};

// m_terms: the three bf16 term matrices in MFMA-operand order.  For term b, tile of 16 output rows ct
// and slice of 32 contraction indices kblk, the 64 lanes' 16-byte operands lie one after the other
// (lane n + 16 kb holds M[16 ct + n][32 kblk + 8 kb ..+8]), so a wavefront's load of one operand is one
// contiguous kilobyte.  (Row-major storage would make every quarter-wavefront touch 16 cache lines.)
template <int D>
__device__ __forceinline__ void load_slice(const uint16_t* __restrict__ m_terms, int wave, int lane, int kblk,
                                           u32x4 (&dst)[KeyGeom<D>::NPW][3]) {
  // one 32-bit per-lane byte offset; everything else is a uniform constant added to the base pointer
  constexpr int KB = KeyGeom<D>::KB, NPW = KeyGeom<D>::NPW;
  const uint32_t lane_off = (uint32_t)((wave * NPW * KB * 64 + lane) * 16);
#pragma unroll
  for (int c = 0; c < NPW; ++c) {
#pragma unroll
    for (int b = 0; b < 3; ++b) {
      const char* base = (const char*)m_terms + ((size_t)(b * (D / 16) + c) * KB + kblk) * 1024;
      dst[c][b] = *(const u32x4*)(base + lane_off);
    }
  }
}

template <int D>
__device__ __forceinline__ void prefetch_matrix(const uint16_t* __restrict__ m_terms, int wave, int lane, MatRegs<D>& mr) {
#pragma unroll
  for (int k = 0; k < MatRegs<D>::BUF; ++k) load_slice<D>(m_terms, wave, lane, k, mr.b[k]);
}

// One contraction: out[t][n] = sum_k A[t][k] * M[n][k] for the wavefront's column tiles.
// a_terms tiles in LDS ([term][TT][RS] bf16); the first BUF slices of M are in `mr` already.
// NA vector terms, 3 matrix terms, pairs with a + b <= 2.
// acc[m][c][i] = out[16 m + (lane & 15)][16 (wave NPW + c) + 4 (lane >> 4) + i].
// As soon as a slice's registers are free they are refilled: with a later slice of M while
// there is one, then with the first BUF slices of m_next, the matrix of the contraction that
// follows.  Those loads have the rest of this contraction and the epilogue to arrive, and
// the requests of a workgroup are spread out instead of coming in one burst.
// (ML: the group's first ML tiles hold vectors; the others are not computed)
template <int D, int NA, bool REFILL = true, int ML = KeyGeom<D>::MT>
__device__ __forceinline__ void contract(const uint16_t* a_terms, const uint16_t* __restrict__ m_terms,
                                         const uint16_t* __restrict__ m_next, int wave, int lane, MatRegs<D>& mr,
                                         f32x4 (&acc)[KeyGeom<D>::MT][KeyGeom<D>::NPW]) {
  using Gm = KeyGeom<D>;
  constexpr int MT = Gm::MT, NPW = Gm::NPW, KB = Gm::KB, RS = Gm::RS, BUF = MatRegs<D>::BUF;
  const int n = lane & 15, kb = lane >> 4;
#pragma unroll
  for (int m = 0; m < ML; ++m)
#pragma unroll
    for (int c = 0; c < NPW; ++c) acc[m][c] = f32x4{0, 0, 0, 0};
#pragma unroll
  for (int kblk = 0; kblk < KB; ++kblk) {
    // consecutive MFMAs go to different accumulators
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      u32x4 av[MT];
#pragma unroll
      for (int m = 0; m < ML; ++m)
        av[m] = *(const u32x4*)(a_terms + ((size_t)a * Gm::TT + 16 * m + n) * RS + 32 * kblk + 8 * kb);
#pragma unroll
      for (int b = 0; b < 3; ++b)
        if (a + b <= 2) {
#pragma unroll
          for (int m = 0; m < ML; ++m)
#pragma unroll
            for (int c = 0; c < NPW; ++c) acc[m][c] = mfma_bf16(mr.b[kblk % BUF][c][b], av[m], acc[m][c]);
        }
    }
    if (kblk + BUF < KB) load_slice<D>(m_terms, wave, lane, kblk + BUF, mr.b[kblk % BUF]);
    else if (REFILL) load_slice<D>(m_next, wave, lane, kblk + BUF - KB, mr.b[kblk % BUF]);
  }
}

// OR / sum of a value over the four lanes that hold the same vector (lane & 15 equal); the result is valid in
// the first of them (lanes 0..15).  The lane-swap instructions move rows of 16 / halves of 32 lanes through
// the vector ALU: no LDS round trip and nothing to wait for.
__device__ __forceinline__ uint32_t or_over_kb(uint32_t v) {
  v |= (uint32_t)__builtin_amdgcn_permlane32_swap(v, v, false, false)[1];       // lanes 0..31: | lane + 32
  v |= (uint32_t)__builtin_amdgcn_permlane16_swap(v, v, false, false)[1];       // lanes 0..15: | lane + 16
  return v;
}
// sum over groups of N neighbouring lanes (N = 4, 8 or 16, inside a row of 16) with DPP moves: quad swaps,
// then half-row / row mirrors (every lane of a quad already holds the quad's sum, so a mirror pairs the quads)
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int N>
__device__ __forceinline__ float sum_lanes(float v) {
  static_assert(N == 4 || N == 8 || N == 16, "4, 8 or 16 lanes");
  v += dpp_mov<0xB1>(v);
  v += dpp_mov<0x4E>(v);
  if (N >= 8) v += dpp_mov<0x141>(v);
  if (N >= 16) v += dpp_mov<0x140>(v);
  return v;
}
__device__ __forceinline__ float sum_over_kb(float f) {
  f += __uint_as_float(__builtin_amdgcn_permlane32_swap(__float_as_uint(f), __float_as_uint(f), false, false)[1]);
  f += __uint_as_float(__builtin_amdgcn_permlane16_swap(__float_as_uint(f), __float_as_uint(f), false, false)[1]);
  return f;
}

// Staging of a group's vectors: a thread holds its 16-byte chunks of the NEXT group in registers while the
// current group is worked on, so the latency of the loads is never waited for.  The KQ_THREADS chunks of
// one round lie in one tile.  Everything that depends on the tile number is uniform and comes from one
// walk over the group's MT consecutive tiles (TileAddr); a lane only adds its own offset, which is the
// same for every group (slot * row stride + chunk, kept in registers on purpose).
template <int DT, int D, class Source>
struct XStage {
  using S = typename Elem<DT>::storage;
  using Gm = KeyGeom<D>;
  static constexpr int CH = 16 / (int)sizeof(S);                // elements per 16-byte chunk
  static constexpr int CPR = D / CH;                            // chunks per vector
  static constexpr int PER = Gm::TT * CPR / KQ_THREADS;         // rounds
  static constexpr int RPR = KQ_THREADS / CPR;                  // vectors per round (<= 16)
  static constexpr int NSL = TILE / RPR;                        // rounds per tile = slots a thread serves
  static_assert(RPR <= TILE && TILE % RPR == 0 && PER == Gm::MT * NSL, "a round of chunks stays inside one tile");
  u32x4 xbuf[PER];
  unsigned xok = 0;
  TileAddr ta[Gm::MT];                                          // tiles of the group looked up last
  bool live[Gm::MT];
  int w_b = 0, w_lpage = 0, w_h = 0;                            // (paged) where the tile this wavefront writes goes
  int64_t lane_off[NSL];
  int slot[NSL];

  __device__ __forceinline__ void init(const Source& src, int tid) {
    const int tr = tid / CPR, ck = tid % CPR;
#pragma unroll
    for (int k = 0; k < NSL; ++k) {
      slot[k] = tr + RPR * k;
      lane_off[k] = (int64_t)slot[k] * src.slot_stride() + ck * CH;
    }
  }
  // uniform part for `group`: tile addresses, and (paged sources) the coordinates of tile group * MT + wtile
  // (ML: tiles of a group that hold vectors - groups are ML tiles apart; the other MT - ML are not loaded)
  template <int ML = Gm::MT>
  __device__ __forceinline__ void lookup(const Source& src, int64_t group, int64_t n_tiles, int wtile) {
    const int64_t tile0 = group * ML;
    const int64_t first = tile0 < n_tiles ? tile0 : 0;
#pragma unroll
    for (int m = 0; m < Gm::MT; ++m) live[m] = m < ML && tile0 + m < n_tiles;
    if constexpr (std::is_same<Source, PagedSource>::value) {
      PagedSource::Coord c[Gm::MT];
      int lpage[Gm::MT];
      c[0] = src.coord(first);
#pragma unroll
      for (int m = 1; m < Gm::MT; ++m) { c[m] = c[m - 1]; src.next(c[m]); }
      src.template tile_addrs<Gm::MT>(c, ta, lpage);
#pragma unroll
      for (int m = 0; m < Gm::MT; ++m)
        if (m == wtile) { w_b = c[m].b; w_lpage = lpage[m]; w_h = c[m].h; }
    } else {
#pragma unroll
      for (int m = 0; m < Gm::MT; ++m) ta[m] = src.tile_addr(first + m);
    }
  }
  // request the chunks of the group looked up last (unconditional loads: a load under a branch makes every
  // later wait a wait for all loads; slots that do not exist read the first vector and are zeroed when stored)
  __device__ __forceinline__ void issue(const void* x) {
    xok = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int m = j / NSL, k = j % NSL;
      const bool ok = live[m] && slot[k] >= ta[m].lo && slot[k] < ta[m].hi;
      xbuf[j] = *(const u32x4*)((const S*)x + (ok ? ta[m].base + lane_off[k] : 0));
      xok |= (unsigned)ok << j;
    }
  }
  // registers -> the LDS tile [TT][XRS], validity flags
  template <int XRS>
  __device__ __forceinline__ void store(S* sx, int* svalid, int tid) const {
    const int tr = tid / CPR, ck = tid % CPR;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const bool ok = (xok >> j) & 1;
      *(u32x4*)(sx + (RPR * j + tr) * XRS + ck * CH) = ok ? xbuf[j] : u32x4{0, 0, 0, 0};
      if (ck == 0) svalid[RPR * j + tr] = ok;
    }
  }
};

// MSE_ONLY (the stage-1 quantiser alone: no residual, no signs) is a template parameter: as a
// run-time flag it adds control flow that costs the register allocator its footing.
//
// FX (head_dim 128, codebooks with single-bit Walsh terms): the centroid contraction x_hat = c[idx] Pi runs on
// the block-scaled fp6 x fp4 MFMA (16x16x128, four times the bf16 rate).  c[idx] = c0 + sum_p k_p bit_p(idx), so
// x_hat = c0 colsum(Pi) + sum_p k_p (plane_p Pi): the index bit planes, which are being built anyway, are the fp4
// operand (a plane word turns into fp4 codes with four ANDs), and Pi^T is the fp6 operand, cut into five
// fp6 digits per value on the host (good to 2^-23 of a block's largest value: below the rounding noise of an
// fp32 product sum).  10 MFMAs per 16 x 16 tile instead of 24, and no centroid terms go through the LDS.
// ML (1 or the MT tiles of a group): small appends - the page write of a decode step - give every 16-vector tile a
// workgroup of its own that computes one tile instead of four, a quarter of the instructions behind one another.
template <int DT, int D, bool MSE_ONLY, bool FX, class Source, class Sink, int ML = KeyGeom<D>::MT>
__global__ void __launch_bounds__(KQ_THREADS, 2)
key_mfma_kernel(const void* __restrict__ x, Source src, tq_layer ly, Sink sink, int64_t n_tiles) {
  static_assert(!FX || (D == 128 && !MSE_ONLY), "the fp6 centroid contraction: head_dim 128, full quantiser");
  constexpr int mse_only = MSE_ONLY;
  using E = Elem<DT>;
  using S = typename E::storage;
  using Gm = KeyGeom<D>;
  using Sm = KeySmem<DT, D>;
  constexpr int TT = Gm::TT, MT = Gm::MT, NPW = Gm::NPW, RS = Gm::RS, W = Gm::W, NA1 = InTerms<DT>::N;
  constexpr int XRS = Sm::XRS, TPR = Gm::TPR, SEG = Gm::SEG;
  const int tid0 = threadIdx.x, wave0 = __builtin_amdgcn_readfirstlane(tid0 >> 6);
  const int mb = ly.mse_bits, n_thr = (1 << mb) - 1;
  const int64_t n_groups = (n_tiles + ML - 1) / ML;             // a group = the TT vectors of one pass
  MatRegs<D> mr;
  prefetch_matrix<D>(ly.Pi_split, wave0, tid0 & 63, mr);        // in flight while the vectors are staged

  extern __shared__ __align__(16) unsigned char smem[];
  S* sx = (S*)(smem + Sm::off_x);                               // [TT][XRS] input
  uint16_t* terms = (uint16_t*)(smem + Sm::off_terms);          // [3][TT][RS]: unit vector, then centroids, then residual
  uint32_t* spl = (uint32_t*)(smem + Sm::off_planes);           // [plane][TT][W]
  float* snorm = (float*)(smem + Sm::off_small);                // [TT]
  float* srn = snorm + TT;                                      // [TT]
  float* spart = srn + TT;                                      // [KQ_WAVES][TT] partial sums of r^2
  int* svalid = (int*)(spart + KQ_WAVES * TT);                  // [TT]
  float* sthr = (float*)(svalid + TT);                          // [16]
  u32x2* slut = (u32x2*)(sthr + 16);                            // [16] bf16 terms of a centroid: {t0 | t1 << 16, t2}

  if (tid0 < n_thr) sthr[tid0] = ly.thresholds[tid0];
  if (tid0 < (1 << mb)) {
    uint32_t t[3];
    split3_pk(ly.centroids[tid0], 0.0f, t);
    slut[tid0] = u32x2{(t[0] & 0xffffu) | (t[1] << 16), t[2] & 0xffffu};
  }
  // FX: Pi^T as fp6 digits (this wavefront's column tiles, resident), their block scales, the plane
  // coefficients and the constant part c0 colsum(Pi) of this lane's output columns
  constexpr int FXT = 5;
  int fs0[FX ? KeyGeom<D>::NPW : 1], fs1[FX ? KeyGeom<D>::NPW : 1];
  float fk[2] = {0.0f, 0.0f};
  f32x4 fconst[FX ? KeyGeom<D>::NPW : 1];
  if constexpr (FX) {
    const int lane0 = tid0 & 63;
#pragma unroll
    for (int c = 0; c < NPW; ++c) {
      const int ct = wave0 * NPW + c;
      fs0[c] = (int)ly.PiT_fp6_scale[((size_t)ct * 64 + lane0) * 2];
      fs1[c] = (int)ly.PiT_fp6_scale[((size_t)ct * 64 + lane0) * 2 + 1];
      const float* cs = ly.Pi_colsum + 16 * ct + 4 * (lane0 >> 4);
      fconst[c] = f32x4{ly.term_const * cs[0], ly.term_const * cs[1], ly.term_const * cs[2], ly.term_const * cs[3]};
    }
    for (int t = 0; t < ly.n_terms; ++t)                          // plane p holds index bit mb - 1 - p
      for (int p = 0; p < 2; ++p)
        if (p < mb && ly.term_mask[t] == (1 << (mb - 1 - p))) fk[p] = ly.term_coef[t];
  }
  // (1) staging (XStage): the next group's chunks wait in registers while the current group is worked on
  XStage<DT, D, Source> stg;
  stg.init(src, tid0);
  stg.template lookup<ML>(src, blockIdx.x, n_tiles, wave0 % ML);
  stg.issue(x);

  for (int64_t g = blockIdx.x; g < n_groups; g += gridDim.x) {
  // The thread index is re-read through an opaque copy in every pass: otherwise the compiler
  // hoists all per-thread address arithmetic out of this loop and spills it.
  int tid = tid0, wave = wave0;
  asm volatile("" : "+v"(tid), "+s"(wave));
  const int lane = tid & 63, n = lane & 15, kb = lane >> 4;
  const int64_t tile0 = g * ML;
  // coordinates of the tile this wavefront writes: looked up one pass ago together with this group's loads;
  // then the lookups of the group to fetch next (long before issue() needs them)
  const int wr_b = stg.w_b, wr_lpage = stg.w_lpage, wr_h = stg.w_h;
  stg.template lookup<ML>(src, g + gridDim.x, n_tiles, wave % ML);
  // page of that tile, read now so that the write phase does not wait for it (a page outside the table or
  // the pool comes back as -1 and is not written)
  int64_t wpage = 0;
  if constexpr (!std::is_same<Sink, KeyFlatSink>::value) {
    if (tile0 + wave % ML < n_tiles) wpage = checked_page(sink.block_table, sink.max_pages, sink.num_pages, wr_b, wr_lpage);
  }
  stg.template store<XRS>(sx, svalid, tid);
  __syncthreads();
  // (2) norm, unit vector in the input dtype (quantizer.py:136-138), its bf16 terms.
  //     TPR neighbouring threads share a vector, 32 coordinates each.
  {
    const int t = tid / TPR, seg = tid % TPR;
    float xs[SEG];
    load_run<DT, SEG>(sx + t * XRS + seg * SEG, xs);
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < SEG; ++c) ss += xs[c] * xs[c];
    ss = sum_lanes<TPR>(ss);
    const float nrm = E::round(sqrtf(ss));
    const float den = E::round(nrm + 1e-10f);
    if (seg == 0) snorm[t] = nrm;
    if constexpr (DT == TQ_BF16) {
      // Quotients of bf16 numbers, rounded to bf16: a / den is either exactly a rounding tie or at least
      // 2^-17 (relative) away from one, so q0 = a (1/den) with one residual correction, which is exact
      // for a tie, rounds like the correctly rounded quotient.  (Compared with the division over every
      // pair of bf16 numbers with |a| <= 2 den and den in the range below, also with the reciprocal an ulp
      // off either way: the only difference is that a = -0 gives +0, which no product sum can tell apart.)  |x_i| <= 2 den holds for any finite norm.
      if (den > 0x1p-60f && den < 0x1p60f) {
        const float rden = __builtin_amdgcn_rcpf(den);          // any reciprocal good to an ulp will do
#pragma unroll
        for (int c = 0; c < SEG; ++c) {
          const float q0 = xs[c] * rden;
          xs[c] = fmaf(fmaf(-q0, den, xs[c]), rden, q0);
        }
      } else {
#pragma unroll
        for (int c = 0; c < SEG; ++c) xs[c] = xs[c] / den;
      }
    }
#pragma unroll
    for (int c8 = 0; c8 < SEG; c8 += 8) {
      uint32_t pk[3][4];
#pragma unroll
      for (int c = 0; c < 8; c += 2) {
        if constexpr (DT == TQ_BF16) {                          // the rounded quotient is its own single term
          pk[0][c >> 1] = cvt_pk_bf16(xs[c8 + c], xs[c8 + c + 1]);
        } else {
          uint32_t tm[3];
          split3_pk(E::round(xs[c8 + c] / den), E::round(xs[c8 + c + 1] / den), tm);
#pragma unroll
          for (int a = 0; a < 3; ++a) pk[a][c >> 1] = tm[a];
        }
      }
#pragma unroll
      for (int a = 0; a < NA1; ++a)
        *(u32x4*)(terms + ((size_t)a * TT + t) * RS + seg * SEG + c8) = u32x4{pk[a][0], pk[a][1], pk[a][2], pk[a][3]};
    }
  }
  __syncthreads();

  f32x4 acc[MT][NPW];
  // (3) y = u Pi^T, bucketise; index bit planes; centroid values as bf16 terms for the next contraction
  // (FX: the matrix registers stay free after this contraction; the fp6 digits of Pi^T take their place until
  // the centroid contraction is done, then S is requested and has the residual pass to arrive)
  contract<D, NA1, !FX, ML>(terms, ly.Pi_split, mse_only ? ly.Pi_split : ly.PiT_split, wave, lane, mr, acc);
  i32x8 fa[FX ? NPW : 1][FX ? FXT : 1];
  if constexpr (FX) {
#pragma unroll
    for (int c = 0; c < NPW; ++c)
#pragma unroll
      for (int t = 0; t < FXT; ++t) {
        const uint32_t* p6 = ly.PiT_fp6 + ((size_t)((wave * NPW + c) * FXT + t) * 64 + lane) * 6;
        fa[c][t] = i32x8{(int)p6[0], (int)p6[1], (int)p6[2], (int)p6[3], (int)p6[4], (int)p6[5], 0, 0};
      }
  }
  __syncthreads();                                              // every wavefront has read the unit-vector terms
  if constexpr (FX) {
    // The index bit planes straight from the comparisons (no index is formed): with the count of thresholds
    // below y as the index (searchsorted; a NaN counts all), the low bit is the parity of the comparisons and,
    // for two bits, the high bit the comparison with the middle threshold.  The comparison results are lane
    // masks, so the parity costs scalar instructions only.
    uint32_t bitc[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) bitc[h][i] = 1u << (16 * h + 4 * kb + i);
    const float t0 = sthr[0], t1 = mb == 2 ? sthr[1] : 0.0f, t2 = mb == 2 ? sthr[2] : 0.0f;
#pragma unroll
    for (int m = 0; m < ML; ++m) {
      const int t = 16 * m + n;
#pragma unroll
      for (int wl = 0; wl < NPW / 2; ++wl) {
        uint32_t hi = 0, lo = 0;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float y = acc[m][2 * wl + h][i];
            const bool c0 = !(y <= t0);
            if (mb == 2) {
              const bool c1 = !(y <= t1), c2 = !(y <= t2);
              hi |= c1 ? bitc[h][i] : 0u;
              lo |= (c0 != c1) != c2 ? bitc[h][i] : 0u;
            } else {
              hi |= c0 ? bitc[h][i] : 0u;
            }
          }
        hi = or_over_kb(hi);
        if (mb == 2) lo = or_over_kb(lo);
        if (kb == 0) {
          spl[(0 * TT + t) * W + (wave * NPW) / 2 + wl] = hi;
          if (mb == 2) spl[(1 * TT + t) * W + (wave * NPW) / 2 + wl] = lo;
        }
      }
      if constexpr (std::is_same<Sink, KeyFlatSink>::value) {
#pragma unroll
        for (int c = 0; c < NPW; ++c) {
          const int col0 = 16 * (wave * NPW + c) + 4 * kb;
          if (sink.y_dbg && svalid[t]) *(f32x4*)(sink.y_dbg + (tile0 * TILE + t) * D + col0) = acc[m][c];
        }
      }
    }
  } else {
    uint32_t idx[MT][NPW][4];
#pragma unroll
    for (int m = 0; m < ML; ++m)
#pragma unroll
      for (int c = 0; c < NPW; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) idx[m][c][i] = 0;
    for (int k = 0; k < n_thr; ++k) {                           // searchsorted: count thresholds below y (NaN counts all)
      const float th = sthr[k];
#pragma unroll
      for (int m = 0; m < ML; ++m)
#pragma unroll
        for (int c = 0; c < NPW; ++c)
#pragma unroll
          for (int i = 0; i < 4; ++i) idx[m][c][i] += !(acc[m][c][i] <= th);
    }
#pragma unroll
    for (int m = 0; m < ML; ++m) {
      const int t = 16 * m + n;
      for (int p = 0; p < mb; ++p) {
        const int sh = mb - 1 - p;
#pragma unroll
        for (int wl = 0; wl < NPW / 2; ++wl) {
          uint32_t v = 0;
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) v |= ((idx[m][2 * wl + h][i] >> sh) & 1u) << (16 * h + 4 * kb + i);
          v = or_over_kb(v);
          if (kb == 0) spl[(p * TT + t) * W + (wave * NPW) / 2 + wl] = v;
        }
      }
#pragma unroll
      for (int c = 0; c < NPW; ++c) {
        const int col0 = 16 * (wave * NPW + c) + 4 * kb;
        if constexpr (!FX) {
          u32x2 e[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) e[i] = slut[idx[m][c][i]];
          // term 0: low halves of .x, term 1: high halves of .x, term 2: low halves of .y
          const u32x2 t0{(e[0].x & 0xffffu) | (e[1].x << 16), (e[2].x & 0xffffu) | (e[3].x << 16)};
          const u32x2 t1{(e[0].x >> 16) | (e[1].x & 0xffff0000u), (e[2].x >> 16) | (e[3].x & 0xffff0000u)};
          const u32x2 t2{e[0].y | (e[1].y << 16), e[2].y | (e[3].y << 16)};
          *(u32x2*)(terms + ((size_t)0 * TT + t) * RS + col0) = t0;
          *(u32x2*)(terms + ((size_t)1 * TT + t) * RS + col0) = t1;
          *(u32x2*)(terms + ((size_t)2 * TT + t) * RS + col0) = t2;
        }
        if constexpr (std::is_same<Sink, KeyFlatSink>::value) {
          if (sink.y_dbg && svalid[t]) *(f32x4*)(sink.y_dbg + (tile0 * TILE + t) * D + col0) = acc[m][c];
        }
      }
    }
  }
  __syncthreads();
  if (mse_only) stg.issue(x);
  if (!mse_only) {
    // (4) x_hat = (c Pi) * norm ; r = x - x_hat ; ||r||^2 partial sums ; r as bf16 terms (quantizer.py:241-245)
    if constexpr (FX) {
      // lane (n, kb) feeds plane word kb of vector 16 m + n: coordinate c of the word sits at contraction
      // index 32 kb + 8 (c % 4) + c / 4 with the fp4 value 0.5, 1, 2, 0.5 (the matrix digits carry the inverse)
      // (the first plane's sum starts from the constant term: no separate initialisation of the accumulators)
      auto plane = [&](int p, f32x4 (&part)[MT][NPW]) {
        u32x4 b[MT];
#pragma unroll
        for (int m = 0; m < ML; ++m) {
          const uint32_t w = spl[(p * TT + 16 * m + n) * W + kb];
          b[m] = u32x4{w & 0x11111111u, w & 0x22222222u, w & 0x44444444u, (w >> 3) & 0x11111111u};
#pragma unroll
          for (int c = 0; c < NPW; ++c) part[m][c] = f32x4{0, 0, 0, 0};
        }
        // digit by digit over all tiles: consecutive MFMAs go to different accumulators
#pragma unroll
        for (int m = 0; m < ML; ++m)
#pragma unroll
          for (int c = 0; c < NPW; ++c) part[m][c] = mfma_fp6_fp4<0>(fa[c][0], b[m], part[m][c], fs0[c], 127);
#pragma unroll
        for (int m = 0; m < ML; ++m)
#pragma unroll
          for (int c = 0; c < NPW; ++c) part[m][c] = mfma_fp6_fp4<1>(fa[c][1], b[m], part[m][c], fs0[c], 127);
#pragma unroll
        for (int m = 0; m < ML; ++m)
#pragma unroll
          for (int c = 0; c < NPW; ++c) part[m][c] = mfma_fp6_fp4<2>(fa[c][2], b[m], part[m][c], fs0[c], 127);
#pragma unroll
        for (int m = 0; m < ML; ++m)
#pragma unroll
          for (int c = 0; c < NPW; ++c) part[m][c] = mfma_fp6_fp4<3>(fa[c][3], b[m], part[m][c], fs0[c], 127);
#pragma unroll
        for (int m = 0; m < ML; ++m)
#pragma unroll
          for (int c = 0; c < NPW; ++c) part[m][c] = mfma_fp6_fp4<0>(fa[c][4], b[m], part[m][c], fs1[c], 127);
      };
      {
        f32x4 part[MT][NPW];
        plane(0, part);
#pragma unroll
        for (int m = 0; m < ML; ++m)
#pragma unroll
          for (int c = 0; c < NPW; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[m][c][i] = fmaf(fk[0], part[m][c][i], fconst[c][i]);
        if (mb == 2) {
          plane(1, part);
#pragma unroll
          for (int m = 0; m < ML; ++m)
#pragma unroll
            for (int c = 0; c < NPW; ++c)
#pragma unroll
              for (int i = 0; i < 4; ++i) acc[m][c][i] = fmaf(fk[1], part[m][c][i], acc[m][c][i]);
        }
      }
      prefetch_matrix<D>(ly.S_split, wave, lane, mr);
    } else {
      contract<D, 3, true, ML>(terms, ly.PiT_split, ly.S_split, wave, lane, mr, acc);
      __syncthreads();                                          // every wavefront has read the centroid terms
    }
#pragma unroll
    for (int m = 0; m < ML; ++m) {
      const int t = 16 * m + n;
      const float nrm = snorm[t];
      float rs = 0.0f;
#pragma unroll
      for (int c = 0; c < NPW; ++c) {
        const int col0 = 16 * (wave * NPW + c) + 4 * kb;
        float r[4], xv[4];
        load_run<DT, 4>(sx + t * XRS + col0, xv);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float xh = acc[m][c][i] * nrm;
          r[i] = xv[i] - xh;
          rs += r[i] * r[i];
        }
        uint32_t lo[3], hi[3];
        split3_pk(r[0], r[1], lo);
        split3_pk(r[2], r[3], hi);
#pragma unroll
        for (int a = 0; a < 3; ++a) *(u32x2*)(terms + ((size_t)a * TT + t) * RS + col0) = u32x2{lo[a], hi[a]};
      }
      rs = sum_over_kb(rs);
      if (kb == 0) spart[wave * TT + t] = rs;
    }
    __syncthreads();
    stg.issue(x);                                               // the input tile is free: fetch the next group
    if (tid < TT) {
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < KQ_WAVES; ++w) v += spart[w * TT + tid];
      srn[tid] = sqrtf(v);
    }
    // (5) p = r S^T ; sign bits (quantizer.py:248-249)
    contract<D, 3, true, ML>(terms, ly.S_split, ly.Pi_split, wave, lane, mr, acc);    // Pi again for the next group
#pragma unroll
    for (int m = 0; m < ML; ++m) {
      const int t = 16 * m + n;
#pragma unroll
      for (int wl = 0; wl < NPW / 2; ++wl) {
        uint32_t v = 0;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) v |= (uint32_t)(acc[m][2 * wl + h][i] > 0.0f) << (16 * h + 4 * kb + i);
        v = or_over_kb(v);
        if (kb == 0) spl[(mb * TT + t) * W + (wave * NPW) / 2 + wl] = v;
      }
      if constexpr (std::is_same<Sink, KeyFlatSink>::value) {
        if (sink.p_dbg && svalid[t]) {
#pragma unroll
          for (int c = 0; c < NPW; ++c)
            *(f32x4*)(sink.p_dbg + (tile0 * TILE + t) * D + 16 * (wave * NPW + c) + 4 * kb) = acc[m][c];
        }
      }
    }
  }
  __syncthreads();
  // (6) write
  if constexpr (std::is_same<Sink, KeyFlatSink>::value) {
    // flat format of the reference (quantizer.py:38-69): indices packed eff_bits apiece, signs 8 per byte
    // A thread builds one dword of a row: n = 32 / eff codes, code s at bit eff * s, plane 0 the top bit of a
    // code.  The n bits a plane contributes are spread to a stride of eff bits with shift-and-mask steps.
    const int eff = eff_bits(mb), n_per = 32 / eff, row_dw = idx_row_bytes(D, mb) >> 2;
    for (int o = tid; o < TT * row_dw; o += KQ_THREADS) {
      const int t = o / row_dw, k = o - t * row_dw;
      if (!svalid[t]) continue;
      const int c0 = k * n_per;                                  // first coordinate of this dword
      uint32_t dw = 0;
      for (int p = 0; p < mb; ++p) {
        uint32_t x = spl[(p * TT + t) * W + (c0 >> 5)] >> (c0 & 31);
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
        }                                                         // eff == 1: the plane word is the dword
        dw |= x << (mb - 1 - p);
      }
      ((uint32_t*)sink.idx)[(tile0 * TILE + t) * row_dw + k] = dw;
    }
    if (!mse_only) {
      for (int o = tid; o < TT * W; o += KQ_THREADS) {
        const int t = o / W, w = o - t * W;
        if (svalid[t]) ((uint32_t*)sink.sign)[(tile0 * TILE + t) * W + w] = spl[(mb * TT + t) * W + w];
      }
    }
    if (tid < TT && svalid[tid]) {
      const int64_t v = tile0 * TILE + tid;
      E::store(sink.norm, v, snorm[tid]);
      if (!mse_only) sink.rnorm[v] = srn[tid];
    }
  } else {
    // pages: a wavefront writes the bit-plane words of one tile, so the page lookup is uniform;
    // lanes run over (word, token) in page order (lane-major: [w & 3][token][w >> 2][plane])
    const tq_page_layout& L = sink.L;
    constexpr int NSUB = KQ_WAVES / ML > 0 ? KQ_WAVES / ML : 1;   // wavefronts that share a tile
    const int planes = mb + 1;
    for (int m = wave % ML; m < ML; m += KQ_WAVES) {
      const int64_t tile = tile0 + m;
      if (tile >= n_tiles) break;
      // a tile none of whose slots exists may lie beyond the block table: do not look it up
      // (and a page outside the table or the pool is not written)
      if (__builtin_amdgcn_ballot_w64(lane < TILE && svalid[16 * m + lane]) == 0 || wpage < 0) continue;
      uint8_t* pg = sink.pool + (wpage * src.H + wr_h) * (int64_t)L.page_bytes;
      for (int p = wave / ML; p < planes; p += NSUB) {
#pragma unroll
        for (int e = lane; e < W * TILE; e += 64) {
          const int jh = e % (W / 4), nn = (e / (W / 4)) % TILE, jl = e / (W / 4) / TILE;
          const int w = jh * 4 + jl;
          if (svalid[16 * m + nn])
            *(uint32_t*)(pg + key_word_off(L, p, w, nn)) = (p == mb && mse_only) ? 0u : spl[(p * TT + 16 * m + nn) * W + w];
        }
      }
      if (wave / ML == 0 && lane < TILE && svalid[16 * m + lane]) {
        float* meta = (float*)(pg + L.off_meta);
        meta[2 * lane] = snorm[16 * m + lane];
        meta[2 * lane + 1] = mse_only ? 0.0f : srn[16 * m + lane];
      }
    }
  }
  __syncthreads();                                              // the next group overwrites what the writers read
  }
}


__host__ static bool aligned_for_chunks(const void* x, int dtype, const FlatSource& s) {
  const int64_t ch = 16 / elem_bytes(dtype);
  return (uintptr_t)x % 16 == 0 && s.row_stride % ch == 0;
}
__host__ static bool aligned_for_chunks(const void* x, int dtype, const PagedSource& s) {
  const int64_t ch = 16 / elem_bytes(dtype);
  return (uintptr_t)x % 16 == 0 && s.stride_b % ch == 0 && s.stride_t % ch == 0 && s.stride_h % ch == 0 &&
         s.stride_blk % ch == 0;
}
__host__ static bool sink_ok(const KeyFlatSink& s, int mse_only) {
  return (uintptr_t)s.y_dbg % 16 == 0 && (uintptr_t)s.p_dbg % 16 == 0 && (uintptr_t)s.idx % 4 == 0 &&
         (mse_only || (uintptr_t)s.sign % 4 == 0);
}
__host__ static bool sink_ok(const KeyPagedSink& s, int) { return s.L.key_lane_major != 0; }

template <int DT, int D, bool MSE_ONLY, bool FX, class Source, class Sink, int ML = KeyGeom<D>::MT>
static int launch_dt_d(const void* x, const Source& src, const tq_layer& ly, const Sink& sink, int64_t tiles,
                       hipStream_t st) {
  using Gm = KeyGeom<D>;
  using Sm = KeySmem<DT, D>;
  // Few tiles, written to pages (the page write of a decode step: a token per sequence): a workgroup per tile, which
  // then computes that tile only, while they all fit the card at once
  if constexpr (ML == Gm::MT && std::is_same<Sink, KeyPagedSink>::value && !MSE_ONLY) {
    const int opt = opt_append_small.load(std::memory_order_relaxed);
    if (opt != 0 && tiles <= (opt < 0 ? 2 * (int64_t)device_compute_units() : (int64_t)opt))
      return launch_dt_d<DT, D, MSE_ONLY, FX, Source, Sink, 1>(x, src, ly, sink, tiles, st);
  }
  auto kern = key_mfma_kernel<DT, D, MSE_ONLY, FX, Source, Sink, ML>;
  static std::atomic<uint64_t> configured{0};           // per instantiation, one bit per device; the attribute is sticky
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return TQ_EINVAL;
  if (dev >= 64 || !(configured.load() >> dev & 1)) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)Sm::bytes);
    if (e != hipSuccess) return (int)e;
    if (dev < 64) configured.fetch_or(1ull << dev);
  }
  // persistent workgroups: as many as stay resident (LDS allows 160 KB / bytes per compute unit)
  static std::atomic<int> n_cu[64];                       // per device
  int cus = dev < 64 ? n_cu[dev].load(std::memory_order_relaxed) : 0;
  if (cus <= 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    if (dev < 64) n_cu[dev].store(cus, std::memory_order_relaxed);
  }
  const int per_cu = (int)(160 * 1024 / Sm::bytes) > 2 ? 2 : (int)(160 * 1024 / Sm::bytes);
  const int64_t groups = (tiles + ML - 1) / ML;
  const int64_t resident = (int64_t)cus * (per_cu > 0 ? per_cu : 1);
  const unsigned grid = (unsigned)(groups < resident ? groups : resident);
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;
  if (std::is_same<Sink, KeyPagedSink>::value && take_time_hook(1, ev_start, ev_stop)) {
    hipExtLaunchKernelGGL(kern, dim3(grid), dim3(KQ_THREADS), Sm::bytes, st, ev_start, ev_stop, 0, x, src, ly, sink, tiles);
  } else {
    kern<<<dim3(grid), dim3(KQ_THREADS), Sm::bytes, st>>>(x, src, ly, sink, tiles);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TQ_OK : (int)e;
}

// TQ_EUNSUPPORTED when there is no matrix-core kernel for this call (head_dim other than
// 128 / 256, no split matrices, or operands not aligned for 16-byte loads): the caller
// falls back to the vector-ALU kernel.
template <class Source, class Sink>
int launch_key_mfma(const void* x, int dtype, const Source& src, const tq_layer& ly, const Sink& sink, int mse_only,
                    int64_t tiles, hipStream_t st) {
  if (!ly.Pi_split || !ly.PiT_split || (!mse_only && !ly.S_split)) return TQ_EUNSUPPORTED;
  if (ly.mse_bits < 1 || ly.mse_bits > 4) return TQ_EUNSUPPORTED;
  if (!aligned_for_chunks(x, dtype, src) || !sink_ok(sink, mse_only)) return TQ_EUNSUPPORTED;
  constexpr bool paged = std::is_same<Sink, KeyPagedSink>::value;     // pages always hold the full code
  if (paged && mse_only) return TQ_EUNSUPPORTED;
  // head_dim 128 with the fp6 digits of Pi^T and a codebook whose Walsh expansion has single-bit terms only:
  // the centroid contraction on the block-scaled MFMA
  bool fx = ly.d == 128 && !mse_only && ly.PiT_fp6 && ly.PiT_fp6_scale && ly.Pi_colsum && ly.mse_bits <= 2 &&
            opt_fp6_centroids.load() != 0;
  for (int t = 0; t < ly.n_terms; ++t) fx = fx && __builtin_popcount((unsigned)ly.term_mask[t]) == 1;
#define TQ_KQ(DT_, D_)                                                                                     \
  if (dtype == DT_ && ly.d == D_) {                                                                        \
    if constexpr (!paged)                                                                                  \
      if (mse_only) return launch_dt_d<DT_, D_, true, false, Source, Sink>(x, src, ly, sink, tiles, st);   \
    if constexpr (D_ == 128)                                                                               \
      if (fx) return launch_dt_d<DT_, D_, false, true, Source, Sink>(x, src, ly, sink, tiles, st);         \
    return launch_dt_d<DT_, D_, false, false, Source, Sink>(x, src, ly, sink, tiles, st);                  \
  }
  TQ_KQ(TQ_BF16, 128) TQ_KQ(TQ_BF16, 256) TQ_KQ(TQ_F16, 128) TQ_KQ(TQ_F16, 256) TQ_KQ(TQ_F32, 128) TQ_KQ(TQ_F32, 256)
#undef TQ_KQ
  return TQ_EUNSUPPORTED;
}

// ------------------------------------------------------------------------------------
// De-quantiser on the matrix cores: x_hat = (c[idx] Pi) * norm + (sigma S) * (qjl_scale * rnorm)
// (quantizer.py:151-165, 259-272) with the machinery of the quantiser.  The centroid values of a
// group of TT vectors go to LDS as three bf16 terms (exact), the signs as one (+-1 is a bf16 number),
// the matrices are the split Pi^T and S^T (a row of the operand = an output coordinate), and the
// products are exact with fp32 accumulation, so the result has the accuracy of an fp32 product sum.
// ------------------------------------------------------------------------------------
template <int D>
struct DeqSmem {
  using G = KeyGeom<D>;
  static constexpr size_t off_terms = 0;                                        // [3][TT][RS] centroid terms
  static constexpr size_t off_sign = 3 * (size_t)G::TT * G::RS * 2;             // [TT][RS] +-1
  static constexpr size_t off_small = off_sign + (size_t)G::TT * G::RS * 2;     // snorm[TT] srn[TT] slut[16]
  static constexpr size_t bytes = off_small + (size_t)G::TT * 8 + 16 * 8;
};

template <int D, bool QJL>
__global__ void __launch_bounds__(KQ_THREADS, 2)
dequant_mfma_kernel(const uint8_t* __restrict__ idx, const uint8_t* __restrict__ signs, const void* __restrict__ norms,
                    int norm_dtype, const float* __restrict__ rnorms, int64_t n_vec, tq_layer ly,
                    float* __restrict__ out) {
  using Gm = KeyGeom<D>;
  using Sm = DeqSmem<D>;
  constexpr int TT = Gm::TT, MT = Gm::MT, NPW = Gm::NPW, RS = Gm::RS, TPR = Gm::TPR, SEG = Gm::SEG;
  static_assert(SEG == 32, "a thread fills 32 coordinates: one word of sign bits");
  const int tid0 = threadIdx.x, wave0 = __builtin_amdgcn_readfirstlane(tid0 >> 6);
  const int mb = ly.mse_bits, eff = eff_bits(mb), row = idx_row_bytes(D, mb);
  const int64_t n_groups = (n_vec + TT - 1) / TT;
  MatRegs<D> mr;
  prefetch_matrix<D>(ly.PiT_split, wave0, tid0 & 63, mr);

  extern __shared__ __align__(16) unsigned char smem[];
  uint16_t* terms = (uint16_t*)(smem + Sm::off_terms);
  uint16_t* sgn = (uint16_t*)(smem + Sm::off_sign);
  float* snorm = (float*)(smem + Sm::off_small);
  float* srn = snorm + TT;
  u32x2* slut = (u32x2*)(srn + TT);                             // bf16 terms of a centroid: {t0 | t1 << 16, t2}
  if (tid0 < (1 << mb)) {
    uint32_t t[3];
    split3_pk(ly.centroids[tid0], 0.0f, t);
    slut[tid0] = u32x2{(t[0] & 0xffffu) | (t[1] << 16), t[2] & 0xffffu};
  }
  // a thread holds the packed codes of its 32 coordinates of the NEXT group: eff index words, one sign word
  const int t = tid0 / TPR, seg = tid0 % TPR;
  uint32_t iw[4] = {0, 0, 0, 0}, sw = 0;
  float nv = 0.0f, rv = 0.0f;
  auto fetch = [&](int64_t g) {
    const int64_t v = g * TT + t;
    const int64_t vv = v < n_vec ? v : 0;                       // vectors that do not exist read the first one
    const uint32_t* ip = (const uint32_t*)(idx + vv * row) + seg * eff;
    iw[0] = ip[0];
    if (eff >= 2) iw[1] = ip[1];
    if (eff == 4) { iw[2] = ip[2]; iw[3] = ip[3]; }
    if (QJL) sw = ((const uint32_t*)(signs + vv * (D / 8)))[seg];
    if (seg == 0) {
      nv = load_as_f32(norms, vv, norm_dtype);
      if (QJL) rv = rnorms[vv];
    }
  };
  if ((int64_t)blockIdx.x < n_groups) fetch(blockIdx.x);
  __syncthreads();

  for (int64_t g = blockIdx.x; g < n_groups; g += gridDim.x) {
    int tid = tid0, wave = wave0;
    asm volatile("" : "+v"(tid), "+s"(wave));
    const int lane = tid & 63, n = lane & 15, kb = lane >> 4;
    // (1) codes -> centroid terms and +-1 in LDS
    auto fill = [&](auto eff_c) {
      constexpr int EFF = decltype(eff_c)::value;
      constexpr uint32_t mask = (1u << EFF) - 1u;
#pragma unroll
      for (int c8 = 0; c8 < SEG; c8 += 8) {
        u32x2 e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int bit = (c8 + i) * EFF;
          e[i] = slut[(iw[bit >> 5] >> (bit & 31)) & mask];
        }
        uint32_t pk[3][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const u32x2 a = e[2 * i], b = e[2 * i + 1];
          pk[0][i] = (a.x & 0xffffu) | (b.x << 16);
          pk[1][i] = (a.x >> 16) | (b.x & 0xffff0000u);
          pk[2][i] = a.y | (b.y << 16);
        }
#pragma unroll
        for (int a = 0; a < 3; ++a)
          *(u32x4*)(terms + ((size_t)a * TT + t) * RS + seg * SEG + c8) = u32x4{pk[a][0], pk[a][1], pk[a][2], pk[a][3]};
      }
    };
    if (eff == 4) fill(std::integral_constant<int, 4>{});
    else if (eff == 2) fill(std::integral_constant<int, 2>{});
    else fill(std::integral_constant<int, 1>{});
    if (QJL) {
#pragma unroll
      for (int c8 = 0; c8 < SEG; c8 += 8) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t b2 = sw >> (c8 + 2 * i);               // bit set = +1 (0x3f80), clear = -1 (0xbf80)
          w[i] = 0xbf80bf80u ^ ((b2 & 1u) << 15) ^ ((b2 & 2u) << 30);
        }
        *(u32x4*)(sgn + (size_t)t * RS + seg * SEG + c8) = u32x4{w[0], w[1], w[2], w[3]};
      }
    }
    if (seg == 0) {
      snorm[t] = nv;
      if (QJL) srn[t] = __fmul_rn(ly.qjl_scale, rv);
    }
    __syncthreads();
    if (g + gridDim.x < n_groups) fetch(g + gridDim.x);         // lands while this group is contracted
    // (2) contractions
    f32x4 acc[MT][NPW], acq[QJL ? MT : 1][QJL ? NPW : 1];
    contract<D, 3>(terms, ly.PiT_split, QJL ? ly.ST_split : ly.PiT_split, wave, lane, mr, acc);
    if constexpr (QJL) contract<D, 1>(sgn, ly.ST_split, ly.PiT_split, wave, lane, mr, acq);
    // (3) scale and store: a lane holds four consecutive coordinates of a vector
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const int tt = 16 * m + n;
      const int64_t v = g * TT + tt;
      if (v < n_vec) {
        const float nrm = snorm[tt];
        const float rn = QJL ? srn[tt] : 0.0f;
#pragma unroll
        for (int c = 0; c < NPW; ++c) {
          f32x4 r;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            r[i] = __fmul_rn(acc[m][c][i], nrm);
            if constexpr (QJL) r[i] = __fadd_rn(r[i], __fmul_rn(acq[m][c][i], rn));
          }
          *(f32x4*)(out + v * D + 16 * (wave * NPW + c) + 4 * kb) = r;
        }
      }
    }
    __syncthreads();                                            // the next group overwrites the tiles
  }
}

template <int D, bool QJL>
static int launch_deq_d(const uint8_t* idx, const uint8_t* signs, const void* norms, int norm_dtype, const float* rnorms,
                        int64_t n_vec, const tq_layer& ly, float* out, hipStream_t st) {
  using Sm = DeqSmem<D>;
  auto kern = dequant_mfma_kernel<D, QJL>;
  static std::atomic<unsigned long long> configured{0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return TQ_EINVAL;
  if (dev >= 64 || !(configured.load() >> dev & 1)) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)Sm::bytes);
    if (e != hipSuccess) return (int)e;
    if (dev < 64) configured.fetch_or(1ull << dev);
  }
  int n_cu = 0;
  if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0) n_cu = 256;
  const int64_t groups = (n_vec + KeyGeom<D>::TT - 1) / KeyGeom<D>::TT;
  const int64_t resident = (int64_t)n_cu * 2;
  const unsigned grid = (unsigned)(groups < resident ? groups : resident);
  kern<<<dim3(grid), dim3(KQ_THREADS), Sm::bytes, st>>>(idx, signs, norms, norm_dtype, rnorms, n_vec, ly, out);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TQ_OK : (int)e;
}

// TQ_EUNSUPPORTED when there is no matrix-core kernel for this call (head_dim other than 128 / 256,
// no split matrices, or operands not aligned for word / 16-byte accesses).
int launch_dequant_mfma(const uint8_t* idx, const uint8_t* signs, const void* norms, int norm_dtype, const float* rnorms,
                        int64_t n_vec, const tq_layer& ly, float* out, hipStream_t st) {
  if (!ly.PiT_split || (signs && !ly.ST_split)) return TQ_EUNSUPPORTED;
  if (ly.mse_bits < 1 || ly.mse_bits > 4 || (ly.d != 128 && ly.d != 256)) return TQ_EUNSUPPORTED;
  if ((uintptr_t)idx % 4 || (uintptr_t)signs % 4 || (uintptr_t)out % 16) return TQ_EUNSUPPORTED;
  if (ly.d == 128)
    return signs ? launch_deq_d<128, true>(idx, signs, norms, norm_dtype, rnorms, n_vec, ly, out, st)
                 : launch_deq_d<128, false>(idx, signs, norms, norm_dtype, rnorms, n_vec, ly, out, st);
  return signs ? launch_deq_d<256, true>(idx, signs, norms, norm_dtype, rnorms, n_vec, ly, out, st)
               : launch_deq_d<256, false>(idx, signs, norms, norm_dtype, rnorms, n_vec, ly, out, st);
}

template int launch_key_mfma<FlatSource, KeyFlatSink>(const void*, int, const FlatSource&, const tq_layer&,
                                                      const KeyFlatSink&, int, int64_t, hipStream_t);
template int launch_key_mfma<PagedSource, KeyPagedSink>(const void*, int, const PagedSource&, const tq_layer&,
                                                        const KeyPagedSink&, int, int64_t, hipStream_t);

}  // namespace tq
