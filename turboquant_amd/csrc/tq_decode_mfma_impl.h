#pragma once
// Page-streaming decode kernel on the matrix cores (gfx950): the kernel template and its launcher, included by
// one translation unit per head size (tq_decode_mfma_d64 / _d128 / _d256.hip), which instantiate it.
//
// The packed bits feed the matrix cores almost directly:
//
//  * keys.  A Lloyd-Max centroid is an affine function of the parities of subsets
//    of its index bits (Walsh expansion; for the symmetric codebooks simply of
//    the individual index bits), so  sum_j q_rot[j] c[idx_j]  is a sum of
//    "query . bit-plane" contractions, exactly like the QJL term
//    sum_j q_sk[j] (2 bit_j - 1).  The contraction runs on
//    v_mfma_scale_f32_16x16x128_f8f6f4 with the bits as the fp4 operand: the nibbles
//    0001, 0010, 0100 are the fp4 numbers 0.5, 1, 2, so  x & 0x11111111,
//    x & 0x22222222, x & 0x44444444 and (x >> 3) & 0x11111111 turn a 32-bit plane
//    word into the four operand dwords (5 vector-ALU instructions for 32
//    coordinates); the query operand carries the inverse factors.  The query is
//    the fp6 (e2m3) operand - the MFMA runs at twice the fp8 rate with it -, split
//    into four fp6 terms with per-row power-of-two scales (good to 2^-20 of the
//    row bound), prepared once per step; every factor and constant of the score
//    that belongs to a query head is folded into those operands, their block
//    scales and the initial accumulator.
//  * softmax.  Weights are exp2(score - reference); the reference of a row only
//    moves when a score exceeds it by more than a small slack, so the usual block
//    needs no row reduction and no rescaling.
//  * values.  A code masked out of its packed word IS a bf16 denormal (exponent
//    field zero, the code in the low mantissa bits): B = code * 2^(s-133) exactly,
//    s being the bit position the code has in its 16-bit half, and the bf16 MFMA
//    (v_mfma_f32_16x16x32_bf16) keeps denormal inputs.  The softmax weight times the
//    group scale times 2^(80-s) is the A operand; the accumulators carry 2^-53
//    until the epilogue.  At most 8 query heads share a KV head, so operand rows
//    0..7 carry the heads weighted with the scales of an even group and rows 8..15
//    the same heads with the scales of the next group: one set of weight products
//    serves the channel tiles of two groups.  The zero points go through one more
//    MFMA (weights x zeros).
//
// head_dim 256 is split over a pair of wavefronts (DS = 2): each scores half of the
// coordinates, the halves of the scores meet in LDS once per block, both wavefronts
// then compute the same softmax and each accumulates half of the channels.  That keeps
// the per-wavefront register footprint of head_dim 128, so two wavefronts fit per SIMD.
//
// One wavefront (pair) owns 64 tokens (4 pages) per iteration: lane (n, kb) = lane%16,
// lane/16 is token n and coordinate quarter kb in the score stage, and (row,
// page kb) in the value stage.  The key words of the next 64 tokens are
// requested right after the current score stage, the value words right after the
// current value stage, so each load has a whole stage to arrive.  Workgroups have 4
// wavefronts; WPS of them share a SIMD so that one wavefront's dependency stalls
// are filled by another.

#include <type_traits>

#include <hip/hip_ext.h>

#include "tq_common.h"
#include "tq_prep.h"
#include "tq_decode_mfma.h"
#include "tq_options.h"

namespace tq {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

// -DTQ_STAMPS (a profiling build, never the shipped one): lane 0 of every wavefront of the first 1024 workgroups
// records the 100 MHz real-time counter at the kernel's phase boundaries - 0 start, 1 operands loaded, 2 first block
// requested and table scanned, 3 loop done, 6 / 7 inside the epilogue, 4 partial stores issued, 5 stores acknowledged;
// tq_debug_stamps copies them out.  The per-phase times quoted for the page kernels come from such a build.
#ifdef TQ_STAMPS
__device__ unsigned long long tq_stamps[4096 * 8];
#define TQ_STAMP(k) do { if (lane == 0) tq_stamps[(((blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * 8 + wave) * 8 + (k)) & 32767] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define TQ_STAMP(k)
#endif
constexpr int MF_WAVES = 4;
constexpr int BLK_TOK = 64;              // tokens per wavefront iteration
constexpr float MF_NEG = -1.0e30f;
constexpr int P_STRIDE = 20;             // floats per row of the LDS softmax-weight tile (16 + skew)
constexpr int X_FLOATS = 2 * 8 * 64;     // score-half exchange slot of a wavefront: [parity][8 values][64 lanes]
__host__ __device__ constexpr int wave_lds_floats(int ng, int ds) {
  return 4 * 8 * P_STRIDE + 16 + 4 * ng * 16 + (ds > 1 ? X_FLOATS : 0);
}
// Staging area of a wavefront for page data that travels HBM -> LDS without passing through registers
// (SG kernels): every piece is what one LDS-direct load instruction writes, 16 bytes per lane:
// [4 pages] key words, [32 lanes] norms, [VW / 4] value words, [2] zero points, [1] scales.
__host__ __device__ constexpr int stage_bytes(int vw) { return 4 * 1024 + 512 + (vw / 4) * 1024 + 2 * 1024 + 1024; }

// LDS-direct loads (gfx950: 12 and 16 bytes per lane): lane l's bytes land at m0 + OFF + 16 l, read from
// its address + OFF.  The compiler does not see these instructions: it neither counts them in vmcnt nor
// orders LDS accesses against them; the kernel waits for them itself (stage_wait) before it reads the area.
template <int OFF>
__device__ __forceinline__ void dma16(const void* vaddr, uint32_t m0) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:%2"
               :: "v"(vaddr), "s"(m0), "n"(OFF) : "memory", "m0");
}
template <int BYTES>
__device__ __forceinline__ void dma_so(uint32_t voff, const void* sbase, uint32_t m0) {
  // (12 bytes: three dwords per lane; anything else is taken as four)
  if (BYTES == 12)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx3 %0, %1" :: "v"(voff), "s"(sbase), "s"(m0) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(voff), "s"(sbase), "s"(m0) : "memory", "m0");
}
// wait until at most N vector-memory instructions of this wavefront are outstanding (they complete in order)
template <int N>
__device__ __forceinline__ void stage_wait() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }
// the LDS reads issued so far have returned: their area may be overwritten
__device__ __forceinline__ void stage_release() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  f32x2 f = {lo, hi};
  bf16x2 r = __builtin_convertvector(f, bf16x2);   // v_cvt_pk_bf16_f32, round to nearest even
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}
__device__ __forceinline__ float bf16_round(float v) { return __uint_as_float(pack_bf16(v, 0.0f) << 16); }
__device__ __forceinline__ f32x4 mfma(const u32x4& a, const u32x4& b, f32x4 c) {
  bf16x8 av, bv;
  __builtin_memcpy(&av, &a, 16);
  __builtin_memcpy(&bv, &b, 16);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, c, 0, 0, 0);
}
// fp16 pages: the zero points are fp16 numbers, so their product with the softmax weights runs on the
// fp16 MFMA with the weights packed as fp16 (they are at most 2^REF_SLACK; weights below the fp16
// denormal range belong to tokens whose share of the sum is below 2^-24)
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  f32x2 f = {lo, hi};
  f16x2 r = __builtin_convertvector(f, f16x2);     // round to nearest even
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}
__device__ __forceinline__ f32x4 mfma_f16(const u32x4& a, const u32x4& b, f32x4 c) {
  f16x8 av, bv;
  __builtin_memcpy(&av, &a, 16);
  __builtin_memcpy(&bv, &b, 16);
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, c, 0, 0, 0);
}
__device__ __forceinline__ float f16_lo(uint32_t w) {
  const f16x2 h = __builtin_bit_cast(f16x2, w);
  return (float)h[0];
}
__device__ __forceinline__ float f16_hi(uint32_t w) {
  const f16x2 h = __builtin_bit_cast(f16x2, w);
  return (float)h[1];
}
// keeps a loop-invariant constant in a vector register, so that three-operand
// bit instructions do not need two scalar operands
__device__ __forceinline__ uint32_t in_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// all-reduce over the 16 lanes of a DPP row (quad swaps, half-row mirror, row mirror)
__device__ __forceinline__ float row_max16(float v) {
  v = fmaxf(v, dpp<0xB1>(v));
  v = fmaxf(v, dpp<0x4E>(v));
  v = fmaxf(v, dpp<0x141>(v));
  v = fmaxf(v, dpp<0x140>(v));
  return v;
}
// all-reduce over the two lanes 32 apart (the half-swap instruction of gfx950: no LDS round trip)
__device__ __forceinline__ float max_xor32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(fmaxf(v, __uint_as_float(r[0])), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_xor32(float v) {
  // r[0] holds the lower half's values in both halves, r[1] the upper half's
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float row_sum16(float v) {
  v += dpp<0xB1>(v);
  v += dpp<0x4E>(v);
  v += dpp<0x141>(v);
  v += dpp<0x140>(v);
  return v;
}

// fp6 (A: 16 rows x 128) x fp4 (B: 128 x 16) MFMA with per-lane power-of-two scales (E8M0 codes).
// Only the first six dwords of the fp6 operand and the first four of the fp4 operand are read.
// SEL picks the byte of scale_a that holds the code.
template <int SEL>
__device__ __forceinline__ f32x4 mfma_f8f4(const i32x8& a, uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3,
                                           f32x4 c, int scale_a, int scale_b) {
  const i32x8 bv = {(int)b0, (int)b1, (int)b2, (int)b3, 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, bv, c, 2 /*A: fp6 e2m3*/, 4 /*B: fp4*/, SEL, scale_a, 0, scale_b);
}

// token held by element (r, h) of MFMA half u of the value stage
template <int VB>
__device__ __forceinline__ constexpr int v_token(int u, int r, int h) {
  // (8-bit codes: dword j of a channel's field holds tokens 4j..4j+3, a byte each; its even bytes are one operand
  // dword, its odd bytes the next)
  return VB == 2 ? 4 * u + r + 8 * h : (VB == 4 ? 8 * u + r + 4 * h : 8 * u + 4 * (r >> 1) + (r & 1) + 2 * h);
}
// bit position (inside its byte) of the code of token t: the weight of the token carries 2^-pos
template <int VB>
__device__ __forceinline__ constexpr int v_bitpos(int t) {
  return VB == 2 ? 2 * (t & 3) : (VB == 4 ? 4 * (t & 1) : 0);
}

// D in {128, 256}; MB stored index bits; NX extra (multi-bit) Walsh terms; VB value bits;
// GS value group size; DS wavefronts that share one block (each takes D/DS coordinates and
// channels); WPS wavefronts per SIMD the register budget is sized for.
// PP (head_dim 64, at most 4 query heads per KV head): one score MFMA serves two pages.  The contraction is
// 128 long and a head has 64 coordinates, so the lanes of the upper two coordinate quarters hold the key
// words of a second page, and the query operand is block-diagonal: rows 0..7 (4 heads x 2 terms) carry the
// query in coordinates 0..63 and score the first page, rows 8..15 carry the same terms in coordinates
// 64..127 and score the second.  Lane (n, kb) then sees heads 2(kb%2), 2(kb%2)+1 of token n of page
// 2 * pair + kb/2; the value stage is the same as without PP.
// NR (at most 4 query heads per KV head, head_dim 128 / 256): the four fp6 terms of a head fill four rows of
// ONE operand (row 4g + t) instead of two rows in each of two, so a plane word takes one score MFMA, the
// query operands half the registers, and lane (n, kb) sees a single head (kb) of token n.
// SG: the page data of the next block goes HBM -> LDS with LDS-direct loads, requested when the current
// block's copy has been taken out of LDS, so every load has a whole trip to arrive (instead of one stage)
// and no register holds data in flight.
// NW: wavefronts per workgroup, 4 (two workgroups per compute unit) or 8 (one): with few blocks per
// wavefront the larger workgroup wins - half as many workgroups to dispatch, prologues and partials.
// IW > 0 (many short sequences, one split): a (sequence, group of heads) is walked by IW wavefronts (1 or 2) of a
// workgroup instead of all four, from the first block to the last, so a workgroup serves 4 / IW of them.  A wavefront
// then makes 4 / IW times the trips after one prologue, a launch has IW / 4 of the workgroups (256 sequences x 8 KV
// heads: one resident round instead of four), and the epilogue merges IW walkers instead of four (IW = 1: none).
// The grid is (1, ceil(items IW / 4), 1).
template <int D, int MB, int NX, int VB, int GS, int DS, int WPS, bool F16P, bool PP, bool NR, bool SG, int NW, int IW>
__global__ void __launch_bounds__(NW * 64, WPS)
decode_mfma_kernel(uint32_t* qa_pack, float* q_stat, int Hq, int Hkv, int kv_div,
                   const uint8_t* __restrict__ pool, const int32_t* __restrict__ block_table,
                   int bt_stride, const int32_t* __restrict__ seq_lens, float sm_scale, tq_layer ly, tq_page_layout L,
                   float* __restrict__ parts, int n_parts, int n_split, int len_sub, int max_pages, int num_pages,
                   int skew16, int n_seq, FusedMerge fm) {
  constexpr int DW = D / DS;                  // coordinates / channels of one wavefront
  constexpr int WPLT = (D + 127) / 128;       // plane words per lane per plane per page, all wavefronts
  constexpr int WPL = (DW + 127) / 128;       // ... of one wavefront (head_dim 64: one, with half of the lanes idle)
  constexpr int NTP = MB + NX + 1;            // term planes fed to the MFMA (stored + XOR terms + sign)
  constexpr int NKW = (MB + 1) * WPL;         // key dwords per lane per page
  constexpr int CT = DW / 16;                 // channel tiles of one wavefront
  constexpr int VW = CT * VB / 2;             // value dwords per lane per block
  constexpr int NG = DW / GS, CTG = GS / 16;  // groups of one wavefront, channel tiles per group
  constexpr int NGT = D / GS;                 // groups of the whole head
  constexpr int PIECES = 2 * NG;              // 16-byte pieces of this wavefront's scales per page
  constexpr int MF_WAVES = NW;
  constexpr int NGRP = MF_WAVES / DS;         // wavefront groups (each walks its own blocks)
  constexpr int WAVE_LDS_FLOATS = wave_lds_floats(NG, DS);
  constexpr int NPG = PP ? 2 : 4;             // score MFMA groups per block: pages, or pairs of pages
  static_assert(NG >= 2 && NG % 2 == 0 && (DW % 128 == 0 || (D == 64 && DS == 1)),
                "a wavefront takes whole 128-coordinate chunks (or a whole head of 64) and whole group pairs");
  static_assert(!PP || (D == 64 && DS == 1), "page pairs are for head_dim 64");
  static_assert(!(PP && NR), "page pairs use both row sets");
  static_assert(!SG || (NKW >= 3 && !PP), "staged loads take 12 or 16 key bytes per lane");
  constexpr int STAGE_BYTES = stage_bytes(VW);
  constexpr int NRS = NR ? 1 : 2;             // fp6 operands (row sets) per plane word
  // Four stored index planes (5-bit keys: nine term planes with the multi-bit terms and the signs): the query
  // operands - 72 to 144 registers - stay in LDS, one copy per workgroup, and the score stage walks a block plane
  // by plane so that an operand is read once for its four pages.
  constexpr bool QL = MB >= 4;
  static_assert(!QL || (!PP && !SG && DS == 1), "operands in LDS: head_dim 128, page data in registers");
  static_assert(IW == 0 || (DS == 1 && !QL && (IW == 1 || IW == 2)), "a (sequence, head group) per wavefront: wavefronts that work alone, operands in registers");
  constexpr int NJ = NR ? 1 : 2;              // heads a lane sees in the score MFMA's output
  // Hkv counts query-head groups: a KV head with more than 8 query heads is served by kv_div groups of at most 8
  // heads each (consecutive groups read the same pages); when the heads do not divide evenly the last group of
  // a KV head has fewer (11 heads: 6 + 5).  G = heads of this workgroup's group, qbase = its first query head.
  int G = Hq / Hkv;
  // skew16 > 0 (an even number of splits; the grid is (n_split / 2, Hkv, 2 n_seq)): the workgroups of the first half
  // of the grid take the even splits, those of the second half the odd ones, and every even split takes
  // skew16 sixteenths of a split's trips over from its odd neighbour.  Workgroups are dispatched in grid order, two
  // to a compute unit, and a SIMD serves its older wavefronts first: with equal shares the first half of the grid
  // finishes early and the second half runs on alone.
  int split = blockIdx.x, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wgrp = wave / DS, hf = wave % DS; // block walker this wavefront belongs to; its share of the head
  // The groups of a KV head are (splits x KV heads) workgroups apart in the grid, not next to each other: workgroups
  // go to the card's eight dies in turn, each die has its own L2, and a distance that is a multiple of eight puts the
  // groups that read the same pages at the same time on the same die.
  int h = blockIdx.y, qbase;
  bool item_live = true;                        // IW: this wavefront has a (sequence, head group) to walk
  constexpr int IWC = IW > 0 ? IW : 1;
  const int wsub = IW > 0 ? wgrp % IWC : wgrp;  // this walker's number among those of its (sequence, head group)
  if constexpr (IW > 0) {
    const int item = blockIdx.y * (NW / DS / IWC) + wgrp / IWC, items = Hkv * n_seq;
    item_live = item < items;
    const int item_c = item_live ? item : items - 1;          // (a wavefront without an item repeats the last one and stores nothing)
    h = item_c % Hkv;
    b = item_c / Hkv;
  }
  if (kv_div > 1) {
    const int kv_heads = Hkv / kv_div, grp = h / kv_heads, kvh = h - grp * kv_heads;
    const int g_tot = Hq / kv_heads, g_max = (g_tot + kv_div - 1) / kv_div;
    h = kvh * kv_div + grp;
    qbase = kvh * g_tot + grp * g_max;
    G = min(g_max, g_tot - grp * g_max);
  } else {
    qbase = h * G;
  }
  if (DS == 2 && skew16 > 0) {                                  // (only the launcher of DS == 2 kernels passes a skew)
    // (n_seq arrives with the other kernel arguments; the grid's size would be one more scalar load of the
    // launch's implicit data in front of everything that depends on the sequence)
    const int late = b >= n_seq;
    b -= late ? n_seq : 0;
    split = 2 * split + late;
  }
  const int n = lane & 15, kb = lane >> 4;    // score stage: token / coordinate quarter; value stage: row / page
  TQ_STAMP(0);

  extern __shared__ __align__(16) unsigned char smem_raw[];
  float* s_p = (float*)smem_raw + wave * WAVE_LDS_FLOATS;   // [4 pages][8 heads][P_STRIDE]
  float* s_alpha = s_p + 4 * 8 * P_STRIDE;                 // [16]
  float* s_scale = s_alpha + 16;                            // [4 pages][NG][16 tokens] fp32, pre-scaled
  float* s_x = s_scale + 4 * NG * 16;                       // DS > 1: [parity][8][64] this wavefront's score halves
  float* s_x_peer = (float*)smem_raw + (wave ^ 1) * WAVE_LDS_FLOATS + (4 * 8 * P_STRIDE + 16 + 4 * NG * 16);
  float* s_red = (float*)smem_raw;                          // after the loop: [NGRP][G][D + 2]
  // SG: this wavefront's staging area behind the wavefronts' private regions
  // QL: the group's packed query operands behind the wavefronts' private regions
  uint32_t* qa_lds = (uint32_t*)(smem_raw + MF_WAVES * WAVE_LDS_FLOATS * sizeof(float));
  // QL: behind the operands, the constant parts of the scores of the heads a lane sees (the same for every wavefront;
  // indexed like the operands, so that the reads share their address register):
  // [64 operand slots][index part of head 0, 1, sign part of head 0, 1]
  float* c_lds = (float*)(qa_lds + (MB + NX + 1) * WPLT * 2 * (64 * 6));
  unsigned char* stage = smem_raw + MF_WAVES * WAVE_LDS_FLOATS * sizeof(float) + wave * STAGE_BYTES;
  unsigned char* stage_m = stage + 4 * 1024;
  unsigned char* stage_v = stage_m + 512;
  unsigned char* stage_z = stage_v + (VW / 4) * 1024;
  unsigned char* stage_s = stage_z + 2 * 1024;

  // ---------------------------------------------------------------- A operands of the score stage
  // fp6 query terms in register order (see the preparation kernel): row set 0 = terms 0, 1 of the 8
  // heads (row 2g + t), row set 1 = terms 2, 3; rows of absent heads are zero.  Six dwords per
  // lane are stored at a stride of eight.
  i32x8 qa[QL ? 1 : NTP][WPL][NRS];
  int sa = 0;
  // QL: an operand in LDS is [64 lanes][4 dwords] followed by [64 lanes][2 dwords] (QA_OP dwords), so that both reads of
  // a lane, 16 and 8 bytes, are contiguous across the lanes; qa_lane = this lane's slot, qa_sel = (NR) its row set's operand
  constexpr int QA_OP = 64 * 6;
  int qa_lane = 0, qa_sel = 0;
  f32x4 cm = {0, 0, 0, 0}, cq = {0, 0, 0, 0};
  auto load_operands = [&]() {
  {
    // PP: rows 8..15 / coordinates 64..127 repeat rows 0..7 / coordinates 0..63; the off-diagonal blocks are zero
    // NR: row 4g + t is row 2g + t % 2 of row set t / 2
    const int slane = PP ? (n & 7) + 16 * (kb & 1) : (NR ? 2 * (n >> 2) + (n & 1) + 16 * kb : lane);
    const bool a_live = !PP || ((n < 8) == (kb < 2));
    const uint32_t* src = qa_pack + (((int64_t)b * Hkv + h) * (NTP * WPLT * 2 * 64) + slane) * 8 +
                          (NR ? ((n >> 1) & 1) * (64 * 8) : 0);
    if constexpr (QL) {
      // the whole block of the group, 16 bytes per lane and step, as it lies in memory
      const uint32_t* blk = qa_pack + ((int64_t)b * Hkv + h) * (NTP * WPLT * 2 * 64 * 8);
      for (int o = tid; o < NTP * WPLT * 2 * 64 * 2; o += MF_WAVES * 64) {       // o: 16-byte piece, two per lane slot
        const u32x4 v = *(const u32x4*)(blk + o * 4);
        uint32_t* op = qa_lds + (o >> 7) * QA_OP;
        const int sl = (o >> 1) & 63;
        if (o & 1) *(uint2*)(op + 64 * 4 + sl * 2) = make_uint2(v[0], v[1]);
        else *(u32x4*)(op + sl * 4) = v;
      }
      qa_lane = slane;
      qa_sel = NR ? ((n >> 1) & 1) * QA_OP : 0;
      __syncthreads();
    } else
#pragma unroll
    for (int tp = 0; tp < NTP; ++tp)
#pragma unroll
      for (int i = 0; i < WPL; ++i)
#pragma unroll
        for (int rs = 0; rs < NRS; ++rs) {
          const uint32_t* p6 = src + ((tp * WPLT + hf * WPL + i) * 2 + rs) * (64 * 8);
          const u32x4 lo = *(const u32x4*)p6;
          const uint32_t d4 = p6[4], d5 = p6[5];
          qa[tp][i][rs] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)d4, (int)d5, 0, 0};
          if (!a_live) qa[tp][i][rs] = i32x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
  }
  // E8M0 block-scale codes of this lane's operand row (head n / 2), one per byte: index planes row
  // set 0, row set 1, sign plane row set 0, row set 1.  4 v / 2^E is stored, so term t carries
  // 2^(E - 2 - 5t); the fp4 bit value 0.5 carries 2^1.
  {
    const int g = PP ? (n & 7) >> 1 : (NR ? n >> 2 : n >> 1);
    const int64_t qrow = (int64_t)b * Hq + qbase + (g < G ? g : 0);
    const int e1 = 127 + (int)q_stat[qrow * 4 + 0];
    const int e2 = 127 + (int)q_stat[qrow * 4 + 1];
    const int t01 = (n & 1) ? 7 : 2, t23 = t01 + 10;
    sa = (e1 - t01) | ((e1 - t23) << 8) | ((e2 - t01) << 16) | ((e2 - t23) << 24);
    if (NR) {                                    // one row set: byte 0 index planes, byte 2 sign plane
      const int tn = 2 + 5 * (n & 3);
      sa = (e1 - tn) | ((e2 - tn) << 16);
    }
  }
  // constant parts of the scores of the two heads this lane sees in the MFMA output (rows 4kb..4kb+3
  // = heads 2kb, 2kb+1), as the initial accumulators; only one wavefront of a pair adds them
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int g = PP ? 2 * (kb & 1) + j : (NR ? kb : 2 * kb + j);
    const bool live = g < G && hf == 0;
    const int64_t qrow = (int64_t)b * Hq + qbase + (g < G ? g : 0);
    const float c2 = q_stat[qrow * 4 + 2], c3 = q_stat[qrow * 4 + 3];
    cm[2 * j] = live ? c2 : 0.0f;
    cq[2 * j] = live ? c3 : 0.0f;
    if (QL) {                                     // (lanes that share an operand slot see the same heads)
      c_lds[qa_lane * 4 + j] = live ? c2 : 0.0f;
      c_lds[qa_lane * 4 + 2 + j] = live ? c3 : 0.0f;
    }
  }
  };
  load_operands();
  const int sb = 127 + 1;
  // head_dim 64: the score MFMA still contracts 128 coordinates; the lanes of the upper two coordinate
  // quarters feed zeros (their masks are zero, whatever their loads return)
  const bool kq_live = D >= 128 || PP || kb < D / 32;
  const uint32_t nib = in_vgpr(kq_live ? 0x11111111u : 0u), nib1 = in_vgpr(kq_live ? 0x22222222u : 0u),
                 nib2 = in_vgpr(kq_live ? 0x44444444u : 0u);
  int xplanes[NX > 0 ? NX : 1];                 // which stored planes each extra term XORs
  {
    int seen = 0;
    for (int t = 0; t < ly.n_terms; ++t) {
      if (__builtin_popcount(ly.term_mask[t]) > 1 && seen < NX) {
        int pl = 0;
        for (int k2 = 0; k2 < MB; ++k2)
          if (ly.term_mask[t] & (1 << k2)) pl |= 1 << (MB - 1 - k2);
        xplanes[seen++] = __builtin_amdgcn_readfirstlane(pl);
      }
    }
  }

  if (PP || NR) {
    // rows of heads 4..7 are never written with at most four heads; the value stage reads them as operand rows
    // whose results nobody uses: keep them finite
    for (int i = lane; i < 4 * 8 * P_STRIDE + 16; i += 64) s_p[i] = 0.0f;
  }
  TQ_STAMP(1);
  // ---------------------------------------------------------------- work range (all scalar)
  // len_sub: newest tokens that are attended to exactly.  A length beyond the block table is cut to the table.
  const int seq_len = item_live ? max(min(seq_lens[b], max_pages * TQ_PAGE_TOKENS) - len_sub, 0) : 0;
  const int n_pages = (seq_len + TQ_PAGE_TOKENS - 1) / TQ_PAGE_TOKENS;
  int blk_begin, blk_end;
  decode_block_range(seq_len, n_split, split, DS == 2 ? skew16 : 0, NGRP, blk_begin, blk_end);
  const int32_t* bt = block_table + (int64_t)b * bt_stride;
  const uint8_t* pool_h = pool + (int64_t)(h / kv_div) * L.page_bytes;
  const int64_t page_stride = (int64_t)(Hkv / kv_div) * L.page_bytes;
  const uint32_t page_stride32 = (uint32_t)page_stride;
  // per lane the key words are [word i][plane], the value fields [channel tile]: a wavefront's share is contiguous
  // (head_dim 64: the idle lanes re-read the last live lane's words)
  // (PP: every lane is live: word kb % 2 of token n, of the pair's first page for kb < 2, else of its second)
  const int klane = D >= 128 ? lane : (PP ? (kb & 1) * 16 + n : min(lane, D / 2 - 1));
  const uint32_t off_keys = L.off_keys + (klane * DS + hf) * (NKW * 4), off_meta = L.off_meta + n * 8;
  const uint32_t off_v = L.off_vdata + (n * DS + hf) * (VW * 4);
  const uint32_t off_scale = L.off_vscale + hf * (NG * 32) + (lane % PIECES) * 16;

  f32x4 acc[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) acc[c] = f32x4{0, 0, 0, 0};
  f32x4 zacc = {0, 0, 0, 0};
  // m_run is the reference the weights are taken against (exp2(score - m_run)); it only moves when
  // a score exceeds it by more than REF_SLACK, so the usual block needs no row reduction.  The slack
  // is small on purpose: a token that dominates its row should sit at (or near) the reference, where
  // its weight 1.0 survives the bf16 rounding of the value-stage operands exactly.
  constexpr float REF_SLACK = 4.0f;
  float m_run[NJ], l_run[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) { m_run[j] = MF_NEG; l_run[j] = 0.0f; }

  struct KeyRegs { uint32_t key[NPG][NKW]; f32x2 meta[NPG]; };
  struct ValRegs { uint32_t v[VW]; u32x4 zero[2]; u32x4 scale; };

  // page ids of block `blk` -> 4 scalars; a page past the end of the sequence (last block only) is
  // replaced by the block's first page, which always exists.  CHECK: a table entry outside the pool (a
  // stale or poisoned entry) is replaced by page 0 and reported in the returned mask (bit pg); the block
  // then takes the masking path, where those tokens get no weight.
  auto page_ids = [&](int blk, int (&pid)[4], auto check_tag) -> int {
    constexpr bool CHECK = decltype(check_tag)::value;
    int bad = 0;
    // one 64-bit address per block; the four entries are read at 32-bit scalar offsets from it
    const int32_t* row = bt + 4 * blk;
    const int last = n_pages - 1 - 4 * blk;               // >= 0: the block has at least one page
#pragma unroll
    for (int pg = 0; pg < 4; ++pg) {
      const int raw = row[min(pg, last)];
      const bool ok = !CHECK || (unsigned)raw < (unsigned)num_pages;
      pid[pg] = ok ? raw : 0;
      bad |= ok ? 0 : 1 << pg;
    }
    return bad;
  };
  auto load_keys = [&](const int (&pid)[4], KeyRegs& R) __attribute__((always_inline)) {
    // the 32-bit lane offsets are re-materialised here, next to their use, so that the loads take
    // the scalar page base plus a 32-bit vector offset instead of a 64-bit vector address
    const uint32_t ok = in_vgpr(off_keys), om = in_vgpr(off_meta);
    if constexpr (PP) {
      const uint32_t p0 = in_vgpr((uint32_t)pid[0]), p1 = in_vgpr((uint32_t)pid[1]), p2 = in_vgpr((uint32_t)pid[2]),
                     p3 = in_vgpr((uint32_t)pid[3]);
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const uint32_t my_pid = kb < 2 ? (pr == 0 ? p0 : p2) : (pr == 0 ? p1 : p3);
        const uint8_t* base = pool_h + (uint64_t)my_pid * page_stride32;
        const uint32_t* kp = (const uint32_t*)(base + ok);
#pragma unroll
        for (int w = 0; w < NKW; ++w) R.key[pr][w] = kp[w];
        R.meta[pr] = *(const f32x2*)(base + om);
      }
    } else
#pragma unroll
    for (int pg = 0; pg < 4; ++pg) {
      // (page numbers are non-negative and the stride fits 32 bits: an unsigned 32 x 32 -> 64 bit product)
      const uint8_t* base = pool_h + (uint64_t)(uint32_t)pid[pg] * page_stride32;
      const uint32_t* kp = (const uint32_t*)(base + ok);
#pragma unroll
      for (int w = 0; w < NKW; ++w) R.key[pg][w] = kp[w];
      R.meta[pg] = *(const f32x2*)(base + om);
    }
  };
  // All loads below are unconditional (lanes without a group / piece of their own read a
  // neighbour's): a load inside a branch would make the wait counters at the join conservative
  // and serialise the prefetch.
  const uint32_t off_zero_c = L.off_vzero + min(n, NGT - 1) * 32;
  const int spg = min(lane / PIECES, 3);
  // The page of a lane is picked among the four page numbers with conditional moves on vector
  // registers (on scalar operands the compiler builds branches instead) and turned into an address
  // with one unsigned 32 x 32 -> 64 bit multiply-add.
  auto load_vals = [&](const int (&pid)[4], ValRegs& R) __attribute__((always_inline)) {
    const uint32_t p0 = in_vgpr((uint32_t)pid[0]), p1 = in_vgpr((uint32_t)pid[1]), p2 = in_vgpr((uint32_t)pid[2]),
                   p3 = in_vgpr((uint32_t)pid[3]);
    const uint32_t my_pid = kb == 0 ? p0 : (kb == 1 ? p1 : (kb == 2 ? p2 : p3));
    const uint8_t* vbase = pool_h + (uint64_t)my_pid * page_stride32;
    const uint32_t* vp = (const uint32_t*)(vbase + off_v);
#pragma unroll
    for (int w = 0; w < VW; ++w) R.v[w] = vp[w];
    const u32x4* zp = (const u32x4*)(vbase + off_zero_c);
    R.zero[0] = zp[0];
    R.zero[1] = zp[1];
    const uint32_t spid = spg == 0 ? p0 : (spg == 1 ? p1 : (spg == 2 ? p2 : p3));
    R.scale = *(const u32x4*)(pool_h + (uint64_t)spid * page_stride32 + off_scale);
  };

  // SG: requests for a block's page data (fixed numbers of instructions: the waits below count them) and the
  // copies LDS -> registers
  constexpr int K_OPS = 5, V_OPS = VW / 4 + 3;
  auto dma_keys = [&](const int (&pid)[4]) {
    const uint32_t ok = in_vgpr(off_keys);
    const uint32_t m0k = (uint32_t)(uintptr_t)stage;
#pragma unroll
    for (int pg = 0; pg < 4; ++pg)
      dma_so<NKW * 4>(ok, pool_h + (uint64_t)(uint32_t)pid[pg] * page_stride32, m0k + pg * 1024);
    // norms: lane l < 32 takes the (norm, residual norm) pairs of tokens 2 (l % 8), 2 (l % 8) + 1 of page l / 8
    const uint32_t p0 = in_vgpr((uint32_t)pid[0]), p1 = in_vgpr((uint32_t)pid[1]), p2 = in_vgpr((uint32_t)pid[2]),
                   p3 = in_vgpr((uint32_t)pid[3]);
    const int mp = (lane >> 3) & 3;
    const uint32_t mpid = mp == 0 ? p0 : (mp == 1 ? p1 : (mp == 2 ? p2 : p3));
    const uint8_t* ma = pool_h + (uint64_t)mpid * page_stride32 + (L.off_meta + (lane & 7) * 16);
    if (lane < 32) dma16<0>(ma, (uint32_t)(uintptr_t)stage_m);
  };
  auto fetch_keys = [&](KeyRegs& R) {
#pragma unroll
    for (int pg = 0; pg < 4; ++pg) {
      const uint32_t* kp = (const uint32_t*)(stage + pg * 1024 + lane * 16);
      if (NKW == 4) {
        const u32x4 t = *(const u32x4*)kp;
#pragma unroll
        for (int w = 0; w < NKW; ++w) R.key[pg][w] = t[w];
      } else {
#pragma unroll
        for (int w = 0; w < NKW; ++w) R.key[pg][w] = kp[w];
      }
      R.meta[pg] = *(const f32x2*)(stage_m + (pg * 16 + n) * 8);
    }
  };
  auto dma_vals = [&](const int (&pid)[4]) {
    const uint32_t p0 = in_vgpr((uint32_t)pid[0]), p1 = in_vgpr((uint32_t)pid[1]), p2 = in_vgpr((uint32_t)pid[2]),
                   p3 = in_vgpr((uint32_t)pid[3]);
    const uint32_t my_pid = kb == 0 ? p0 : (kb == 1 ? p1 : (kb == 2 ? p2 : p3));
    const uint8_t* vbase = pool_h + (uint64_t)my_pid * page_stride32;
    const uint32_t m0v = (uint32_t)(uintptr_t)stage_v, m0z = (uint32_t)(uintptr_t)stage_z;
    // (the instruction offset moves the LDS address as well as the memory address)
    static_assert(!SG || VW == 8 || VW == 16, "two or four pieces of value words");
    dma16<0>(vbase + off_v, m0v);
    dma16<16>(vbase + off_v, m0v + 1 * (1024 - 16));
    if (VW == 16) {
      dma16<32>(vbase + off_v, m0v + 2 * (1024 - 16));
      dma16<48>(vbase + off_v, m0v + 3 * (1024 - 16));
    }
    dma16<0>(vbase + off_zero_c, m0z);
    dma16<16>(vbase + off_zero_c, m0z + (1024 - 16));
    const uint32_t spid = spg == 0 ? p0 : (spg == 1 ? p1 : (spg == 2 ? p2 : p3));
    dma16<0>(pool_h + (uint64_t)spid * page_stride32 + off_scale, (uint32_t)(uintptr_t)stage_s);
  };
  auto fetch_vals = [&](ValRegs& R) {
#pragma unroll
    for (int j = 0; j < VW / 4; ++j) {
      const u32x4 t = *(const u32x4*)(stage_v + (j * 64 + lane) * 16);
#pragma unroll
      for (int w = 0; w < 4; ++w) R.v[4 * j + w] = t[w];
    }
    R.zero[0] = *(const u32x4*)(stage_z + lane * 16);
    R.zero[1] = *(const u32x4*)(stage_z + (64 + lane) * 16);
    R.scale = *(const u32x4*)(stage_s + lane * 16);
  };

  // A value code masked in place is a bf16 number: a pattern n < 256 in a 16-bit half is n * 2^-133
  // exactly (denormals, and the first binade continues them linearly), so B = code * 2^(s - 133)
  // where s is the bit position the code has inside its byte; the softmax weight carries 2^(80 - s).
  // Only the codes in the upper byte of each half need a shift.
  const uint32_t m0 = in_vgpr(VB == 2 ? 0x00030003u : (VB == 4 ? 0x000F000Fu : 0x00FF00FFu));
  const uint32_t m1 = in_vgpr(VB == 2 ? 0x000C000Cu : 0x00F000F0u), m2 = in_vgpr(0x00300030u), m3 = in_vgpr(0x00C000C0u);

  // ---------------------------------------------------------------- one block of 64 tokens
  // scores of the 4 pages of block blk, online softmax, weights -> LDS
  // PARTIAL: some tokens of the block do not exist (the ragged end of the sequence, pages named in `bad`)
  auto tokens_of_page = [&](int blk, int pg, int bad) -> int {          // existing tokens of page pg: a prefix
    return ((bad >> pg) & 1) ? 0 : min(max(seq_len - (blk * BLK_TOK + pg * 16), 0), 16);
  };
  bool fresh = true;                            // this walker has not seen a token yet: no reference
  // (always inlined: an outlined stage would pass the block's page data through memory)
  auto score_stage = [&](int blk, int it, bool first, const KeyRegs& K, int bad, auto partial_tag)
                         __attribute__((always_inline)) -> bool {
    constexpr bool PARTIAL = decltype(partial_tag)::value;
    float s2[NJ][NPG];
    float mref[NJ];                             // only one wavefront of a pair subtracts it
#pragma unroll
    for (int j = 0; j < NJ; ++j) mref[j] = (first || hf != 0) ? 0.0f : m_run[j];
    // The MFMA-dense parts run at raised wavefront priority (the value stage above the score
    // stage): the SIMD's other wavefront then fills the gaps with its vector-ALU work instead of
    // both alternating between the two kinds of instruction.
    __builtin_amdgcn_s_setprio(1);
    if constexpr (QL) {
      f32x4 dmp[NPG], dqp[NPG];
#pragma unroll
      for (int pg = 0; pg < NPG; ++pg) { dmp[pg] = f32x4{0, 0, 0, 0}; dqp[pg] = f32x4{0, 0, 0, 0}; }
#pragma unroll
      for (int i = 0; i < WPL; ++i) {
#pragma unroll
        for (int tp = 0; tp < NTP; ++tp) {
          i32x8 a[NRS];
#pragma unroll
          for (int rs = 0; rs < NRS; ++rs) {
            const uint32_t* op = qa_lds + ((tp * WPLT + hf * WPL + i) * 2 + rs) * QA_OP + qa_sel;
            const u32x4 lo = *(const u32x4*)(op + qa_lane * 4);
            const uint2 hi = *(const uint2*)(op + 64 * 4 + qa_lane * 2);
            a[rs] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi.x, (int)hi.y, 0, 0};
          }
#pragma unroll
          for (int pg = 0; pg < NPG; ++pg) {
            uint32_t x;
            if (tp < MB) x = K.key[pg][i * (MB + 1) + tp];
            else if (tp == NTP - 1) x = K.key[pg][i * (MB + 1) + MB];
            else {
              x = 0;
#pragma unroll
              for (int p = 0; p < MB; ++p) x ^= ((xplanes[tp - MB] >> p) & 1) ? K.key[pg][i * (MB + 1) + p] : 0u;
            }
            const uint32_t b0 = x & nib, b1 = x & nib1, b2 = x & nib2, b3 = (x >> 3) & nib;
            if (tp == NTP - 1) {
              dqp[pg] = mfma_f8f4<2>(a[0], b0, b1, b2, b3, dqp[pg], sa, sb);
              if (!NR) dqp[pg] = mfma_f8f4<3>(a[NRS - 1], b0, b1, b2, b3, dqp[pg], sa, sb);
            } else {
              dmp[pg] = mfma_f8f4<0>(a[0], b0, b1, b2, b3, dmp[pg], sa, sb);
              if (!NR) dmp[pg] = mfma_f8f4<1>(a[NRS - 1], b0, b1, b2, b3, dmp[pg], sa, sb);
            }
          }
          // (the next plane's operands are not to be read before this plane is done: all nine at once do not fit)
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // The constant parts of the scores are added here, from LDS.  As initial accumulators they would sit in eight
      // registers through the whole loop, the register allocator would keep them in scratch memory instead, and a
      // reload from scratch inside the loop is the worst there is: vector memory instructions return in order, so
      // waiting for it means waiting for the page data requested just before, which has the whole stage to arrive.
      const f32x4 cc = *(const f32x4*)(c_lds + qa_lane * 4);
#pragma unroll
      for (int pg = 0; pg < NPG; ++pg) {
        const f32x4 dm = dmp[pg], dq = dqp[pg];
        const float nk = K.meta[pg][0], rk = K.meta[pg][1];
        if (NR) {
          s2[0][pg] = fmaf(nk, ((dm[0] + cc[0]) + dm[1]) + (dm[2] + dm[3]),
                           fmaf(rk, ((dq[0] + cc[2]) + dq[1]) + (dq[2] + dq[3]), -mref[0]));
        } else {
#pragma unroll
          for (int j = 0; j < NJ; ++j)
            s2[j][pg] = fmaf(nk, (dm[2 * j] + cc[j]) + dm[2 * j + 1], fmaf(rk, (dq[2 * j] + cc[2 + j]) + dq[2 * j + 1], -mref[j]));
        }
      }
    } else {
#pragma unroll
    for (int pg = 0; pg < NPG; ++pg) {
      f32x4 dm = cm, dq = cq;
#pragma unroll
      for (int i = 0; i < WPL; ++i) {
#pragma unroll
        for (int tp = 0; tp < NTP; ++tp) {
          uint32_t x;
          if (tp < MB) x = K.key[pg][i * (MB + 1) + tp];
          else if (tp == NTP - 1) x = K.key[pg][i * (MB + 1) + MB];
          else {
            x = 0;
#pragma unroll
            for (int p = 0; p < MB; ++p) x ^= ((xplanes[tp - MB] >> p) & 1) ? K.key[pg][i * (MB + 1) + p] : 0u;
          }
          const uint32_t b0 = x & nib, b1 = x & nib1, b2 = x & nib2, b3 = (x >> 3) & nib;
          if (tp == NTP - 1) {
            dq = mfma_f8f4<2>(qa[tp][i][0], b0, b1, b2, b3, dq, sa, sb);
            if (!NR) dq = mfma_f8f4<3>(qa[tp][i][NRS - 1], b0, b1, b2, b3, dq, sa, sb);
          } else {
            dm = mfma_f8f4<0>(qa[tp][i][0], b0, b1, b2, b3, dm, sa, sb);
            if (!NR) dm = mfma_f8f4<1>(qa[tp][i][NRS - 1], b0, b1, b2, b3, dm, sa, sb);
          }
        }
      }
      const float nk = K.meta[pg][0], rk = K.meta[pg][1];
      // this wavefront's share of the score (the whole score when DS == 1), relative to the reference
      if (NR) {
        s2[0][pg] = fmaf(nk, (dm[0] + dm[1]) + (dm[2] + dm[3]), fmaf(rk, (dq[0] + dq[1]) + (dq[2] + dq[3]), -mref[0]));
      } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          s2[j][pg] = fmaf(nk, dm[2 * j] + dm[2 * j + 1], fmaf(rk, dq[2 * j] + dq[2 * j + 1], -mref[j]));
      }
    }
    // Wanted issue order of the section above: the bit expansion of the first page, then every MFMA
    // followed by a few vector instructions (the next page's expansion, the previous page's score
    // arithmetic), which run in the shadow of the matrix pipe.
    __builtin_amdgcn_sched_group_barrier(0x002, 5 * NTP * WPL, 0);
#pragma unroll
    for (int k = 0; k < NPG * NRS * NTP * WPL; ++k) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
    }
    }
    __builtin_amdgcn_s_setprio(0);
    if constexpr (DS > 1) {
      // exchange with the wavefront that scored the other coordinates: own share -> LDS, workgroup
      // barrier, partner's share <- LDS.  a + b == b + a, so both end with bit-identical scores.
      float* mine = s_x + (it & 1) * (8 * 64);
      const float* theirs = s_x_peer + (it & 1) * (8 * 64);
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int pg = 0; pg < 4; ++pg) mine[(j * 4 + pg) * 64 + lane] = s2[j][pg];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int pg = 0; pg < 4; ++pg) s2[j][pg] += theirs[(j * 4 + pg) * 64 + lane];
    }
    bool gone[NPG];
#pragma unroll
    for (int pg = 0; pg < NPG; ++pg) gone[pg] = false;
    if (PARTIAL) {
      bool any = false;
#pragma unroll
      for (int pg = 0; pg < NPG; ++pg) {
        gone[pg] = n >= tokens_of_page(blk, PP ? 2 * pg + (kb >> 1) : pg, bad);
        any |= !gone[pg];
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          if (gone[pg]) s2[j][pg] = MF_NEG;
      }
      // a block without a single token leaves the walker as it was (the next block is still its first)
      fresh = fresh && __builtin_amdgcn_ballot_w64(any) == 0;
    }
    // ---- online softmax (log2 domain) against a lazily updated reference
    float mx = fmaxf(s2[0][0], s2[NJ - 1][0]);
#pragma unroll
    for (int pg = 1; pg < NPG; ++pg) mx = fmaxf(mx, fmaxf(s2[0][pg], s2[NJ - 1][pg]));
    const bool rescale = first || __builtin_amdgcn_ballot_w64(mx > REF_SLACK) != 0;
    if (rescale) {
      // move the reference to the row maximum (never down, except for the first block, where the
      // accumulators are still empty and keep their scale); every lane of a row computes the same
      float alpha[NJ];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        float mj = s2[j][0];
#pragma unroll
        for (int pg = 1; pg < NPG; ++pg) mj = fmaxf(mj, s2[j][pg]);
        mj = row_max16(mj);
        if (PP) mj = max_xor32(mj);                 // the lanes 32 apart hold the same heads
        const float delta = first ? mj : fmaxf(mj, 0.0f);
        alpha[j] = first ? 1.0f : __builtin_amdgcn_exp2f(-delta);
        m_run[j] = first ? delta : m_run[j] + delta;
        l_run[j] *= alpha[j];
#pragma unroll
        for (int pg = 0; pg < NPG; ++pg) s2[j][pg] -= delta;
      }
      if (NR) {
        if (n == 0) s_alpha[kb] = alpha[0];
      } else if (n == 0 && (!PP || kb < 2)) {
        s_alpha[2 * kb] = alpha[0];
        s_alpha[2 * kb + 1] = alpha[NJ - 1];
      }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      float psum = 0.0f;
#pragma unroll
      for (int pg = 0; pg < NPG; ++pg) {
        // (a token that does not exist has weight 0 even when the whole block is empty and the
        // reference therefore sits at the masking value itself)
        const float p = PARTIAL && gone[pg] ? 0.0f : __builtin_amdgcn_exp2f(s2[j][pg]);
        psum += p;
        if (PP) s_p[((2 * pg + (kb >> 1)) * 8 + 2 * (kb & 1) + j) * P_STRIDE + n] = p;
        else if (NR) s_p[(pg * 8 + kb) * P_STRIDE + n] = p;
        else s_p[(pg * 8 + 2 * kb + j) * P_STRIDE + n] = p;
      }
      l_run[j] += psum;
    }
    return rescale;
  };
  // weights x (codes, scales, zeros) of block blk into the accumulators
  auto value_stage = [&](int blk, const ValRegs& V, bool rescale, int bad, auto partial_tag) __attribute__((always_inline)) {
    constexpr bool PARTIAL = decltype(partial_tag)::value;
    // scales -> LDS as fp32 [page][group][16 tokens]; first use of the value loads.  The lane that
    // holds a 16-byte piece widens it once (instead of all 16 row lanes later), folds in the
    // 2^-s of its tokens' code position and zeroes tokens past the end of the sequence.
    if (lane < 4 * PIECES) {
      const int spage = lane / PIECES, pc = lane % PIECES;
      float f[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        f[2 * i] = F16P ? f16_lo(V.scale[i]) : __uint_as_float(V.scale[i] << 16);
        f[2 * i + 1] = F16P ? f16_hi(V.scale[i]) : __uint_as_float(V.scale[i] & 0xffff0000u);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        constexpr float k_pow[4] = {0x1p80f, 0x1p78f, 0x1p76f, 0x1p74f};
        f[e] *= k_pow[v_bitpos<VB>(e) / 2];
      }
      if (PARTIAL) {
        const int nv = tokens_of_page(blk, spage, bad) - 8 * (pc & 1);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = e < nv ? f[e] : 0.0f;
      }
      f32x4* dst = (f32x4*)(s_scale + (spage * NG + (pc >> 1)) * 16 + 8 * (pc & 1));
      dst[0] = f32x4{f[0], f[1], f[2], f[3]};
      dst[1] = f32x4{f[4], f[5], f[6], f[7]};
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (rescale) {
      const f32x4 a4 = *(const f32x4*)(s_alpha + 4 * (kb & 1)); // accumulator rows 4kb..4kb+3 = heads 4(kb%2)..
#pragma unroll
      for (int c = 0; c < CT; ++c) acc[c] *= a4;
      zacc *= a4;
    }
    // ---- value stage: lane = (row n = head n % 8 with the scales of group parity n / 8, page kb)
    float pr[16];
    {
      const f32x4* pp = (const f32x4*)(s_p + (kb * 8 + (n & 7)) * P_STRIDE);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 t = pp[q4];
        pr[4 * q4] = t[0]; pr[4 * q4 + 1] = t[1]; pr[4 * q4 + 2] = t[2]; pr[4 * q4 + 3] = t[3];
      }
    }
    // validity of this lane's page tokens (last block only): bit t set = token t of page kb exists
    uint32_t keep[8];
    if (PARTIAL) {
      const int nv = tokens_of_page(blk, kb, bad);
      const uint32_t tokmask = (1u << nv) - 1u;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        keep[i] = ((tokmask >> (2 * i)) & 1u ? 0x0000ffffu : 0u) | ((tokmask >> (2 * i + 1)) & 1u ? 0xffff0000u : 0u);
    }
    // zero points: weights (natural token order) x zeros
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      u32x4 ap, bz = V.zero[u];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        ap[r] = F16P ? pack_f16(pr[8 * u + 2 * r], pr[8 * u + 2 * r + 1])
                     : pack_bf16(pr[8 * u + 2 * r], pr[8 * u + 2 * r + 1]);
        if (PARTIAL) bz[r] &= keep[4 * u + r];
      }
      zacc = F16P ? mfma_f16(ap, bz, zacc) : mfma(ap, bz, zacc);
    }
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int gp = 0; gp < NG / 2; ++gp) {
      // w = weight * scale for the 16 tokens of page kb, then the two A operands in the value token order
      float w[16];
      {
        const f32x4* sp = (const f32x4*)(s_scale + (kb * NG + 2 * gp + (n >> 3)) * 16);
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const f32x4 sv = sp[q4];
#pragma unroll
          for (int e = 0; e < 4; ++e) w[4 * q4 + e] = pr[4 * q4 + e] * sv[e];
        }
      }
      u32x4 aw[2];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) aw[u][r] = pack_bf16(w[v_token<VB>(u, r, 0)], w[v_token<VB>(u, r, 1)]);
#pragma unroll
      for (int cc = 0; cc < 2 * CTG; ++cc) {
        const int c = gp * 2 * CTG + cc;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          u32x4 bc;
          if (VB == 2) {
            // 16 two-bit fields; register r of MFMA u takes fields 4u+r (low half) and 4u+r+8 (high half)
            const uint32_t x = u == 0 ? V.v[c] : V.v[c] >> 8;
            bc = u32x4{x & m0, x & m1, x & m2, x & m3};
          } else if (VB == 4) {
            // 8 four-bit fields; register r takes fields r (low half) and r+4 (high half)
            const uint32_t x = V.v[2 * c + u], x8 = x >> 8;
            bc = u32x4{x & m0, x & m1, x8 & m0, x8 & m1};
          } else {
            // four bytes per dword: the even bytes are one register (a code in the low byte of each half is a bf16
            // denormal as it stands), the odd bytes, shifted down, the next
            const uint32_t x = V.v[4 * c + 2 * u], y = V.v[4 * c + 2 * u + 1];
            bc = u32x4{x & m0, (x >> 8) & m0, y & m0, (y >> 8) & m0};
          }
          acc[c] = mfma(aw[u], bc, acc[c]);
        }
      }
    }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_wave_barrier();
  };

  // ---------------------------------------------------------------- pipeline over this walker's blocks
  // Registers are reloaded as soon as their last reader is done: the key words of
  // the next block are requested right after the score stage, its value words
  // right after the value stage.  With DS > 1 the score stage contains a workgroup
  // barrier, so every wavefront makes the same number of trips; a walker that has
  // run out of blocks only attends the barrier.
  {
    KeyRegs K;
    ValRegs V;
    int pid[4];
    constexpr int WSTEP = IW > 0 ? IW : NGRP;              // distance of a walker's consecutive blocks
    const int trips = (max(blk_end - blk_begin, 0) + WSTEP - 1) / WSTEP;
    int blk = blk_begin + wsub;
    int bad = 0;                                          // pages of the current block that lie outside the pool
    if (blk < blk_end) {
      bad = page_ids(blk, pid, std::true_type{});
      if constexpr (SG) {
        dma_keys(pid);
        dma_vals(pid);
      } else {
        load_keys(pid, K);
        load_vals(pid, V);
      }
    }
    // Block tables are device data nobody has checked: every wavefront looks once at the table entries of its
    // workgroup's blocks, a lane per entry: up to 256 entries in straight-line code (all loads unconditional
    // and inside the table row, requested behind the first block's loads so that nothing waits for them
    // alone), a loop for longer ranges.  Only a workgroup that finds an entry outside the pool runs the
    // checking loop.
    bool entry_bad = false;
    {
      const int e0 = 4 * blk_begin, e1 = min(4 * blk_end, n_pages), last = max(e1 - 1, 0);
      uint32_t raw[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) raw[i] = (uint32_t)bt[min(max(e0 + lane + 64 * i, 0), last)];
#pragma unroll
      for (int i = 0; i < 4; ++i) entry_bad |= e0 + lane + 64 * i < e1 && raw[i] >= (unsigned)num_pages;
      for (int e = e0 + 4 * 64 + lane; e < e1; e += 4 * 64) {
#pragma unroll
        for (int i = 0; i < 4; ++i) entry_bad |= (unsigned)bt[min(e + 64 * i, e1 - 1)] >= (unsigned)num_pages;
      }
    }
    // CHECKED: page ids are validated and every trip takes the masking (PARTIAL) path
    auto run = [&](auto checked_tag) __attribute__((always_inline)) {
      constexpr bool CHECKED = decltype(checked_tag)::value;
      // one trip of a walker that still has a block; PARTIAL: some tokens of the block may not exist
      // LAST: the walker's last trip (a code instance of its own behind the loop): nothing is requested
      auto trip = [&](int it, auto partial_tag, auto last_tag) __attribute__((always_inline)) {
        constexpr bool LAST = decltype(last_tag)::value;
        // the block after this walker's last one does not exist: re-request the current one instead,
        // so that the loads stay outside any branch
        const int nxt = blk + WSTEP;
        const int nxt_c = nxt < blk_end ? nxt : blk;
        int pid_n[4] = {0, 0, 0, 0};
        int bad_n = 0;
        if constexpr (!LAST) bad_n = page_ids(nxt_c, pid_n, checked_tag);   // scalar loads, consumed after the score stage
        if constexpr (LAST && !SG) {
          const bool rescale = score_stage(blk, it, CHECKED ? fresh : it == 0, K, bad, partial_tag);
          value_stage(blk, V, rescale, bad, partial_tag);
        } else if constexpr (LAST) {
          stage_wait<0>();                                  // this block's keys and values are all that is outstanding
          fetch_keys(K);
          const bool rescale = score_stage(blk, it, CHECKED ? fresh : it == 0, K, bad, partial_tag);
          fetch_vals(V);
          stage_release();
          value_stage(blk, V, rescale, bad, partial_tag);
        } else if constexpr (SG) {
          // outstanding, oldest first: this block's keys, this block's values
          stage_wait<V_OPS>();
          fetch_keys(K);
          stage_release();
          dma_keys(pid_n);
          const bool rescale = score_stage(blk, it, CHECKED ? fresh : it == 0, K, bad, partial_tag);
          // outstanding: this block's values, the next block's keys
          stage_wait<K_OPS>();
          fetch_vals(V);
          stage_release();
          dma_vals(pid_n);
          value_stage(blk, V, rescale, bad, partial_tag);
        } else {
          const bool rescale = score_stage(blk, it, CHECKED ? fresh : it == 0, K, bad, partial_tag);
          load_keys(pid_n, K);
          value_stage(blk, V, rescale, bad, partial_tag);
          load_vals(pid_n, V);
        }
        blk = nxt;
        bad = bad_n;
      };
      // A walker takes every NGRP-th block of the workgroup's range, so it can only run out of blocks,
      // and only meet the ragged end of the sequence, in the last trip: the loop before it is
      // straight-line code.
      for (int it = 0; it < trips - 1; ++it) trip(it, std::integral_constant<bool, CHECKED>{}, std::false_type{});
      if (trips > 0) {
        if (blk >= blk_end) {                              // uniform per wavefront pair
          if (DS > 1) __syncthreads();
        } else if (CHECKED || (blk + 1) * BLK_TOK > seq_len) {
          trip(trips - 1, std::true_type{}, std::true_type{});
        } else {
          trip(trips - 1, std::false_type{}, std::true_type{});
        }
      }
    };
    TQ_STAMP(2);
    if (__builtin_amdgcn_ballot_w64(entry_bad) != 0) run(std::true_type{});
    else run(std::false_type{});
  }

  // ---------------------------------------------------------------- merge the walkers, write the partial
  TQ_STAMP(3);
  if (SG) stage_wait<0>();   // the last trip's requests (a repeat of its own block) have landed
  __syncthreads();      // every wave is done with its private LDS region
  TQ_STAMP(6);
 const int g_rows = IW > 0 ? 8 : G;                              // rows of a walker in s_red (IW: the walkers' groups may differ in size)
  float* s_z = s_red + NGRP * g_rows * (D + 2);                // [MF_WAVES][16 rows][16 groups]
#pragma unroll
  for (int i = 0; i < 4; ++i) s_z[(wave * 16 + 4 * kb + i) * 16 + n] = zacc[i];
  if (hf == 0) {                                               // the wavefronts of a pair hold the same (m, l)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      float lsum = row_sum16(l_run[j]);
      if (PP) lsum = sum_xor32(lsum);
      const int g = PP ? 2 * (kb & 1) + j : (NR ? kb : 2 * kb + j);
      if (n == 0 && g < G && (!PP || kb < 2)) {
        float* r = s_red + (wgrp * g_rows + g) * (D + 2);
        r[0] = m_run[j] * 0.6931471805599453f;     // back to the natural-log domain of the partials
        r[1] = lsum;
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  // Accumulator rows 0..7 are valid for the channel tiles of even groups, rows 8..15 for odd groups:
  // a lane owns heads 4(kb%2)..+3 and the groups of parity kb/2.  Everything is read before the
  // first conditional store, so that no memory latency sits inside a branch.
  {
    const int par = kb >> 1;
    float zz[NG / 2][4];
#pragma unroll
    for (int gpi = 0; gpi < NG / 2; ++gpi)
#pragma unroll
      for (int i = 0; i < 4; ++i) zz[gpi][i] = s_z[(wave * 16 + 4 * (kb & 1) + i) * 16 + hf * NG + 2 * gpi + par];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int g = 4 * (kb & 1) + i;
      if (g < G) {
        float* row = s_red + (wgrp * g_rows + g) * (D + 2) + 2 + hf * DW + par * (16 * CTG) + n;
#pragma unroll
        for (int gpi = 0; gpi < NG / 2; ++gpi)
#pragma unroll
          for (int cc = 0; cc < CTG; ++cc) {
            const float v = par ? acc[(2 * gpi + 1) * CTG + cc][i] : acc[2 * gpi * CTG + cc][i];
            row[16 * (2 * gpi * CTG + cc)] = fmaf(v, 0x1p53f, zz[gpi][i]);
          }
      }
    }
  }
  __syncthreads();
  TQ_STAMP(7);
  if constexpr (IW > 0) {
    // The IW wavefronts of a (sequence, head group) finish it among themselves: their rows of s_red hold its walkers.
    constexpr int TP = 64 * IWC;                 // threads of a (sequence, head group)
    const int tsub = wsub * 64 + lane, w0 = wgrp - wsub;
    // log-sum-exp merge of the walkers' element e (0: the maximum itself, 1: the sum of weights, 2 + ch: a channel)
    auto merged = [&](int g, int e, float& mm, float& ll) -> float {
      float m_w[IWC], l_w[IWC], a_w[IWC];
      mm = MF_NEG;
#pragma unroll
      for (int w = 0; w < IWC; ++w) {
        const float* r = s_red + ((w0 + w) * g_rows + g) * (D + 2);
        m_w[w] = r[0]; l_w[w] = r[1]; a_w[w] = r[e];
        mm = fmaxf(mm, m_w[w]);
      }
      ll = 0.0f;
      float aa = 0.0f;
#pragma unroll
      for (int w = 0; w < IWC; ++w) {
        const float wgt = __expf(m_w[w] - mm);
        ll = fmaf(wgt, l_w[w], ll);
        aa = fmaf(wgt, a_w[w], aa);
      }
      return aa;
    };
    if (fm.out != nullptr && fm.n_extra <= 1) {
      // the attention output, merged with the exact tail's partial if there is one (an earlier launch wrote it)
#pragma unroll
      for (int k = 0; k < 8 * D / TP; ++k) {
        const int o = tsub + k * TP;
        const int g_o = o / D, ch = o % D;
        const bool live = item_live && g_o < G;
        const int g = live ? g_o : 0;
        float mm, ll;
        const float aa = merged(g, 2 + ch, mm, ll);
        if (live && fm.n_extra == 0) {
          const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;
          store_from_f32(fm.out, ((int64_t)b * Hq + qbase + g) * D + ch, aa * inv, fm.out_dtype);
        } else if (live) {
          const float* x = parts + (((int64_t)b * Hq + qbase + g) * n_parts + 1) * (D + 2);     // the exact tail's part
          const float m_x = x[0], l_x = x[1], a_x = x[2 + ch];
          float top = MF_NEG;
          if (ll > 0.0f) top = fmaxf(top, mm);
          if (l_x > 0.0f) top = fmaxf(top, m_x);
          const float w0x = ll > 0.0f ? __expf(mm - top) : 0.0f, w1x = l_x > 0.0f ? __expf(m_x - top) : 0.0f;
          const float l_all = fmaf(w1x, l_x, fmaf(w0x, ll, 0.0f)), a_all = fmaf(w1x, a_x, fmaf(w0x, aa, 0.0f));
          const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
          store_from_f32(fm.out, ((int64_t)b * Hq + qbase + g) * D + ch, a_all * inv, fm.out_dtype);
        }
      }
    } else {
      // the partial (m, l, acc[D]) of every head, for the merge kernel
      constexpr int PAIRS = (D + 2) / 2;
      for (int o = tsub; o < 8 * PAIRS; o += TP) {
        const int g = o / PAIRS, pr = o % PAIRS;
        if (item_live && g < G) {
          float mm, ll, m2, l2;
          const float a0 = merged(g, 2 * pr, mm, ll), a1 = merged(g, 2 * pr + 1, m2, l2);
          float* out = parts + (((int64_t)b * Hq + qbase + g) * n_parts + split) * (D + 2);
          store_coherent2(out + 2 * pr, pr == 0 ? f32x2{mm, ll} : f32x2{a0, a1});
        }
      }
    }
    return;
  }
  // merge of the walkers: thread -> (head, channel); loads are unconditional (clamped), stores guarded
  auto walkers_sum = [&](int g, int ch, float& mm, float& ll, float& aa) {
    float m_w[NGRP], l_w[NGRP], a_w[NGRP];
    mm = MF_NEG;
#pragma unroll
    for (int w = 0; w < NGRP; ++w) {
      const float* r = s_red + (w * G + g) * (D + 2);
      m_w[w] = r[0]; l_w[w] = r[1]; a_w[w] = r[2 + ch];
      mm = fmaxf(mm, m_w[w]);
    }
    ll = 0.0f; aa = 0.0f;
#pragma unroll
    for (int w = 0; w < NGRP; ++w) {
      const float wgt = __expf(m_w[w] - mm);
      ll = fmaf(wgt, l_w[w], ll);
      aa = fmaf(wgt, a_w[w], aa);
    }
  };
  // A launch that merges its splits itself and has a single split is done here (the kernels whose wavefronts work
  // alone; a path of its own, so that the others' epilogue stays what it was): the walkers' sum, merged with the
  // exact tail's partial if there is one (an earlier launch wrote it: plain loads), is the result - what the merge
  // further down would compute from the same parts in the same order, without the trip through memory and the counting.
  if (DS == 1 && fm.out != nullptr && n_split == 1 && fm.n_extra <= 1) {
#pragma unroll
    for (int k = 0; k < 8 * D / (MF_WAVES * 64); ++k) {
      const int o = tid + k * (MF_WAVES * 64);
      const bool live = o < G * D;
      const int g = live ? o / D : 0, ch = o % D;
      float mm, ll, aa;
      walkers_sum(g, ch, mm, ll, aa);
      if (live && fm.n_extra == 0) {
        const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;
        store_from_f32(fm.out, ((int64_t)b * Hq + qbase + g) * D + ch, aa * inv, fm.out_dtype);
      } else if (live) {
        const float* x = parts + (((int64_t)b * Hq + qbase + g) * n_parts + 1) * (D + 2);     // the exact tail's part
        const float m_x = x[0], l_x = x[1], a_x = x[2 + ch];
        float top = MF_NEG;
        if (ll > 0.0f) top = fmaxf(top, mm);
        if (l_x > 0.0f) top = fmaxf(top, m_x);
        const float w0 = ll > 0.0f ? __expf(mm - top) : 0.0f, w1 = l_x > 0.0f ? __expf(m_x - top) : 0.0f;
        const float l_all = fmaf(w1, l_x, fmaf(w0, ll, 0.0f)), a_all = fmaf(w1, a_x, fmaf(w0, aa, 0.0f));
        const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
        store_from_f32(fm.out, ((int64_t)b * Hq + qbase + g) * D + ch, a_all * inv, fm.out_dtype);
      }
    }
    return;
  }
  // The partial of this workgroup: a thread owns a pair of channels of HPP heads in turn.  All LDS reads of all
  // passes are issued first and all stores last, so the epilogue pays one LDS latency and no wait inside a branch.
  {
    constexpr int PAIRS = D / 2, THREADS = MF_WAVES * 64;
    constexpr int HPP = THREADS / PAIRS, NPASS = (8 + HPP - 1) / HPP;
    const int pr = tid % PAIRS, hsub = tid / PAIRS;
    float m_w[NPASS][NGRP], l_w[NPASS][NGRP];
    f32x2 a_w[NPASS][NGRP];
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int g = min(ps * HPP + hsub, G - 1);
#pragma unroll
      for (int w = 0; w < NGRP; ++w) {
        const float* r = s_red + (w * G + g) * (D + 2);
        const f32x2 ml = *(const f32x2*)r;
        m_w[ps][w] = ml[0]; l_w[ps][w] = ml[1];
        a_w[ps][w] = *(const f32x2*)(r + 2 + 2 * pr);
      }
    }
    f32x2 res[NPASS], ml_out[NPASS];
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      float mm = MF_NEG;
#pragma unroll
      for (int w = 0; w < NGRP; ++w) mm = fmaxf(mm, m_w[ps][w]);
      float ll = 0.0f, a0 = 0.0f, a1 = 0.0f;
#pragma unroll
      for (int w = 0; w < NGRP; ++w) {
        const float wgt = __expf(m_w[ps][w] - mm);
        ll = fmaf(wgt, l_w[ps][w], ll);
        a0 = fmaf(wgt, a_w[ps][w][0], a0);
        a1 = fmaf(wgt, a_w[ps][w][1], a1);
      }
      res[ps] = f32x2{a0, a1};
      ml_out[ps] = f32x2{mm, ll};
    }
    // Write-through (device-coherent) stores in every case.  A merging workgroup of this launch needs them
    // (it reads the partial from another compute die); and with a merge kernel behind, partials that left the
    // L2 as they were produced are not waiting for the write-back at the end of the kernel, which every
    // launch pays before the next one starts (4 x 131072, 64 splits: page kernel 42.6 -> 42.2 us, step -0.45).
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int g = ps * HPP + hsub;
      if (g < G) {
        float* out = parts + (((int64_t)b * Hq + qbase + g) * n_parts + split) * (D + 2);
        store_coherent2(out + 2 + 2 * pr, res[ps]);
        if (pr == 0) store_coherent2(out, ml_out[ps]);
      }
    }
  }
  TQ_STAMP(4);
#ifdef TQ_STAMPS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  TQ_STAMP(5);
#endif
  // ---------------------------------------------------------------- merge of the splits inside this launch
  // Every workgroup counts itself in after its partial has been written (one atomic increment of the group's
  // counter, which the preparation kernel of this step has zeroed); the one that counts last merges.
  if (fm.out != nullptr) {
    __shared__ int s_last;
    // Release: the partial was written with device-coherent (agent-scope, write-through) stores, so there is
    // nothing to write back; what the hand-off needs is that every one of them has been acknowledged before
    // the counter moves.  Each wavefront therefore waits for its own outstanding stores (s_waitcnt vmcnt(0):
    // on this target stores count in vmcnt, and a workgroup-scope fence does not wait for them), the barrier
    // collects all wavefronts, and only then does thread 0 count the workgroup in.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      const unsigned long long before = __hip_atomic_fetch_add(fm.counters + ((int64_t)b * Hkv + h), 1ull, __ATOMIC_RELAXED,
                                                               __HIP_MEMORY_SCOPE_AGENT);
      s_last = before + 1ull == (unsigned long long)n_split;
    }
    __syncthreads();
    if (s_last) {
      // Acquire: the loads below are device-coherent loads issued after the counter's value has come back
      // (s_last depends on it), and every other workgroup's stores were acknowledged before its increment.
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
      for (int k = 0; k < 8 * D / (MF_WAVES * 64); ++k) {
        const int o = tid + k * (MF_WAVES * 64);
        const bool live = o < G * D;
        const int g = live ? o / D : 0, ch = o % D;
        const float* row = parts + ((int64_t)b * Hq + qbase + g) * n_parts * (D + 2);
        // all loads first (clamped to an existing part), then the log-sum-exp merge
        constexpr int NP = MERGE_IN_KERNEL_MAX_SPLITS + 1;
        const int n_merge = n_split + fm.n_extra;
        float m_s[NP], l_s[NP], a_s[NP];
#pragma unroll
        for (int sp = 0; sp < NP; ++sp) {
          const float* r = row + (int64_t)min(sp, n_merge - 1) * (D + 2);
          m_s[sp] = load_coherent(r); l_s[sp] = load_coherent(r + 1); a_s[sp] = load_coherent(r + 2 + ch);
        }
        float mm = MF_NEG;
#pragma unroll
        for (int sp = 0; sp < NP; ++sp)
          if (sp < n_merge && l_s[sp] > 0.0f) mm = fmaxf(mm, m_s[sp]);
        float ll = 0.0f, aa = 0.0f;
#pragma unroll
        for (int sp = 0; sp < NP; ++sp) {
          const float wgt = (sp < n_merge && l_s[sp] > 0.0f) ? __expf(m_s[sp] - mm) : 0.0f;
          ll = fmaf(wgt, l_s[sp], ll);
          aa = fmaf(wgt, a_s[sp], aa);
        }
        const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;
        if (live) store_from_f32(fm.out, ((int64_t)b * Hq + qbase + g) * D + ch, aa * inv, fm.out_dtype);
      }
    }
  }
}

template <int D, int MB, int NX, int VB, int GS, int DS, int WPS, bool F16P, bool PP = false, bool NR = false, bool SG = false,
          int NW = MF_WAVES, int IW = 0>
static int launch_one(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                      const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                      float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts, int n_split,
                      int len_sub, int max_pages, int num_pages, const FusedMerge& fm, bool wide_wg,
                      hipStream_t st) {
  // (heads of the largest group of a KV head; kv_div groups share a KV head's heads, the last one may have fewer)
  const int G = kv_div > 1 ? (Hq / (Hkv / kv_div) + kv_div - 1) / kv_div : Hq / Hkv;
  size_t per_wave = (size_t)wave_lds_floats(D / DS / GS, DS) * sizeof(float);
  size_t merge = (size_t)(NW / DS * (IW > 0 ? 8 : G) * (D + 2) + NW * 16 * 16) * sizeof(float);
  if (SG) per_wave += stage_bytes((D / DS / 16) * VB / 2);
  size_t smem = per_wave * NW > merge ? per_wave * NW : merge;
  // four index planes: the group's packed query operands in LDS, behind the wavefronts' regions
  if (MB >= 4)
    smem = per_wave * NW + (size_t)(MB + NX + 1) * ((D + 127) / 128) * 2 * 64 * 6 * sizeof(uint32_t) + (size_t)64 * 4 * sizeof(float);
  if (MB >= 4 && smem < merge) smem = merge;
  if (D == 64 && !PP && decode_mfma_head_rows(D, G) == 4)
    return launch_one<D, MB, NX, VB, GS, DS, WPS, F16P, D == 64, false, false, MF_WAVES, IW>(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table,
                                                                 bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts,
                                                                 n_split, len_sub, max_pages, num_pages, fm, wide_wg, st);
  if (D >= 128 && !NR && decode_mfma_head_rows(D, G) == 4)
    return launch_one<D, MB, NX, VB, GS, DS, WPS, F16P, false, D >= 128, false, MF_WAVES, IW>(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table,
                                                                         bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts,
                                                                         n_split, len_sub, max_pages, num_pages, fm, wide_wg, st);
  // Three index planes (4-bit keys) at head_dim 128 / 256: always the variant that stages the next block's page data in
  // LDS.  With that data in registers these kernels spill 21 - 98 of them (16 x 8192: 63.3 vs 46.6 us per step), so the
  // register variant is not built; for fewer planes the staged variant measured 2 - 5 % slower and is not built either.
  constexpr bool can_stage = D >= 128 && MB == 3;
  if constexpr (can_stage && !SG) {
    return launch_one<D, MB, NX, VB, GS, DS, WPS, F16P, PP, NR, true, MF_WAVES, IW>(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table,
                                                                      bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts,
                                                                      n_split, len_sub, max_pages, num_pages, fm, wide_wg, st);
  } else {
  // eight wavefronts per workgroup (one workgroup per compute unit) for the kernels whose wavefronts work alone
  // Many short sequences in one split: the fewer wavefronts walk a (sequence, head group), the fewer workgroups the
  // launch has and the more trips follow each prologue; the most wavefronts per pair (4, 2 or 1) with which all of the
  // launch's wavefronts are resident at once (8 per compute unit) wins at every size measured (page kernel, 32 q / 8 KV
  // heads, four / two / one wavefront per pair: 64 x 2048 28.1 / 37.2 / 63.5 us, 96 x 2048 51.9 / 45.6 / 67.0,
  // 128 x 2048 60.4 / 56.0 / 69.7, 128 x 512 21.7 / 18.8 / 22.2, 160 x 1024 46.6 / 48.9 / 44.1, 192 x 1024 51.4 / 52.7 /
  // 47.0, 256 x 1024 66.7 / 61.5 / 58.0); with more pairs than wavefront slots, one.
  constexpr bool can_iw = DS == 1 && MB < 4 && NW == MF_WAVES;
  if constexpr (can_iw && IW == 0) {
    if (n_split == 1 && !wide_wg) {
      int walkers = opt_sequence_walkers.load(std::memory_order_relaxed);
      if (walkers < 0) {
        const int64_t slots = (int64_t)8 * device_compute_units(), items = (int64_t)Hkv * B;
        walkers = slots <= 0 || 4 * items <= slots ? 4 : (2 * items <= slots ? 2 : 1);
      }
      if (walkers == 1)
        return launch_one<D, MB, NX, VB, GS, DS, WPS, F16P, PP, NR, SG, NW, 1>(
            qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts, n_split,
            len_sub, max_pages, num_pages, fm, false, st);
      if (walkers == 2)
        return launch_one<D, MB, NX, VB, GS, DS, WPS, F16P, PP, NR, SG, NW, 2>(
            qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts, n_split,
            len_sub, max_pages, num_pages, fm, false, st);
    }
  }
  constexpr bool can_widen = DS == 1 && NW == MF_WAVES && IW == 0;
  if (can_widen && wide_wg)
    return launch_one<D, MB, NX, VB, GS, DS, WPS, F16P, PP, NR, SG, can_widen ? 2 * MF_WAVES : NW>(
        qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts, n_split,
        len_sub, max_pages, num_pages, fm, false, st);
  // two workgroups of four wavefronts share a compute unit: see the kernel's comment on skew16.  Only the
  // head_dim 256 kernels, which are bound by instruction issue, gain (4 x 131072: 46.4 -> 45.5 us); the head_dim 128
  // kernels wait for memory, their workgroups advance side by side whatever their age, and unequal shares cost
  // what they move (32 x 32768: 203 -> 208 us).
  const int skew16 = NW == MF_WAVES && WPS == 2 && DS == 2 ? decode_mfma_split_skew(n_split, Hkv * B) : 0;
  constexpr int IPW = NW / DS / (IW > 0 ? IW : 1);          // (sequence, head group) pairs of a workgroup with IW > 0
  const dim3 grid = IW > 0 ? dim3(1, (unsigned)(((int64_t)Hkv * B + IPW - 1) / IPW), 1)
                       : (skew16 > 0 ? dim3(n_split / 2, Hkv, 2 * B) : dim3(n_split, Hkv, B));
  auto kern = decode_mfma_kernel<D, MB, NX, VB, GS, DS, WPS, F16P, PP, NR, SG, NW, IW>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return (int)e;
  }
  hipEvent_t t_start_event = nullptr, t_stop_event = nullptr;
  if (take_time_hook(0, t_start_event, t_stop_event)) {
    hipExtLaunchKernelGGL(kern, grid, dim3(NW * 64), smem, st, t_start_event, t_stop_event, 0,
                          qa_pack, q_stat, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts,
                          n_parts, n_split, len_sub, max_pages, num_pages, skew16, B, fm);
  } else {
    kern<<<grid, dim3(NW * 64), smem, st>>>(qa_pack, q_stat, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens,
                                            sm_scale, ly, L, parts, n_parts, n_split, len_sub, max_pages, num_pages, skew16,
                                            B, fm);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TQ_OK : (int)e;
  }
}


// TQ_POOL_F16, defined by a translation unit before it includes this file: 0 = it holds the kernels for bf16 pools only,
// 1 = those for fp16 pools only (head_dim 64 / 128: two units each, so that they compile side by side); else both.
#ifndef TQ_POOL_F16
#define TQ_POOL_F16 -1
#endif
#define TQ_LAUNCH_POOL(F16P_, D_, MB_, NX_, VB_, GS_, DS_, WPS_)                                                \
  if (sh.f16p == F16P_)                                                                                            \
    return launch_one<D_, MB_, NX_, VB_, GS_, DS_, WPS_, F16P_>(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table,     \
                                                                bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts,      \
                                                                n_split, len_sub, max_pages, num_pages, fm, wide_wg, st);
#if TQ_POOL_F16 == 0
#define TQ_LAUNCH_POOLS(...) TQ_LAUNCH_POOL(false, __VA_ARGS__)
#elif TQ_POOL_F16 == 1
#define TQ_LAUNCH_POOLS(...) TQ_LAUNCH_POOL(true, __VA_ARGS__)
#else
#define TQ_LAUNCH_POOLS(...) TQ_LAUNCH_POOL(true, __VA_ARGS__) TQ_LAUNCH_POOL(false, __VA_ARGS__)
#endif
#define TQ_TRY(D_, MB_, NX_, VB_, GS_, DS_, WPS_)                                                               \
  if (sh.d == D_ && sh.mb == MB_ && sh.nx == NX_ && sh.vb == VB_ && sh.gs == GS_) {                                            \
    TQ_LAUNCH_POOLS(D_, MB_, NX_, VB_, GS_, DS_, WPS_)                                                              \
    return TQ_EUNSUPPORTED;                                                                                        \
  }

}  // namespace tq
