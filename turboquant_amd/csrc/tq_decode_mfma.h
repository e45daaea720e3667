// Interface between the host side of the decode path (tq_decode.hip) and the matrix-core page kernel
// (tq_decode_mfma.hip).
#pragma once

#include "tq_common.h"
#include "tq_options.h"

namespace tq {

// Merge of the context splits inside the page kernel's launch (out == nullptr: a merge kernel follows).  The
// workgroup that finishes last among the n_split workgroups of a (sequence, group of query heads) reads the
// others' partials and writes the attention output; nobody waits for anybody.  `counters` holds one arrival
// counter per group, zeroed by the query preparation kernel of the same step.
struct FusedMerge {
  void* out = nullptr;               // (B, Hq, d) in out_dtype
  int out_dtype = 0;
  unsigned long long* counters = nullptr;
  int n_extra = 0;                   // parts after the n_split splits that an earlier launch has written (the exact tail)
};
constexpr int MERGE_IN_KERNEL_MAX_SPLITS = 8;

// Operand rows (query heads) of a group that the page kernel reads from the packed query operands: with at most four
// heads per group the kernels that take them (two pages per score instruction at head_dim 64, one operand per plane
// word at head_dim 128 / 256) only touch the rows of heads 0..3, so the preparation need not write zeros into the rest.
inline int decode_mfma_head_rows(int d, int G) {
  const bool four = G <= 4 && (d == 64 ? opt_page_pairs.load(std::memory_order_relaxed) != 0
                                       : opt_narrow_rows.load(std::memory_order_relaxed) != 0);
  return four ? 4 : 8;
}

// The blocks (64 tokens) a page-kernel workgroup walks: split `split` of n_split over a sequence of seq_len
// compressed tokens.  skew16 > 0 (head_dim 256, two workgroups per compute unit): every even split takes skew16
// sixteenths of a split's trips over from its odd neighbour; ngrp = block walkers of a workgroup.  The page kernel
// and the page prefetch of the preparation launch both call this, so they agree on who reads what.
__host__ __device__ inline void decode_block_range(int seq_len, int n_split, int split, int skew16, int ngrp,
                                                   int& blk_begin, int& blk_end) {
  const int n_blocks = (seq_len + 63) / 64;
  const int per_split = (n_blocks + n_split - 1) / n_split;
  blk_begin = split * per_split;
  blk_end = blk_begin + per_split < n_blocks ? blk_begin + per_split : n_blocks;
  if (skew16 > 0) {
    int moved = ngrp * ((((per_split + ngrp - 1) / ngrp) * skew16 + 8) >> 4);
    moved = moved < per_split ? moved : per_split;
    if (split & 1) blk_begin = blk_begin + moved < blk_end ? blk_begin + moved : blk_end;
    else blk_end = blk_end + moved < n_blocks ? blk_end + moved : n_blocks;
  }
}

// Page prefetch inside the preparation launch of a decode step.  The preparation is a short, latency-bound
// launch that leaves most compute units and the whole memory system idle; workgroups added to its grid read
// the pages that every page-kernel workgroup will ask for first (the first `blocks` blocks of its range), so
// that they sit in the cache hierarchy (the die's L2 when the reader shares the die, the memory-side cache
// otherwise) when the page kernel starts.  Nothing depends on it: with blocks = 0 the step is the same minus
// the head start.  The fields mirror the page kernel's launch (launch_one) so that the same ranges come out.
struct PagePrefetch {
  const uint8_t* pool = nullptr;
  const int32_t* block_table = nullptr;
  const int32_t* seq_lens = nullptr;
  int bt_stride = 0, max_pages = 0, num_pages = 0, len_sub = 0;
  int n_split = 0, groups = 0, kv_div = 1, n_seq = 0, skew16 = 0, ngrp = 1;
  int gx = 1;                        // x extent of the page kernel's grid (n_split, or n_split / 2 with a skew)
  uint32_t page_bytes = 0, page_stride = 0;
  uint32_t fetch_bytes = 0;          // leading bytes of a page that are read ahead (a multiple of 16, <= page_bytes)
  int blocks = 0;                    // blocks to read per page-kernel workgroup (0: no prefetch workgroups)
  int n_wg = 0;                      // page-kernel workgroups = prefetch workgroups
  int front = 0;                     // workgroups of this launch in front of the prefetch ones
};

// Shape of the page kernel's launch for a step (what launch_one will decide), for the prefetch: fills n_split,
// groups, kv_div, n_seq, skew16, ngrp, gx, n_wg.
void decode_mfma_plan(PagePrefetch& pf, int d, int B, int groups, int kv_div, int n_split, bool wide_wg);

// Events armed by tq_time_next_page_kernel (which = 0) / tq_time_next_key_kernel (which = 1) on this thread:
// returns them and disarms; false when none is armed.
bool take_time_hook(int which, hipEvent_t& start, hipEvent_t& stop);

// words of packed query operands tq_decode_workspace_bytes reserves
size_t decode_mfma_pack_words(int B, int Hq, int d);

// The instantiations of the matrix-core page kernel, one list per head size: X(head_dim, index bits, multi-bit
// Walsh terms, value bits, value group size, wavefronts per block, wavefronts per SIMD).  The launchers and the
// host-side predicate below both expand these lists, so they cannot disagree.
#define TQ_MFMA_SHAPES_D64(X) \
  X(64, 2, 0, 2, 32, 1, 2) X(64, 2, 0, 4, 32, 1, 2) X(64, 1, 0, 2, 32, 1, 2) X(64, 1, 0, 4, 32, 1, 2) \
  X(64, 3, 1, 2, 32, 1, 2) X(64, 3, 1, 4, 32, 1, 2) X(64, 2, 0, 8, 32, 1, 2)
#define TQ_MFMA_SHAPES_D128(X) \
  X(128, 2, 0, 2, 32, 1, 2) X(128, 2, 0, 4, 32, 1, 2) X(128, 1, 0, 2, 32, 1, 2) X(128, 1, 0, 4, 32, 1, 2) \
  X(128, 3, 1, 2, 32, 1, 2) X(128, 3, 1, 4, 32, 1, 2) X(128, 2, 0, 2, 64, 1, 2) X(128, 2, 0, 4, 64, 1, 2) \
  X(128, 2, 0, 8, 32, 1, 2) X(128, 4, 4, 4, 32, 1, 2) X(128, 4, 4, 2, 32, 1, 2)
#define TQ_MFMA_SHAPES_D256(X) \
  X(256, 2, 0, 2, 32, 2, 2) X(256, 2, 0, 4, 32, 2, 2) X(256, 1, 0, 2, 32, 2, 2) X(256, 1, 0, 4, 32, 2, 2) \
  X(256, 3, 1, 2, 32, 2, 2) X(256, 3, 1, 4, 32, 2, 2) X(256, 2, 0, 2, 64, 2, 2) X(256, 2, 0, 4, 64, 2, 2) \
  X(256, 2, 0, 8, 32, 2, 2)

// the parameters of a layer that pick an instantiation
struct MfmaShape { int d, mb, nx, vb, gs; bool f16p; };
inline MfmaShape mfma_shape_of(const tq_layer& ly, const tq_page_layout& L) {
  MfmaShape s{ly.d, ly.mse_bits, 0, L.value_bits, L.group_size, L.dtype == TQ_F16};
  for (int t = 0; t < ly.n_terms; ++t)
    if (__builtin_popcount(ly.term_mask[t]) > 1) ++s.nx;
  return s;
}

// Whether launch_decode_mfma has a kernel for this layer and page layout (head size, bit widths, codebook terms,
// group size, page dtype and key order); the host side decides the step's shape - split count, operand packing,
// workspace carving - from this, before anything is launched.
bool decode_mfma_has_kernel(const tq_layer& ly, const tq_page_layout& L);

// Returns TQ_EUNSUPPORTED when the shape has no matrix-core kernel (nothing was launched); the caller then
// uses the general vector-ALU kernel.
int launch_decode_mfma(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div, const uint8_t* pool,
                       const int32_t* block_table, int bt_stride, const int32_t* seq_lens, float sm_scale,
                       const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts, int n_split, int len_sub,
                       int max_pages, int num_pages, const FusedMerge& fm, bool wide_wg,
                       hipStream_t st);

// Packed query operands of the wide-head kernel (head sizes 320 .. 704), written by the rotation launch of the step
// and read by every page-kernel workgroup of the group: per group of at most 8 query heads of a KV head
// [term plane][row set][chunk] operands of WD_QA_OP dwords ([64 lanes][4] then [64 lanes][2]); a last chunk of 64
// coordinates takes half an operand ([32][4] then [32][2]).  q_stat per query row: {E_index, E_sign, constant part of the
// index score, of the sign score}.
constexpr int WD_QA_OP = 64 * 6;
__host__ __device__ constexpr int wide_qa_stride(int d) { return ((d + 127) / 128) * WD_QA_OP - (d % 128 ? WD_QA_OP / 2 : 0); }   // dwords per (plane, row set)
struct WidePack {
  uint32_t* qa = nullptr;            // nullptr: the page kernel packs its operands itself
  float* q_stat = nullptr;
  int Hq = 0, Hkv = 0, kv_div = 1, ntp = 0;
  float sm_scale = 0.0f;
};

// The matrix-core kernel for head sizes above 256 (tq_decode_wide.hip; a workgroup per block of 32 tokens): reads the
// fp32 rotated / sketched queries the general kernel reads and writes the same partials.  TQ_EUNSUPPORTED when the
// shape has no such kernel (nothing was launched).
bool decode_wide_has_kernel(const tq_layer& ly, const tq_page_layout& L);
int launch_decode_wide(const float* q_rot, const float* q_sk, int B, int Hq, int Hkv, const uint8_t* pool,
                       const int32_t* block_table, int bt_stride, const int32_t* seq_lens, float sm_scale,
                       const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts, int n_split, int len_sub,
                       int max_pages, int num_pages, const WidePack& pre, hipStream_t st);
// term planes of a layer on that kernel (0: its codebook has other Walsh terms than the kernel takes)
int decode_wide_term_planes(const tq_layer& ly);

// Whether a step of this shape runs workgroups of eight wavefronts: the caller then passes HALF its split count
// (and wide_wg = true) to launch_decode_mfma and uses that count for everything that follows.
bool decode_mfma_wide_workgroups(int d, int G, int n_split, int max_pages);

// Sixteenths of a split that every even split takes over from its odd neighbour (0: equal shares), for a launch of
// n_split x rows workgroups of four wavefronts that sit two to a compute unit.
int decode_mfma_split_skew(int n_split, int rows);

// Compute units of the device (looked up once); 0 if unknown.
int device_compute_units();

}  // namespace tq
