// Interface between the host side of the decode path (tq_decode.hip) and the matrix-core page kernel
// (tq_decode_mfma.hip).
#pragma once

#include "tq_common.h"

namespace tq {

// Query preparation as a prologue of the page kernel's own launch (q == nullptr: the operands in
// qa_pack / q_stat were prepared by an earlier launch).
struct FusedPrep {
  const void* q = nullptr;           // (B, Hq, d) raw queries
  int q_dtype = 0;
  int n_units = 0;                   // units per group of query heads (<= 64): (8 / hp) head sets x d / 32 plane words
  int hp = 8;                        // heads per unit: 1, 2, 4 or 8
  int spin_limit = 0;                // polls before a workgroup stops waiting for the others' units
  unsigned long long* flags = nullptr;   // 64 words per group
  unsigned long long nonce = 0;      // value of a published flag in this call (never 0)
};

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

// Events armed by tq_time_next_page_kernel (which = 0) / tq_time_next_key_kernel (which = 1) on this thread:
// returns them and disarms; false when none is armed.
bool take_time_hook(int which, hipEvent_t& start, hipEvent_t& stop);

// whether the library was built with the in-launch preparation (-DTQ_FUSED_PREP)
bool decode_mfma_has_fused_prep();

// words of packed query operands tq_decode_workspace_bytes reserves
size_t decode_mfma_pack_words(int B, int Hq, int d);

// Returns TQ_EUNSUPPORTED when the shape has no matrix-core kernel (nothing was launched); the caller then
// uses the general vector-ALU kernel.
int launch_decode_mfma(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div, const uint8_t* pool,
                       const int32_t* block_table, int bt_stride, const int32_t* seq_lens, float sm_scale,
                       const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts, int n_split, int len_sub,
                       int max_pages, int num_pages, const FusedPrep& fz, const FusedMerge& fm, bool wide_wg,
                       hipStream_t st);

// Whether a step of this shape runs workgroups of eight wavefronts: the caller then passes HALF its split count
// (and wide_wg = true) to launch_decode_mfma and uses that count for everything that follows.
bool decode_mfma_wide_workgroups(int d, int G, int n_split, int max_pages);

// Sixteenths of a split that every even split takes over from its odd neighbour (0: equal shares), for a launch of
// n_split x rows workgroups of four wavefronts that sit two to a compute unit.
int decode_mfma_split_skew(int n_split, int rows);

// Compute units of the device (looked up once); 0 if unknown.
int device_compute_units();

}  // namespace tq
