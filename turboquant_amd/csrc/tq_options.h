// Process-wide knobs set through tq_set_option (defined in tq_decode.hip).
#pragma once

#include <atomic>

namespace tq {
extern std::atomic<int> opt_append_parts;      // measurement: 3 keys and values (the product), 1 keys only, 2 values only
extern std::atomic<int> opt_fp6_centroids;     // key quantiser, head_dim 128: centroid contraction on the fp6 x fp4 MFMA
extern std::atomic<int> opt_page_pairs;        // decode, head_dim 64 with at most 4 query heads per KV head: one score MFMA per two pages
extern std::atomic<int> opt_narrow_rows;       // decode, head_dim 128 / 256 with at most 4 query heads per KV head: one score MFMA per plane word
extern std::atomic<int> opt_wide_workgroups;   // decode, head_dim 64 / 128, short contexts: workgroups of 8 wavefronts
extern std::atomic<int> opt_split_skew;        // decode, two workgroups per compute unit: sixteenths of a split moved to the workgroup dispatched first (0: none)
extern std::atomic<int> opt_tail_chunks;        // hybrid decode with many splits: up to 4 workgroups share the exact tokens of a head group
extern std::atomic<int> opt_merge_row_groups;  // merge kernel: with few rows, several workgroups share a row's channels
extern std::atomic<int> opt_prefetch_trips;     // decode: trips of every block walker whose pages the preparation launch reads ahead (0: none, -1: one at head_dim 256)
extern std::atomic<int> opt_prep_mfma;           // decode: bf16 queries at head_dim 128 / 256 are prepared on the matrix cores
extern std::atomic<int> opt_sequence_walkers;     // decode, one split, head_dim 64 / 128: wavefronts that walk a (sequence, head group): 4, 2, 1, or -1 = as many of those as keep the whole launch resident
extern std::atomic<int> opt_prep_words;           // decode, matrix-core preparation: a workgroup per tile of query rows, a plane word per wavefront (1), a workgroup per (tile, word) (0), -1: the first when the second would not be resident at once
extern std::atomic<int> opt_append_small;         // key quantiser into pages: up to this many 16-vector tiles get a workgroup each that computes one tile (0: never, -1: two per compute unit)
extern std::atomic<int> opt_wide_prepack;          // decode, wide-head kernel: the rotation launch packs the query operands (0: every page-kernel workgroup its own)
extern std::atomic<int> opt_wide_heads;             // decode: head sizes above 256 run the workgroup-per-block matrix-core kernel (0: the general kernel)
extern std::atomic<int> opt_merge_in_kernel;    // decode: few context splits are merged by the last workgroup of the page kernel
}  // namespace tq
