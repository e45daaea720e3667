// Matrix-core page kernel: what is not a template - the dispatch over head sizes, the choice of the workgroup
// size, the timing hooks.  The kernel itself is in tq_decode_mfma_impl.h, instantiated by one translation unit per
// head size so that they compile side by side.

#include <hip/hip_ext.h>

#include <atomic>

#include "tq_common.h"
#include "tq_prep.h"
#include "tq_decode_mfma.h"
#include "tq_options.h"

namespace tq {

constexpr int MF_WAVES = 4;              // wavefronts of the (smaller) workgroup, as in tq_decode_mfma_impl.h
constexpr int BLK_TOK = 64;              // tokens per wavefront iteration

// events the next launch of this thread attaches to its dispatch (see tq_time_next_page_kernel /
// tq_time_next_key_kernel): [0] the page kernel of the decode path, [1] the paged key-quantise kernel
static thread_local hipEvent_t t_hook_events[2][2] = {{nullptr, nullptr}, {nullptr, nullptr}};

bool take_time_hook(int which, hipEvent_t& start, hipEvent_t& stop) {
  start = t_hook_events[which][0];
  stop = t_hook_events[which][1];
  t_hook_events[which][0] = t_hook_events[which][1] = nullptr;
  return start != nullptr || stop != nullptr;
}

// Whether a step of this shape should run workgroups of eight wavefronts (the caller then halves its split
// count: the launch keeps its number of wavefronts).  Taken when a wavefront would walk at most 16 blocks of
// the longest sequence the block table can hold: 16 x 8192 tokens at 32 q / 8 KV heads 39.7 -> 38.2 us per
// step, at 64 q / 8 KV heads 42.9 -> 40.5 us, but 32 x 32768 (64 blocks per wavefront) 212 -> 216 us.
bool decode_mfma_wide_workgroups(int d, int G, int n_split, int max_pages) {
  if (!(d == 64 || d == 128) || G > 8 || n_split < 2 || (n_split & 1)) return false;
  if (opt_wide_workgroups.load(std::memory_order_relaxed) == 0) return false;
  const int64_t blocks = ((int64_t)max_pages * TQ_PAGE_TOKENS + BLK_TOK - 1) / BLK_TOK;
  return blocks <= (int64_t)16 * MF_WAVES * n_split;
}

// Compute units of the device that is current at the first call (the cards of one machine are alike); 0 if unknown.
// compute units of the current device (looked up once per device)
int device_compute_units() {
  static std::atomic<int> units[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  const bool cached = dev >= 0 && dev < 64;
  int n = cached ? units[dev].load(std::memory_order_relaxed) : 0;
  if (n <= 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    if (cached && n > 0) units[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Unequal shares for the two workgroups of a compute unit.  Workgroups are dispatched in grid order and spread
// over the compute units, so when the launch fills (nearly) every compute unit twice, the first half of the grid
// holds the older workgroup of every unit; a SIMD serves its older wavefronts first, and with equal shares those
// finish about a tenth of the kernel's time before the younger ones.  4 x 131072 tokens, 16 q / 2 KV heads,
// head_dim 256 (512 workgroups of 16 trips): one trip moved.  If the dispatch order were another one the shares
// would merely be as unequal as they are unlucky: results do not depend on it.
int decode_mfma_split_skew(int n_split, int rows) {
  const int skew = opt_split_skew.load(std::memory_order_relaxed);
  if (skew <= 0 || n_split < 2 || (n_split & 1)) return 0;
  const int units = device_compute_units();
  const int64_t groups = (int64_t)n_split * rows;
  return units > 0 && groups <= 2 * (int64_t)units && groups * 16 >= 30 * (int64_t)units ? skew : 0;
}

void decode_mfma_plan(PagePrefetch& pf, int d, int B, int groups, int kv_div, int n_split, bool wide_wg) {
  const int ds = d == 256 ? 2 : 1, nw = wide_wg ? 2 * MF_WAVES : MF_WAVES;
  pf.n_split = n_split; pf.groups = groups; pf.kv_div = kv_div; pf.n_seq = B;
  pf.ngrp = nw / ds;
  pf.skew16 = !wide_wg && ds == 2 ? decode_mfma_split_skew(n_split, groups * B) : 0;
  pf.gx = pf.skew16 > 0 ? n_split / 2 : n_split;
  pf.n_wg = n_split * groups * B;
}

// words of packed query operands tq_decode_attn_paged reserves in its workspace
size_t decode_mfma_pack_words(int B, int Hq, int d) { return (size_t)B * Hq * 9 * (d / 128 + 1) * 1024; }   // d = 64: one chunk

bool decode_mfma_has_kernel(const tq_layer& ly, const tq_page_layout& L) {
  if ((L.dtype != TQ_BF16 && L.dtype != TQ_F16) || !L.key_lane_major) return false;
  const MfmaShape sh = mfma_shape_of(ly, L);
#define TQ_HAS(D_, MB_, NX_, VB_, GS_, DS_, WPS_) \
  if (sh.d == D_ && sh.mb == MB_ && sh.nx == NX_ && sh.vb == VB_ && sh.gs == GS_) return true;
  TQ_MFMA_SHAPES_D64(TQ_HAS) TQ_MFMA_SHAPES_D128(TQ_HAS) TQ_MFMA_SHAPES_D256(TQ_HAS)
#undef TQ_HAS
  return false;
}

// the launchers of the three head sizes (tq_decode_mfma_d64 / _d128 / _d256.hip; head_dim 64 / 128: bf16 and fp16
// pools in units of their own, _f16)
int launch_decode_mfma_d64(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, int len_sub, int max_pages, int num_pages, const FusedMerge& fm,
                       bool wide_wg, hipStream_t st);
int launch_decode_mfma_d128(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, int len_sub, int max_pages, int num_pages, const FusedMerge& fm,
                       bool wide_wg, hipStream_t st);
int launch_decode_mfma_d64_f16(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, int len_sub, int max_pages, int num_pages, const FusedMerge& fm,
                       bool wide_wg, hipStream_t st);
int launch_decode_mfma_d128_f16(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, int len_sub, int max_pages, int num_pages, const FusedMerge& fm,
                       bool wide_wg, hipStream_t st);
int launch_decode_mfma_d256(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, int len_sub, int max_pages, int num_pages, const FusedMerge& fm,
                       bool wide_wg, hipStream_t st);

// Returns TQ_EUNSUPPORTED when the shape has no matrix-core kernel; the caller then
// uses the general vector-ALU kernel.
int launch_decode_mfma(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, int len_sub, int max_pages, int num_pages, const FusedMerge& fm,
                       bool wide_wg, hipStream_t st) {
  const int G = kv_div > 1 ? (Hq / (Hkv / kv_div) + kv_div - 1) / kv_div : Hq / Hkv, d = ly.d;
  if (G > 8 || (L.dtype != TQ_BF16 && L.dtype != TQ_F16) || !L.key_lane_major) return TQ_EUNSUPPORTED;
  if (d == 64 && L.dtype == TQ_F16)
    return launch_decode_mfma_d64_f16(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts,
                                      n_split, len_sub, max_pages, num_pages, fm, wide_wg, st);
  if (d == 64) return launch_decode_mfma_d64(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts, n_split,
                                   len_sub, max_pages, num_pages, fm, wide_wg, st);
  if (d == 128 && L.dtype == TQ_F16)
    return launch_decode_mfma_d128_f16(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts,
                                       n_split, len_sub, max_pages, num_pages, fm, wide_wg, st);
  if (d == 128) return launch_decode_mfma_d128(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts, n_split,
                                   len_sub, max_pages, num_pages, fm, wide_wg, st);
  if (d == 256) return launch_decode_mfma_d256(qa_pack, q_stat, B, Hq, Hkv, kv_div, pool, block_table, bt_stride, seq_lens, sm_scale, ly, L, parts, n_parts, n_split,
                                   len_sub, max_pages, num_pages, fm, wide_wg, st);
  return TQ_EUNSUPPORTED;
}

}  // namespace tq

extern "C" void tq_time_next_page_kernel(void* start_event, void* stop_event) {
  tq::t_hook_events[0][0] = (hipEvent_t)start_event;
  tq::t_hook_events[0][1] = (hipEvent_t)stop_event;
}

extern "C" void tq_time_next_key_kernel(void* start_event, void* stop_event) {
  tq::t_hook_events[1][0] = (hipEvent_t)start_event;
  tq::t_hook_events[1][1] = (hipEvent_t)stop_event;
}
