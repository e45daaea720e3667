// Instantiations of the matrix-core page kernel for head_dim 128, fp16 pools (see tq_decode_mfma_impl.h).

#define TQ_POOL_F16 1
#include "tq_decode_mfma_impl.h"

namespace tq {

int launch_decode_mfma_d128_f16(uint32_t* qa_pack, float* q_stat, int B, int Hq, int Hkv, int kv_div,
                       const uint8_t* pool, const int32_t* block_table, int bt_stride, const int32_t* seq_lens,
                       float sm_scale, const tq_layer& ly, const tq_page_layout& L, float* parts, int n_parts,
                       int n_split, int len_sub, int max_pages, int num_pages, const FusedMerge& fm,
                       bool wide_wg, hipStream_t st) {
  const MfmaShape sh = mfma_shape_of(ly, L);
  TQ_MFMA_SHAPES_D128(TQ_TRY)
  return TQ_EUNSUPPORTED;
}

}  // namespace tq

