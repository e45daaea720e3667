// Shared device helpers for the TurboQuant gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tq_hip.h"

#define TQ_WAVE 64

#define TQ_CHECK_LAUNCH()                         \
  do {                                            \
    hipError_t e__ = hipGetLastError();           \
    if (e__ != hipSuccess) return (int)e__;       \
  } while (0)

namespace tq {

// ---- 16-bit float <-> fp32, bit-level so that the rounding is explicit --------------

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// round-to-nearest-even, NaN kept quiet: the rounding torch applies when an op
// on bf16 tensors is computed in fp32 and stored back.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;  // v_cvt_f16_f32: round-to-nearest-even
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

// DT is one of the TQ_F32 / TQ_F16 / TQ_BF16 tags.
template <int DT>
struct Elem;
template <>
struct Elem<TQ_F32> {
  using storage = float;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <>
struct Elem<TQ_F16> {
  using storage = uint16_t;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return f16_bits_to_f32(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = f32_to_f16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }
};
template <>
struct Elem<TQ_BF16> {
  using storage = uint16_t;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return bf16_bits_to_f32(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
};

__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dt) {
  if (dt == TQ_F32) return ((const float*)p)[i];
  uint16_t b = ((const uint16_t*)p)[i];
  return dt == TQ_F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
}

__device__ __forceinline__ void store_from_f32(void* p, int64_t i, float v, int dt) {
  if (dt == TQ_F32) ((float*)p)[i] = v;
  else ((uint16_t*)p)[i] = dt == TQ_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
}

// ---- wave reductions ---------------------------------------------------------------

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// The same reductions with DPP row operations and four lane reads instead of shared-memory permutes (no LDS
// round trip per step).  The sum adds in a different order than wave_sum.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// sum / maximum over groups of 4, 8 or 16 neighbouring lanes (quad swaps, half-row mirror, row mirror); every
// lane of a group ends with the group's result
template <int N>
__device__ __forceinline__ float lanes_sum_dpp(float v) {
  static_assert(N == 4 || N == 8 || N == 16, "4, 8 or 16 lanes");
  v += dpp_f32<0xB1>(v);
  v += dpp_f32<0x4E>(v);
  if (N >= 8) v += dpp_f32<0x141>(v);
  if (N >= 16) v += dpp_f32<0x140>(v);
  return v;
}
template <int N>
__device__ __forceinline__ float lanes_max_dpp(float v) {
  static_assert(N == 4 || N == 8 || N == 16, "4, 8 or 16 lanes");
  v = fmaxf(v, dpp_f32<0xB1>(v));
  v = fmaxf(v, dpp_f32<0x4E>(v));
  if (N >= 8) v = fmaxf(v, dpp_f32<0x141>(v));
  if (N >= 16) v = fmaxf(v, dpp_f32<0x140>(v));
  return v;
}
__device__ __forceinline__ float wave_sum_fast(float v) {
  const int b = __builtin_bit_cast(int, lanes_sum_dpp<16>(v));
  return (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16))) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48)));
}
__device__ __forceinline__ float wave_max_fast(float v) {
  const int b = __builtin_bit_cast(int, lanes_max_dpp<16>(v));
  return fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16))),
               fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48))));
}

// ---- index packing of the reference's flat layout (quantizer.py:38-69) --------------

__host__ __device__ __forceinline__ int eff_bits(int mse_bits) { return mse_bits == 1 ? 1 : (mse_bits == 2 ? 2 : (mse_bits <= 4 ? 4 : 8)); }
__host__ __device__ __forceinline__ int idx_row_bytes(int d, int mse_bits) {
  int per = 8 / eff_bits(mse_bits);
  return (d + per - 1) / per;
}

// ---- page geometry -----------------------------------------------------------------

// byte offset of word j (coordinates 32j..32j+31) of plane p of token n
__host__ __device__ __forceinline__ int key_word_off(const tq_page_layout& L, int p, int j, int n) {
  const int W = L.d >> 5, planes = L.mse_bits + 1;
  // (head_dim 64 has two words per plane: [j][n][p])
  if (L.key_lane_major)
    return L.off_keys + (((((j & 3) * TQ_PAGE_TOKENS + n) * (W >= 4 ? W >> 2 : 1)) + (j >> 2)) * planes + p) * 4;
  return L.off_keys + ((p * W + j) * TQ_PAGE_TOKENS + n) * 4;
}

// byte offset of the value field (16 * value_bits bits) of channel c
__host__ __device__ __forceinline__ int vfield_off(const tq_page_layout& L, int c) {
  return L.off_vdata + (((c & 15) * (L.d >> 4)) + (c >> 4)) * (L.value_bits * 2);
}

__host__ __device__ __forceinline__ int elem_bytes(int dtype) { return dtype == TQ_F32 ? 4 : 2; }

}  // namespace tq
