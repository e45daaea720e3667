// Streaming-read probe: what the card delivers to a kernel that only reads.  The decode kernels are
// bound by HBM reads, so their bandwidth is reported against this figure next to the vendor peak.
#include "tq_common.h"

namespace tq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Grid-stride 16-byte loads, FLIGHT of them issued per lane before the first is used.  The words are
// folded into one value that is stored only when it equals a constant the data never produces, so the
// loads cannot be dropped and nothing is written.
template <int FLIGHT>
__global__ void __launch_bounds__(256)
stream_read_kernel(const u32x4* __restrict__ p, size_t n, uint32_t* __restrict__ sink) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  uint32_t s = 0;
  for (; i + (FLIGHT - 1) * stride < n; i += FLIGHT * stride) {
    u32x4 v[FLIGHT];
#pragma unroll
    for (int u = 0; u < FLIGHT; ++u) v[u] = p[i + u * stride];
#pragma unroll
    for (int u = 0; u < FLIGHT; ++u) s ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  for (; i < n; i += stride) {
    const u32x4 v = p[i];
    s ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (s == 0x9e3779b9u && sink) sink[0] = s;
}

}  // namespace tq

using namespace tq;

extern "C" int tq_stream_read(const void* src, size_t bytes, int workgroups_per_cu, int loads_in_flight,
                              uint32_t* sink, void* stream) {
  if (!src) return TQ_ENULL;
  if (((uintptr_t)src & 15) || (bytes & 15) || workgroups_per_cu < 1 || workgroups_per_cu > 64) return TQ_EINVAL;
  if (loads_in_flight != 1 && loads_in_flight != 4 && loads_in_flight != 8) return TQ_EINVAL;
  if (bytes == 0) return TQ_OK;
  int dev = 0, n_cu = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  const dim3 grid((unsigned)(n_cu * workgroups_per_cu)), block(256);
  const u32x4* p = (const u32x4*)src;
  const size_t n = bytes / 16;
  hipStream_t st = (hipStream_t)stream;
  if (loads_in_flight == 1) stream_read_kernel<1><<<grid, block, 0, st>>>(p, n, sink);
  else if (loads_in_flight == 4) stream_read_kernel<4><<<grid, block, 0, st>>>(p, n, sink);
  else stream_read_kernel<8><<<grid, block, 0, st>>>(p, n, sink);
  TQ_CHECK_LAUNCH();
  return TQ_OK;
}
