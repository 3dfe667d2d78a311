// A plain device-to-device copy kernel, exported as a measurement aid: the yardstick
// that the transform kernels' time per launch is held against (same bytes, no
// arithmetic).  Each wave moves 16 KB: sixteen 16-byte loads per lane, all issued
// before the first store, loads and stores with the nontemporal hint - the fastest of
// the shapes tried for a 66 MiB copy whose operands come from HBM (24.9-25.0 us; the
// same with plain loads 26.1-26.5 us, one 16-byte word per lane 25.6-26.0 us, 4 per lane
// 27.8-28.3, 32 per lane 30.7-31.3, the runtime's own copy 28.0 us).  (For the
// transforms themselves the hint pays on the stores only: on their loads it costs 5 %.)
#include "common.h"

namespace fbfft_amd {
namespace {

constexpr int kCopyWords = 16;  // 16-byte words per lane

__global__ __launch_bounds__(64) void benchCopyKernel(const vfloat4* __restrict__ src,
                                                      vfloat4* __restrict__ dst, long words) {
  const long base = (long)blockIdx.x * 64 * kCopyWords + threadIdx.x;
  vfloat4 r[kCopyWords];
#pragma unroll
  for (int u = 0; u < kCopyWords; ++u) {
    const long i = base + 64 * u;
    if (i < words) r[u] = __builtin_nontemporal_load(src + i);
  }
#pragma unroll
  for (int u = 0; u < kCopyWords; ++u) {
    const long i = base + 64 * u;
    if (i < words) __builtin_nontemporal_store(r[u], dst + i);
  }
}

}  // namespace
}  // namespace fbfft_amd

extern "C" int fbfft_bench_copy(const void* src, void* dst, size_t bytes, hipStream_t stream) {
  using namespace fbfft_amd;
  if (bytes == 0) return FBFFT_SUCCESS;
  if (!src || !dst || bytes % 16 != 0 || !aligned(src, 16) || !aligned(dst, 16))
    return FBFFT_UNSUPPORTED_DIMENSION;
  const long words = (long)(bytes / 16);
  const long perGroup = 64L * kCopyWords;
  const long groups = (words + perGroup - 1) / perGroup;
  if (groups > 0x7fffffffL) return FBFFT_UNSUPPORTED_SIZE;
  benchCopyKernel<<<dim3((unsigned)groups), dim3(64), 0, stream>>>(
      static_cast<const vfloat4*>(src), static_cast<vfloat4*>(dst), words);
  return launchStatus();
}
