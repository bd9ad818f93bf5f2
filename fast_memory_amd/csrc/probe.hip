// Plain streaming copy of a known size: the yardstick that HBM traffic counters
// of the other kernels are scaled against when profiling.
#include "common.hpp"

namespace fm {
__global__ __launch_bounds__(256) void copy_probe_kernel(const uint4* __restrict__ src,
                                                         uint4* __restrict__ dst, int64_t n) {
  int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (; i < n; i += stride) dst[i] = src[i];
}
}  // namespace fm

extern "C" int fm_debug_copy(void* dst, const void* src, int64_t nbytes, void* stream) {
  using namespace fm;
  FM_REQUIRE(dst && src && nbytes >= 0 && nbytes % 16 == 0, FM_ERR_ARG, "fm_debug_copy: nbytes=%lld",
             (long long)nbytes);
  if (nbytes == 0) return FM_OK;
  hipLaunchKernelGGL(copy_probe_kernel, dim3(4096), dim3(256), 0, as_stream(stream),
                     (const uint4*)src, (uint4*)dst, nbytes / 16);
  return launch_status("fm_debug_copy");
}
