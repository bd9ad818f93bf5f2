// Kernels of known size: a plain streaming copy (the yardstick that HBM traffic counters of the other
// kernels are scaled against when profiling), a read-only stream and a register-resident MFMA stream (the
// rates a kernel can actually reach on the device, beside the published peaks).
#include "common.hpp"
#include "mfma_tile.hpp"

namespace fm {
__global__ __launch_bounds__(256) void copy_probe_kernel(const uint4* __restrict__ src,
                                                         uint4* __restrict__ dst, int64_t n) {
  int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (; i < n; i += stride) dst[i] = src[i];
}

// Read-only stream: eight 16-byte loads in flight per thread, results folded into a word that is
// written only if it takes an impossible value.  Its rate is the read bandwidth a kernel can
// actually reach on the device, the practical ceiling beside the published peak.
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ src, int64_t n,
                                                         uint32_t* __restrict__ sink) {
  constexpr int U = 8;
  int64_t i = int64_t(blockIdx.x) * 256 * U + threadIdx.x;
  const int64_t stride = int64_t(gridDim.x) * 256 * U;
  uint32_t acc = 0;
  for (; i + 256 * (U - 1) < n; i += stride) {
    uint4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = src[i + u * 256];
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= x[u].x ^ x[u].y ^ x[u].z ^ x[u].w;
  }
  if (acc == 0x9e3779b9u && n < 0) sink[0] = acc;
}

// Gather of 256-byte rows from a region small enough to stay in the last-level cache and much larger than an
// XCD's L2: sixteen lanes read one row with one 16-byte load each (the shape of the attention kernels' row
// fetches), eight rows in flight per group of sixteen lanes.  The rows of a pass are a permutation of the
// region (an odd multiplier modulo a power of two), so no row is read twice in a pass, and the groups move on by
// 17 places from pass to pass, so the next reader of a row sits behind another L2.  Nothing is written.  From
// the second pass on every byte comes out of the last-level cache through the fabric into an L2: the rate is
// what that path sustains for scattered rows.  With a region that every L2 holds (1 or 2 MiB) the same loads
// are answered by the L2s: the rate of the path L2 -> compute unit for scattered rows.
__global__ __launch_bounds__(256) void gather_probe_kernel(const uint4* __restrict__ src, uint32_t region_rows,
                                                           int passes, uint32_t* __restrict__ sink) {
  constexpr int U = 8;
  const uint32_t n_grp = gridDim.x * 16u, lane16 = threadIdx.x & 15u;
  const uint32_t grp0 = blockIdx.x * 16u + (threadIdx.x >> 4);
  uint32_t acc = 0;
  for (int pass = 0; pass < passes; ++pass) {
    const uint32_t grp = (grp0 + uint32_t(pass) * 17u) % n_grp;
    // (a region of fewer rows than a sweep of the grid, 2^17, is read 2^17 / region_rows times per pass)
    const uint32_t sweep_rows = max(region_rows, U * n_grp);
    for (uint32_t r = grp; r + (U - 1) * n_grp < sweep_rows; r += U * n_grp) {
      uint4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t row = ((r + u * n_grp) * 0x9E3779B1u) & (region_rows - 1u);
        x[u] = src[size_t(row) * 16u + lane16];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) acc ^= x[u].x ^ x[u].y ^ x[u].z ^ x[u].w;
    }
  }
  if (acc == 0x9e3779b9u && passes < 0) sink[0] = acc;
}

// Register-resident stream of bf16 MFMAs: every wave loads ten operand fragments once and then issues nothing
// but v_mfma_f32_32x32x16_bf16, four independent accumulator chains in turn (with fewer, the next instruction
// of a chain waits for the one before it).  No memory, LDS or VALU work inside the loop: its rate is what the
// matrix pipes sustain on this device for the operand values given -- the device is power-bound in such a loop
// and clocks it lower the more the operand bits toggle -- i.e. the practical ceiling beside the published peak.
constexpr int kMfmaProbeGrid = 1024;      // workgroups of 8 waves
constexpr int kMfmaProbeOperands = 5120;  // 10 fragments x 64 lanes x 8 elements
__global__ __launch_bounds__(512) void mfma_probe_kernel(const bf16_t* __restrict__ operands, int iters,
                                                         float* __restrict__ sink) {
  const int l = threadIdx.x & 63;
  bf16x8 a[8], b[2];
#pragma unroll
  for (int i = 0; i < 10; ++i) {
    union {
      uint4 u;
      bf16x8 v;
    } cvt;
    cvt.u = reinterpret_cast<const uint4*>(operands)[i * 64 + l];
    if (i < 8)
      a[i] = cvt.v;
    else
      b[i - 8] = cvt.v;
  }
  f32x16 acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  for (int t = 0; t < iters; ++t) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = mfma32<false>(a[ks], b[c & 1], acc[c]);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[c][r];
  if (s == 123456.789f && iters < 0) sink[0] = s;  // never true; keeps the loop alive
}
}  // namespace fm

extern "C" int fm_debug_mfma(const void* operands, int64_t n_operands, int iters, void* sink, void* stream) {
  using namespace fm;
  FM_REQUIRE(operands && sink && n_operands >= kMfmaProbeOperands && iters >= 0, FM_ERR_ARG,
             "fm_debug_mfma: n_operands=%lld (at least %d bf16 values) iters=%d", (long long)n_operands,
             kMfmaProbeOperands, iters);
  if (iters == 0) return FM_OK;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(kMfmaProbeGrid), dim3(512), 0, as_stream(stream),
                     (const bf16_t*)operands, iters, (float*)sink);
  return launch_status("fm_debug_mfma");
}

extern "C" int fm_debug_read(const void* src, int64_t nbytes, void* sink, void* stream) {
  using namespace fm;
  FM_REQUIRE(src && sink && nbytes >= 0 && nbytes % (16 * 256 * 8) == 0, FM_ERR_ARG,
             "fm_debug_read: nbytes=%lld must be a multiple of 32768", (long long)nbytes);
  if (nbytes == 0) return FM_OK;
  hipLaunchKernelGGL(read_probe_kernel, dim3(4096), dim3(256), 0, as_stream(stream), (const uint4*)src,
                     nbytes / 16, (uint32_t*)sink);
  return launch_status("fm_debug_read");
}

extern "C" int fm_debug_gather(const void* src, int64_t region_bytes, int passes, void* sink, void* stream) {
  using namespace fm;
  const int64_t rows = region_bytes / 256;
  FM_REQUIRE(src && sink && passes >= 0 && rows >= (1 << 10) && rows <= (int64_t(1) << 31) && (rows & (rows - 1)) == 0 &&
                 region_bytes % 256 == 0,
             FM_ERR_ARG, "fm_debug_gather: region_bytes=%lld must be 256 x a power of two >= 2^10, passes=%d",
             (long long)region_bytes, passes);
  if (passes == 0) return FM_OK;
  // 1024 workgroups x 16 groups x 8 rows = 2^17 rows per sweep of the grid
  hipLaunchKernelGGL(gather_probe_kernel, dim3(1024), dim3(256), 0, as_stream(stream), (const uint4*)src,
                     uint32_t(rows), passes, (uint32_t*)sink);
  return launch_status("fm_debug_gather");
}

extern "C" int fm_debug_copy(void* dst, const void* src, int64_t nbytes, void* stream) {
  using namespace fm;
  FM_REQUIRE(dst && src && nbytes >= 0 && nbytes % 16 == 0, FM_ERR_ARG, "fm_debug_copy: nbytes=%lld",
             (long long)nbytes);
  if (nbytes == 0) return FM_OK;
  hipLaunchKernelGGL(copy_probe_kernel, dim3(4096), dim3(256), 0, as_stream(stream),
                     (const uint4*)src, (uint4*)dst, nbytes / 16);
  return launch_status("fm_debug_copy");
}
