// Arg-top-Z over the rows of an fp32 matrix (memory.py:273, triton_kernel.py:278).
//
// Contract: output row r lists the min(Z,N) indices of the largest entries of
// Y[r,:], ordered by (value descending, index ascending).  Every element is
// mapped to a unique 64-bit composite  (float_key(y) << 32) | (2^32-1 - index),
// so "value desc, index asc" is plain descending order of composites and no
// stability argument is needed anywhere below.
//
// One workgroup per row:
//   1. radix select of the Zc-th largest composite: 12+10+10 bits of the value
//      key, then (only if equal values straddle the cut) 11+11+10 bits of the
//      index part; every pass re-reads the row and histograms one digit in LDS;
//      the loop stops as soon as the digit bin that holds the cut is needed in
//      full;
//   2. one more read collects the exactly Zc composites >= the cut into LDS;
//   3. bitonic sort (descending) in LDS, indices written out.
// HBM traffic: (passes + 1) reads of the row, typically 4; LDS: 8*pow2(Zc) +
// 16 KiB.
#include "common.hpp"

namespace fm {

constexpr int kSelThreads = 1024;
constexpr int kSelMaxBins = 4096;

__device__ __forceinline__ uint64_t composite(float y, uint32_t i) {
  return (uint64_t(float_key(y)) << 32) | uint64_t(0xffffffffu - i);
}

// Calls f(value, index) for every element of the row; 128-bit loads on the
// aligned body.
template <typename F>
__device__ __forceinline__ void for_each_in_row(const float* row, int N, F f) {
  int tid = threadIdx.x;
  int head = int((4 - ((reinterpret_cast<uintptr_t>(row) >> 2) & 3)) & 3);
  if (head > N) head = N;
  if (tid < head) f(row[tid], uint32_t(tid));
  int nvec = (N - head) >> 2;
  const float4* v = reinterpret_cast<const float4*>(row + head);
  for (int i = tid; i < nvec; i += kSelThreads) {
    float4 x = v[i];
    uint32_t b = uint32_t(head + 4 * i);
    f(x.x, b);
    f(x.y, b + 1);
    f(x.z, b + 2);
    f(x.w, b + 3);
  }
  int tail0 = head + 4 * nvec;
  if (tail0 + tid < N) f(row[tail0 + tid], uint32_t(tail0 + tid));
}

__global__ __launch_bounds__(kSelThreads) void argtopz_kernel(const float* __restrict__ Y, int N,
                                                              int64_t ldy, int Zc, int P,
                                                              int32_t* __restrict__ idx_out) {
  extern __shared__ uint64_t buf[];  // P composites
  __shared__ uint32_t hist[kSelMaxBins];
  __shared__ int scan_tmp[17];
  __shared__ uint64_t s_prefix;
  __shared__ int s_need, s_hit, s_cnt;

  const float* row = Y + int64_t(blockIdx.x) * ldy;
  const int tid = threadIdx.x;
  if (tid == 0) {
    s_prefix = 0;
    s_need = Zc;
    s_cnt = 0;
    s_hit = 0;
  }
  const int kBits[6] = {12, 10, 10, 11, 11, 10};
  int top = 64;  // bits [top,64) of the cut are known and equal s_prefix
  for (int pass = 0; pass < 6; ++pass) {
    const int bits = kBits[pass];
    const int shift = top - bits;
    const int nb = 1 << bits;
    for (int i = tid; i < nb; i += kSelThreads) hist[i] = 0;
    __syncthreads();
    const uint64_t prefix = s_prefix;
    const int need = s_need;
    const bool first = (top == 64);
    for_each_in_row(row, N, [&](float y, uint32_t i) {
      uint64_t c = composite(y, i);
      if (first || (c >> top) == prefix) atomicAdd(&hist[(c >> shift) & uint64_t(nb - 1)], 1u);
    });
    __syncthreads();
    // thread t owns `per` bins, walking digits from the largest down
    const int per = nb >> 10;
    int local = 0;
    for (int j = 0; j < per; ++j) local += int(hist[nb - 1 - (tid * per + j)]);
    int total;
    int running = block_excl_scan(local, scan_tmp, &total);
    for (int j = 0; j < per; ++j) {
      int b = nb - 1 - (tid * per + j);
      int h = int(hist[b]);
      if (running < need && need <= running + h) {
        s_prefix = (prefix << bits) | uint64_t(b);
        s_need = need - running;
        s_hit = (h == need - running);
      }
      running += h;
    }
    __syncthreads();
    top = shift;
    if (s_hit || top == 0) break;
  }
  const uint64_t cut = s_prefix << top;  // top == 0 only after the last pass
  for_each_in_row(row, N, [&](float y, uint32_t i) {
    uint64_t c = composite(y, i);
    if (c >= cut) {
      int pos = atomicAdd(&s_cnt, 1);
      if (pos < P) buf[pos] = c;
    }
  });
  for (int i = Zc + tid; i < P; i += kSelThreads) buf[i] = 0;
  __syncthreads();
  // bitonic sort, descending
  for (int k = 2; k <= P; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < (P >> 1); t += kSelThreads) {
        int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
        int p = i | j;
        uint64_t a = buf[i], b = buf[p];
        bool desc = (i & k) == 0;
        if (desc ? (a < b) : (a > b)) {
          buf[i] = b;
          buf[p] = a;
        }
      }
      __syncthreads();
    }
  }
  int32_t* o = idx_out + int64_t(blockIdx.x) * Zc;
  for (int i = tid; i < Zc; i += kSelThreads) o[i] = int32_t(0xffffffffu - uint32_t(buf[i]));
}

static int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

}  // namespace fm

extern "C" size_t fm_argtopz_workspace(int64_t, int, int) { return 0; }

extern "C" int fm_argtopz_f32(const float* Y, int64_t rows, int N, int64_t ldy, int Z,
                              int32_t* idx_out, void* ws, size_t ws_bytes, void* stream) {
  using namespace fm;
  (void)ws;
  (void)ws_bytes;
  FM_REQUIRE(rows >= 0 && N >= 1 && Z >= 1, FM_ERR_ARG, "fm_argtopz_f32: rows=%lld N=%d Z=%d",
             (long long)rows, N, Z);
  FM_REQUIRE(ldy >= N, FM_ERR_ARG, "fm_argtopz_f32: ldy=%lld < N=%d", (long long)ldy, N);
  if (rows == 0) return FM_OK;
  FM_REQUIRE(Y && idx_out, FM_ERR_ARG, "fm_argtopz_f32: null pointer");
  FM_REQUIRE(rows <= 0x7fffffffLL, FM_ERR_UNSUPPORTED, "fm_argtopz_f32: too many rows");
  const int Zc = Z < N ? Z : N;
  FM_REQUIRE(Zc <= FM_MAX_Z, FM_ERR_UNSUPPORTED, "fm_argtopz_f32: min(Z,N)=%d exceeds FM_MAX_Z=%d",
             Zc, FM_MAX_Z);
  const int P = next_pow2(Zc);
  const size_t dyn = size_t(P) * sizeof(uint64_t);
  FM_ALLOW_LDS(argtopz_kernel, FM_MAX_Z * sizeof(uint64_t), "fm_argtopz_f32: lds");
  hipLaunchKernelGGL(argtopz_kernel, dim3(unsigned(rows)), dim3(kSelThreads), dyn,
                     as_stream(stream), Y, N, ldy, Zc, P, idx_out);
  return launch_status("fm_argtopz_f32");
}
