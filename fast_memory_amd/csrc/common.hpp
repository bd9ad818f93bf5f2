// Shared host/device helpers of libfastmem (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>
#include <atomic>
#include <mutex>

#include "../../include/fastmem_debug.h"

namespace fm {

// ---- host side: status + message ------------------------------------------
void set_error(const char* fmt, ...);
int launch_status(const char* what);  // FM_OK, or FM_ERR_LAUNCH with message
bool debug_hooks_enabled();            // FASTMEM_DEBUG_HOOKS=1 was set when the library was first called

#define FM_REQUIRE(cond, code, ...)   \
  do {                                \
    if (!(cond)) {                    \
      ::fm::set_error(__VA_ARGS__);   \
      return (code);                  \
    }                                 \
  } while (0)

// Raises the dynamic-LDS ceiling of a kernel (needed above 64 KiB).
static inline int allow_lds(const void* fn, size_t bytes, const char* what) {
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes)) != hipSuccess)
    return launch_status(what);
  return FM_OK;
}
#define FM_ALLOW_LDS(kernel, bytes, what)                                              \
  do {                                                                                 \
    static bool done_ = false;                                                         \
    if (!done_) {                                                                      \
      int rc_ = ::fm::allow_lds(reinterpret_cast<const void*>(kernel), (bytes), what); \
      if (rc_ != FM_OK) return rc_;                                                    \
      done_ = true;                                                                    \
    }                                                                                  \
  } while (0)

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- device side ------------------------------------------------------------
constexpr int kWave = 64;
constexpr float kLog2e = 1.44269504f;           // constant the reference kernel uses
constexpr float kLn2 = 0.69314718055994531f;

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t x) { return __uint_as_float(uint32_t(x) << 16); }
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {  // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t(0x7fc0);
  u += 0x7fffu + ((u >> 16) & 1u);
  return bf16_t(u >> 16);
}

struct f16_t {  // raw IEEE half bits (a type of its own: bf16_t is the plain uint16_t)
  uint16_t b;
};
static inline bool dtype_ok(int dtype) { return dtype == FM_F32 || dtype == FM_BF16 || dtype == FM_F16; }
static inline int dtype_bytes(int dtype) { return dtype == FM_F32 ? 4 : 2; }

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int dtype = FM_F32;
  __device__ static __forceinline__ float load(const float* p) { return *p; }
  __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
  __device__ static __forceinline__ float round(float v) { return v; }
};
template <> struct Elem<bf16_t> {
  static constexpr int dtype = FM_BF16;
  __device__ static __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  __device__ static __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
  __device__ static __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

template <> struct Elem<f16_t> {
  static constexpr int dtype = FM_F16;
  __device__ static __forceinline__ float load(const f16_t* p) { return float(__builtin_bit_cast(_Float16, p->b)); }
  __device__ static __forceinline__ void store(f16_t* p, float v) {
    p->b = __builtin_bit_cast(uint16_t, _Float16(v));  // round to nearest even
  }
  __device__ static __forceinline__ float round(float v) { return float(_Float16(v)); }
};

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
// inclusive scan across the wave
__device__ __forceinline__ int wave_incl_scan(int v) {
  int l = lane_id();
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    int t = __shfl_up(v, o);
    if (l >= o) v += t;
  }
  return v;
}
// The same scan on the data-parallel-primitive path of the VALU (no LDS-pipe permutes): shifts within the
// 16-lane rows, then the last lane of row 0 / 2 into row 1 / 3 and lane 31 into the upper half.  Lanes
// without a source add 0.  All 64 lanes must be active.
__device__ __forceinline__ int wave_incl_scan_dpp(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}
__device__ __forceinline__ long long wave_incl_scan_ll(long long v) {
  int l = lane_id();
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    long long t = __shfl_up(v, o);
    if (l >= o) v += t;
  }
  return v;
}

// Exclusive scan over a block of up to 1024 threads (<= 16 waves).
// `smem` needs 17 ints.  Returns the exclusive prefix; *total gets the block sum.
__device__ __forceinline__ int block_excl_scan(int v, int* smem, int* total) {
  int l = lane_id(), w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  int inc = wave_incl_scan(v);
  if (l == 63) smem[w] = inc;
  __syncthreads();
  if (w == 0) {
    int s = (l < nw) ? smem[l] : 0;
    int si = wave_incl_scan(s);
    if (l < nw) smem[l] = si - s;
    if (l == nw - 1) smem[16] = si;
  }
  __syncthreads();
  int res = inc - v + smem[w];
  *total = smem[16];
  __syncthreads();
  return res;
}
__device__ __forceinline__ long long block_excl_scan_ll(long long v, long long* smem, long long* total) {
  int l = lane_id(), w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  long long inc = wave_incl_scan_ll(v);
  if (l == 63) smem[w] = inc;
  __syncthreads();
  if (w == 0) {
    long long s = (l < nw) ? smem[l] : 0;
    long long si = wave_incl_scan_ll(s);
    if (l < nw) smem[l] = si - s;
    if (l == nw - 1) smem[16] = si;
  }
  __syncthreads();
  long long res = inc - v + smem[w];
  *total = smem[16];
  __syncthreads();
  return res;
}

// Index of the first work item of a row >= `row` (n_it if there is none); the items are in row order.  A
// search every wave runs for itself with all 64 lanes active, 64 probes a round: three rounds of
// dependent loads for 2^18 items.
__device__ __forceinline__ int first_item_of_row(const fm_item* __restrict__ items, int n_it, int row) {
  const int lane = lane_id();
  int lo = 0, hi = n_it;  // the answer lies in [lo, hi]
  while (hi > lo) {
    const int step = (hi - lo + 63) >> 6;
    const int probe = lo + lane * step;
    const bool ge = probe >= hi || items[probe].row >= row;
    const unsigned long long m = __ballot(ge);
    const int f = m ? __ffsll(m) - 1 : 64;  // the first lane whose probe is at or past the row
    hi = min(hi, lo + f * step);
    lo = f == 0 ? hi : lo + (f - 1) * step + 1;
  }
  return lo;
}

// Order-preserving map float -> uint32 (larger float <=> larger key);
// -0 is folded onto +0 and every NaN becomes the largest key.
__device__ __forceinline__ uint32_t float_key(float x) {
  if (x != x) return 0xffffffffu;
  uint32_t u = __float_as_uint(x + 0.0f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

}  // namespace fm
