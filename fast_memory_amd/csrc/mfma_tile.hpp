// MFMA building blocks shared by the projection-type kernels (gfx950).
//
// v_mfma_f32_32x32x16_bf16: A is 32x16, B is 16x32, both bf16; lane l supplies
// row/column (l % 32) and the 8 consecutive contraction elements starting at
// (l / 32) * 8.  The 16 accumulator floats of lane l are column (l % 32), rows
// acc_row_32(r, l), r = 0..15.
#pragma once
#include "common.hpp"

namespace fm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

// v_mfma_f32_32x32x16_bf16 or, with F16, v_mfma_f32_32x32x16_f16 on the same registers (the fragment layouts
// are the same; a kernel instantiated with F16 reads IEEE half data through its bf16_t pointers)
template <bool F16>
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  if constexpr (F16) {
    typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 h8;
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
}

__device__ __forceinline__ int acc_row_32(int r, int lane) {
  return 8 * (r >> 2) + ((lane >> 5) << 2) + (r & 3);
}

// Copies `rows` rows [r0, r0+rows) of a [R, d] bf16 matrix into LDS with row
// stride `ld` elements; rows past R are zero.  d % 8 == 0.  256 threads.
__device__ __forceinline__ void stage_rows_bf16(bf16_t* dst, int ld, const bf16_t* src, int r0,
                                                int R, int d, int rows) {
  const int cpr = d >> 3;
  const int total = rows * cpr;
  for (int e = threadIdx.x; e < total; e += 256) {
    int r = e / cpr, ch = e - r * cpr;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (r0 + r < R) v = *reinterpret_cast<const uint4*>(src + int64_t(r0 + r) * d + ch * 8);
    *reinterpret_cast<uint4*>(dst + r * ld + ch * 8) = v;
  }
}

// acc[mi][ni] = sum over k of sa[mi*32 + i][k] * sb[ni*32 + j][k], contraction
// in ascending 16-element steps (the order every projection-type kernel
// shares, so equal operands give bit-equal sums).  d % 16 == 0.
template <bool F16 = false>
__device__ __forceinline__ void mfma_tile_64x64(const bf16_t* sa, const bf16_t* sb, int ld, int d,
                                                f32x16 (&acc)[2][2]) {
  const int l = lane_id();
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;
  const bf16_t* pa = sa + (l & 31) * ld + (l >> 5) * 8;
  const bf16_t* pb = sb + (l & 31) * ld + (l >> 5) * 8;
  for (int k = 0; k < d; k += 16) {
    bf16x8 a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      a[i] = *reinterpret_cast<const bf16x8*>(pa + i * 32 * ld + k);
      b[i] = *reinterpret_cast<const bf16x8*>(pb + i * 32 * ld + k);
    }
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
        acc[mi][ni] = mfma32<F16>(a[mi], b[ni], acc[mi][ni]);
  }
}

}  // namespace fm
