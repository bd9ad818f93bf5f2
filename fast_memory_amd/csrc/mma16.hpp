// The two 16-bit element types of the MFMA kernels behind one interface: operands travel as raw
// 128-bit registers (eight elements), only the MFMA instruction and the fp32 -> 16-bit rounding
// differ between bf16 and fp16 (fp16 is what the reference's performance harness runs,
// triton_kernel.py:496).  Fragment layouts of the f16 and bf16 forms of an instruction are the same.
#pragma once
#include "common.hpp"

namespace fm {

template <bool F16>
struct Mma {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 b8;
  typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 h8;
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 b2;
  typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 h2;
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f2;
  typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f4;
  typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f16v;

  // v_mfma_f32_16x16x32_{bf16,f16}
  __device__ static __forceinline__ f4 m16(uint4 a, uint4 b, f4 c) {
    if constexpr (F16)
      return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
  }
  // v_mfma_f32_32x32x16_{bf16,f16}
  __device__ static __forceinline__ f16v m32(uint4 a, uint4 b, f16v c) {
    if constexpr (F16)
      return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
  }
  // v_mfma_f32_16x16x16_{bf16_1k,f16}: four elements per operand
  __device__ static __forceinline__ f4 m16k16(uint2 a, uint2 b, f4 c) {
    typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s4;
    typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 h4;
    if constexpr (F16)
      return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h4, a), __builtin_bit_cast(h4, b), c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s4, a), __builtin_bit_cast(s4, b), c, 0, 0, 0);
  }
  // the two elements of a packed word as floats
  __device__ static __forceinline__ float lo(uint32_t w) {
    if constexpr (F16)
      return float(__builtin_bit_cast(_Float16, uint16_t(w & 0xffffu)));
    else
      return __uint_as_float(w << 16);
  }
  __device__ static __forceinline__ float hi(uint32_t w) {
    if constexpr (F16)
      return float(__builtin_bit_cast(_Float16, uint16_t(w >> 16)));
    else
      return __uint_as_float(w & 0xffff0000u);
  }
  // two floats rounded to nearest even and packed (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32)
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    f2 x = {lo, hi};
    if constexpr (F16)
      return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, h2));
    else
      return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, b2));
  }
};

// A vector instruction may touch what an MFMA of 8 passes wrote 11 issue slots after it at the earliest.  The
// compiler counts the slots within a basic block and fills up with s_nop, but not across a branch -- and the
// attention kernels have one, around the masking of a ragged tile, between the last MFMAs of the scores and
// the row maxima.  Read too early, a maximum comes from a register the MFMA has not written yet: the online
// softmax gives the same result for any running maximum, so results still meet the oracle, but the rounding
// of P, and with it the output bits, then depend on timing (seen with one slot between: outputs differing in
// the last bit from run to run).  These statements spend the slots (other waves of the SIMD issue meanwhile)
// and take the accumulators through, so that every later use of them comes after.
#define FM_MFMA_SETTLE "s_nop 7\n\ts_nop 3"
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float settle_f4;
__device__ __forceinline__ void mfma_settle(settle_f4& a) { asm volatile(FM_MFMA_SETTLE : "+v"(a)); }
__device__ __forceinline__ void mfma_settle(settle_f4& a, settle_f4& b) { asm volatile(FM_MFMA_SETTLE : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void mfma_settle(settle_f4& a, settle_f4& b, settle_f4& c) {
  asm volatile(FM_MFMA_SETTLE : "+v"(a), "+v"(b), "+v"(c));
}
// the accumulators of T query tiles x 4 key tiles
template <int T, int NQW>
__device__ __forceinline__ void mfma_settle_scores(settle_f4 (&s)[NQW][4]) {
  static_assert(T >= 1 && T <= 3 && T <= NQW, "one to three query tiles");
  if constexpr (T == 1)
    asm volatile(FM_MFMA_SETTLE : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[0][2]), "+v"(s[0][3]));
  else if constexpr (T == 2)
    asm volatile(FM_MFMA_SETTLE
                 : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[0][2]), "+v"(s[0][3]), "+v"(s[1][0]), "+v"(s[1][1]), "+v"(s[1][2]),
                   "+v"(s[1][3]));
  else
    asm volatile(FM_MFMA_SETTLE
                 : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[0][2]), "+v"(s[0][3]), "+v"(s[1][0]), "+v"(s[1][1]), "+v"(s[1][2]),
                   "+v"(s[1][3]), "+v"(s[2][0]), "+v"(s[2][1]), "+v"(s[2][2]), "+v"(s[2][3]));
}

}  // namespace fm
