// Projection Y = A.K^T (memory.py:261, triton_kernel.py:277) and query hashing
// argmax_c A.q (memory.py:281-283, triton_kernel.py:280-281).
#include "common.hpp"
#include "mfma_tile.hpp"

namespace fm {

// ---------------------------------------------------------------------------
// bf16 projection on MFMA: one workgroup = 128 keys x 128 buckets, the whole
// contraction (d <= 256) staged once in LDS, four waves in a 2x2 grid of 64x64
// sub-tiles, each 2x2 v_mfma_f32_32x32x16_bf16 with keys on the A operand and
// ascending contraction steps (the fused index build computes Y the same way,
// so both give bit-equal values).  The accumulators are transposed through LDS
// so that every Y row segment leaves as 512 contiguous bytes.
// Bound: HBM write of Y (4 B per 2*d flops).
// ---------------------------------------------------------------------------
constexpr int kProjYLd = 132;  // floats per staged output row (128 + 4 pad)

template <bool F16>
__global__ __launch_bounds__(256) void project_bf16_kernel(const bf16_t* __restrict__ A,
                                                           const bf16_t* __restrict__ K,
                                                           float* __restrict__ Y, int C, int N,
                                                           int d, int64_t ldy) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lds_ld = d + 8;  // bf16 elements per staged row (16 B pad: conflict-free b128 reads)
  bf16_t* sK = reinterpret_cast<bf16_t*>(smem);
  bf16_t* sA = sK + 128 * lds_ld;
  float* sY = reinterpret_cast<float*>(smem);  // reused after the MFMA phase: [128 buckets][132]
  const int h = blockIdx.z;
  const int c0 = blockIdx.y * 128;
  const int n0 = blockIdx.x * 128;
  const bf16_t* Ah = A + int64_t(h) * C * d;
  const bf16_t* Kh = K + int64_t(h) * N * d;
  stage_rows_bf16(sK, lds_ld, Kh, n0, N, d, 128);
  stage_rows_bf16(sA, lds_ld, Ah, c0, C, d, 128);
  __syncthreads();
  const int w = threadIdx.x >> 6, l = lane_id();
  const int wm = w >> 1, wn = w & 1;  // wm: key half, wn: bucket half
  f32x16 acc[2][2];
  mfma_tile_64x64<F16>(sK + (wm * 64) * lds_ld, sA + (wn * 64) * lds_ld, lds_ld, d, acc);
  __syncthreads();  // operands consumed; the same LDS now takes the output tile
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      const int bc = wn * 64 + ni * 32 + (l & 31);          // bucket column of this lane
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {                      // rows 8*q4 + 4*(l/32) + 0..3
        const int kr = wm * 64 + mi * 32 + 8 * q4 + ((l >> 5) << 2);
        float4 v = make_float4(acc[mi][ni][4 * q4], acc[mi][ni][4 * q4 + 1], acc[mi][ni][4 * q4 + 2],
                               acc[mi][ni][4 * q4 + 3]);
        *reinterpret_cast<float4*>(&sY[bc * kProjYLd + kr]) = v;
      }
    }
  __syncthreads();
  float* Yh = Y + int64_t(h) * C * ldy;
  const bool vec_ok = ((ldy & 3) == 0) && ((reinterpret_cast<uintptr_t>(Y) & 15) == 0) && (n0 + 128 <= N);
  // 32 threads per row (512 B), 8 rows per pass
  for (int r = threadIdx.x >> 5; r < 128; r += 8) {
    const int c = c0 + r;
    if (c >= C) break;
    const int k4 = (threadIdx.x & 31) * 4;
    const float4 v = *reinterpret_cast<const float4*>(&sY[r * kProjYLd + k4]);
    float* dst = Yh + int64_t(c) * ldy + n0 + k4;
    if (vec_ok) {
      *reinterpret_cast<float4*>(dst) = v;
    } else {
      if (n0 + k4 < N) dst[0] = v.x;
      if (n0 + k4 + 1 < N) dst[1] = v.y;
      if (n0 + k4 + 2 < N) dst[2] = v.z;
      if (n0 + k4 + 3 < N) dst[3] = v.w;
    }
  }
}

// ---------------------------------------------------------------------------
// bf16, d = 128: bucket-stationary streaming form of the same product.  The kernel
// is a fill of Y (4 B written per 256 flops: HBM-write-bound by a wide margin), so
// it is built to keep stores flowing: a workgroup of four waves holds a slab of
// buckets as MFMA A-operand fragments in registers for its whole life and walks
// a range of keys step by step; the keys of a step go through a
// double-buffered LDS tile (global loads of step i+1 are in flight while step i
// computes and stores; one barrier per step), and the accumulators are stored
// straight from registers: with the keys on the B operand a register holds 32
// consecutive keys of one bucket row across lanes, i.e. every store instruction
// writes two full 128-byte lines.  Same contraction order per output as the
// tile kernel above (ascending 16-element steps into one fp32 accumulator).
// grid (key ranges, slabs, H).
// ---------------------------------------------------------------------------
constexpr int kPsLd = 136;  // bf16 elements per staged key row (128 + 8 pad)

// 16-byte chunks of keys key0, key0 + 16, ... (clamped to the last key) into registers.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // (an array of HIP's uint4 structs stays in scratch)
template <int NCH>
__device__ __forceinline__ void ps_fetch(u32x4 (&st)[NCH], const bf16_t* __restrict__ kp, int key0, int N) {
#pragma unroll
  for (int i = 0; i < NCH; ++i) st[i] = *reinterpret_cast<const u32x4*>(kp + int64_t(min(key0 + 16 * i, N - 1)) * 128);
}

// BT bucket tiles per wave (the slab of a workgroup is 4 * 32 BT buckets), KT key tiles per step.
template <int BT, int KT, bool F16>
__global__ __launch_bounds__(256) void project_stream_bf16_d128_kernel(const bf16_t* __restrict__ A,
                                                                       const bf16_t* __restrict__ K,
                                                                       float* __restrict__ Y, int C, int N,
                                                                       int64_t ldy, int steps_per_wg) {
  constexpr int kKeys = 32 * KT, kWaveRows = 32 * BT;
  __shared__ __attribute__((aligned(16))) bf16_t sK[2][kKeys * kPsLd];
  const int h = blockIdx.z;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), l = lane_id();
  const int b0 = blockIdx.y * (4 * kWaveRows) + w * kWaveRows;  // first bucket of this wave
  const bf16_t* Ah = A + int64_t(h) * C * 128;
  const bf16_t* Kh = K + int64_t(h) * N * 128;
  float* Yh = Y + int64_t(h) * C * ldy;
  const int n_steps_total = (N + kKeys - 1) / kKeys;
  const int s0 = blockIdx.x * steps_per_wg;
  const int s1 = min(s0 + steps_per_wg, n_steps_total);
  if (s0 >= s1) return;
  // A fragments: bucket tile bt, contraction step ks -> 8 bf16 of row (l % 32) at k = 16 ks + 8 (l / 32)
  bf16x8 af[BT][8];
#pragma unroll
  for (int bt = 0; bt < BT; ++bt) {
    const int row = min(b0 + bt * 32 + (l & 31), C - 1);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      af[bt][ks] = *reinterpret_cast<const bf16x8*>(Ah + int64_t(row) * 128 + ks * 16 + (l >> 5) * 8);
  }
  // staging: kKeys x 16 chunks of 16 B, 2 KT per thread (thread t: chunk t % 16 of keys t / 16 + 16 i)
  u32x4 st[2 * KT];
  const int e_row = threadIdx.x >> 4, e_ch = (threadIdx.x & 15) * 8;
  const bf16_t* kp = Kh + e_ch;
  ps_fetch<2 * KT>(st, kp, s0 * kKeys + e_row, N);
  const bool rows_full = b0 + kWaveRows <= C;
  const uint32_t lane_off = uint32_t(4 * (l >> 5)) * uint32_t(ldy) + uint32_t(l & 31);
  for (int step = s0; step < s1; ++step) {
    bf16_t* buf = sK[(step - s0) & 1];
#pragma unroll
    for (int i = 0; i < 2 * KT; ++i) *reinterpret_cast<u32x4*>(buf + (e_row + 16 * i) * kPsLd + e_ch) = st[i];
    __syncthreads();
    ps_fetch<2 * KT>(st, kp, min(step + 1, s1 - 1) * kKeys + e_row, N);  // (the last step fetches its own tile again)
    if (b0 >= C) continue;  // a wave past the last bucket only helps staging
    f32x16 acc[BT][KT];
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[bt][kt][r] = 0.f;
    const bf16_t* pb = buf + (l & 31) * kPsLd + (l >> 5) * 8;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      bf16x8 kf[KT];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) kf[kt] = *reinterpret_cast<const bf16x8*>(pb + kt * 32 * kPsLd + ks * 16);
#pragma unroll
      for (int bt = 0; bt < BT; ++bt)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
          acc[bt][kt] = mfma32<F16>(af[bt][ks], kf[kt], acc[bt][kt]);
    }
    // store: wave-uniform 64-bit base per (tile, register) + one 32-bit lane offset
    const int n0 = step * kKeys;
    const bool full = rows_full && n0 + kKeys <= N;
    float* ubase = Yh + int64_t(b0) * ldy + n0;
#pragma unroll
    for (int bt = 0; bt < BT; ++bt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
          const int key = n0 + kt * 32 + (l & 31);
          float* ur = ubase + int64_t(bt * 32 + 8 * (r >> 2) + (r & 3)) * ldy + kt * 32;
          const int row = b0 + bt * 32 + acc_row_32(r, l);
          if (full || (row < C && key < N)) ur[lane_off] = acc[bt][kt][r];
        }
  }
}

// ---------------------------------------------------------------------------
// Generic projection (any d <= 256, fp32 or bf16 storage, fp32 FMA chain over
// k = 0..d-1).  64 keys staged in LDS per workgroup; lane = key, waves stride
// over buckets.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void project_generic_kernel(const T* __restrict__ A,
                                                              const T* __restrict__ K,
                                                              float* __restrict__ Y, int C, int N,
                                                              int d, int64_t ldy) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* sK = reinterpret_cast<float*>(smem);  // [64][d+1]
  const int ld = d + 1;
  const int h = blockIdx.y;
  const int n0 = blockIdx.x * 64;
  const T* Kh = K + int64_t(h) * N * d;
  const T* Ah = A + int64_t(h) * C * d;
  for (int e = threadIdx.x; e < 64 * d; e += 256) {
    int r = e / d, k = e - r * d;
    int n = n0 + r;
    sK[r * ld + k] = n < N ? Elem<T>::load(Kh + int64_t(n) * d + k) : 0.f;
  }
  __syncthreads();
  const int w = threadIdx.x >> 6, l = lane_id();
  const int n = n0 + l;
  float* Yh = Y + int64_t(h) * C * ldy;
  for (int c = w; c < C; c += 4) {
    const T* a = Ah + int64_t(c) * d;
    float s = 0.f;
    for (int k = 0; k < d; ++k) s = fmaf(Elem<T>::load(a + k), sK[l * ld + k], s);
    if (n < N) Yh[int64_t(c) * ldy + n] = s;
  }
}

// ---------------------------------------------------------------------------
// Generic query hash: 64 queries staged in LDS, lane = query, each wave scans a
// quarter of the buckets keeping (best score, first index), waves combined with
// the same rule: larger score wins, equal scores keep the lower bucket.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qhash_generic_kernel(const T* __restrict__ A,
                                                            const T* __restrict__ q,
                                                            int32_t* __restrict__ hash_out,
                                                            float* __restrict__ scores_out, int C,
                                                            int Sq, int d) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* sQ = reinterpret_cast<float*>(smem);  // [64][d+1]
  __shared__ float s_best[4][64];
  __shared__ int s_idx[4][64];
  const int ld = d + 1;
  const int h = blockIdx.y;
  const int i0 = blockIdx.x * 64;
  const T* qh = q + int64_t(h) * Sq * d;
  const T* Ah = A + int64_t(h) * C * d;
  for (int e = threadIdx.x; e < 64 * d; e += 256) {
    int r = e / d, k = e - r * d;
    int i = i0 + r;
    sQ[r * ld + k] = i < Sq ? Elem<T>::load(qh + int64_t(i) * d + k) : 0.f;
  }
  __syncthreads();
  const int w = threadIdx.x >> 6, l = lane_id();
  const int i = i0 + l;
  const int per = (C + 3) / 4;
  const int cb = w * per, ce = min(C, cb + per);
  float best = -INFINITY;
  int besti = 0x7fffffff;
  for (int c = cb; c < ce; ++c) {
    const T* a = Ah + int64_t(c) * d;
    float s = 0.f;
    for (int k = 0; k < d; ++k) s = fmaf(Elem<T>::load(a + k), sQ[l * ld + k], s);
    if (scores_out && i < Sq) scores_out[(int64_t(h) * Sq + i) * C + c] = s;
    if (besti == 0x7fffffff || s > best) {
      best = s;
      besti = c;
    }
  }
  s_best[w][l] = best;
  s_idx[w][l] = besti;
  __syncthreads();
  if (w == 0 && i < Sq) {
    for (int ww = 1; ww < 4; ++ww) {
      float b = s_best[ww][l];
      int bi = s_idx[ww][l];
      if (bi != 0x7fffffff && (besti == 0x7fffffff || b > best)) {  // later waves hold higher buckets
        best = b;
        besti = bi;
      }
    }
    hash_out[int64_t(h) * Sq + i] = besti;
  }
}

// ---------------------------------------------------------------------------
// bf16 query hash on MFMA: workgroup = 128 queries of one KV head; loops over
// bucket tiles of 128 staged in LDS; accumulator layout puts one query per lane
// column, so the running (max, first index) is kept per lane without shuffles
// and combined across the two lane halves and the two bucket-side waves at the
// end.
// ---------------------------------------------------------------------------
template <bool F16>
__global__ __launch_bounds__(256) void qhash_bf16_kernel(const bf16_t* __restrict__ A,
                                                         const bf16_t* __restrict__ q,
                                                         int32_t* __restrict__ hash_out,
                                                         float* __restrict__ scores_out, int C,
                                                         int Sq, int d) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lds_ld = d + 8;
  bf16_t* sA = reinterpret_cast<bf16_t*>(smem);  // bucket tile (M side)
  bf16_t* sB = sA + 128 * lds_ld;                // query tile  (N side)
  __shared__ float s_best[2][128];
  __shared__ int s_idx[2][128];
  const int h = blockIdx.y;
  const int i0 = blockIdx.x * 128;
  const bf16_t* Ah = A + int64_t(h) * C * d;
  const bf16_t* qh = q + int64_t(h) * Sq * d;
  const int w = threadIdx.x >> 6, l = lane_id();
  const int wm = w >> 1, wn = w & 1;
  stage_rows_bf16(sB, lds_ld, qh, i0, Sq, d, 128);
  float best[2] = {-INFINITY, -INFINITY};
  int besti[2] = {0x7fffffff, 0x7fffffff};
  for (int c0 = 0; c0 < C; c0 += 128) {
    __syncthreads();  // previous tile consumed (and sB staged on the first trip)
    stage_rows_bf16(sA, lds_ld, Ah, c0, C, d, 128);
    __syncthreads();
    f32x16 acc[2][2];
    mfma_tile_64x64<F16>(sA + (wm * 64) * lds_ld, sB + (wn * 64) * lds_ld, lds_ld, d, acc);
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      int i = i0 + wn * 64 + ni * 32 + (l & 31);
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) {  // rows ascend with r inside a tile
          int c = c0 + wm * 64 + mi * 32 + acc_row_32(r, l);
          float s = acc[mi][ni][r];
          if (c < C) {
            if (scores_out && i < Sq) scores_out[(int64_t(h) * Sq + i) * C + c] = s;
            if (besti[ni] == 0x7fffffff || s > best[ni] || (s == best[ni] && c < besti[ni])) {
              best[ni] = s;
              besti[ni] = c;
            }
          }
        }
    }
  }
  // combine lane halves (rows interleave between the halves, so compare indices on ties)
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    float ob = __shfl_xor(best[ni], 32);
    int oi = __shfl_xor(besti[ni], 32);
    if (oi != 0x7fffffff && (besti[ni] == 0x7fffffff || ob > best[ni] || (ob == best[ni] && oi < besti[ni]))) {
      best[ni] = ob;
      besti[ni] = oi;
    }
    if (l < 32) {
      s_best[wm][wn * 64 + ni * 32 + l] = best[ni];
      s_idx[wm][wn * 64 + ni * 32 + l] = besti[ni];
    }
  }
  __syncthreads();
  if (threadIdx.x < 128) {
    int i = i0 + threadIdx.x;
    float b0 = s_best[0][threadIdx.x], b1 = s_best[1][threadIdx.x];
    int i0x = s_idx[0][threadIdx.x], i1x = s_idx[1][threadIdx.x];
    int res = i0x;
    if (i1x != 0x7fffffff && (i0x == 0x7fffffff || b1 > b0 || (b1 == b0 && i1x < i0x))) res = i1x;
    if (i < Sq) hash_out[int64_t(h) * Sq + i] = res;
  }
}

// ---------------------------------------------------------------------------
// bf16 query hash, d = 128, streaming form (no scores written): a workgroup of 8
// waves holds 512 queries as resident MFMA B fragments (64 per wave) and streams
// the bucket rows of A through LDS tiles of 64 rows.  One query per lane column:
// the running maximum and its position are per-lane registers, updated with three
// VALU instructions per accumulator register (compare, select value, select the
// row number as an inline constant); buckets arrive in ascending order, so
// "strictly greater" keeps the first maximum.  The loop is software-pipelined in
// tiles: the 32 MFMAs of a tile -- four independent chains, (32-row sub-tile,
// 32-query fragment) -- alternate in the instruction stream with the scan of the
// tile before it, which sits in a second set of accumulators, and with the LDS
// reads of the next A fragments.  Measured on this hardware with register-resident
// loops: with four chains the VALU work of the same wave is issued in the shadow of
// its MFMAs (four VALU instructions per MFMA cost nothing, six cost 12 %); with two
// chains it is not, and VALU work of the SIMD's other wave mostly adds to the MFMA
// time.  The device is power-bound in such loops and clocks them lower the more
// their operands toggle and the more LDS and VALU work they carry: a stream of these
// MFMAs alone sustains 78 % of the nominal peak on operands of a few values and
// 64 % on random ones, and with six VALU instructions per MFMA 56 %.  The scores are
// the same MFMA sums as in qhash_bf16_kernel (same instruction, operand roles and
// contraction order), so both kernels return identical hashes.
// Roofline: MFMA, 2*C*d flops per query.
// ---------------------------------------------------------------------------
constexpr int kQsLd = 128 + 8;

template <int K>
__device__ __forceinline__ void argmax_step(float& best, int& pos, float s) {
  asm volatile("v_cmp_gt_f32 vcc, %2, %0\n\tv_cndmask_b32_e32 %0, %0, %2, vcc\n\tv_cndmask_b32_e64 %1, %1, %3, vcc"
               : "+v"(best), "+v"(pos)
               : "v"(s), "n"(K)
               : "vcc");
}
// two steps in one statement (the compiler puts a wait state between two statements that write vcc)
template <int K0, int K1>
__device__ __forceinline__ void argmax_step2(float& best, int& pos, float s0, float s1) {
  asm volatile(
      "v_cmp_gt_f32 vcc, %2, %0\n\tv_cndmask_b32_e32 %0, %0, %2, vcc\n\tv_cndmask_b32_e64 %1, %1, %4, vcc\n\t"
      "v_cmp_gt_f32 vcc, %3, %0\n\tv_cndmask_b32_e32 %0, %0, %3, vcc\n\tv_cndmask_b32_e64 %1, %1, %5, vcc"
      : "+v"(best), "+v"(pos)
      : "v"(s0), "v"(s1), "n"(K0), "n"(K1)
      : "vcc");
}

// position of accumulator register R of the 32-row sub-tile MI inside the 64-row tile, for
// lanes 0..31 (lanes 32..63 hold the rows 4 further down)
constexpr int qs_row(int MI, int R) { return MI * 32 + 8 * (R >> 2) + (R & 3); }

// One tile step of the pipeline, slot I of 32: k-step I / 4, chain I % 4 = (sub-tile mi, query half ni).
//   MFMA: X[mi][ni] += A fragment (sub-tile mi of the tile at frag_lds, k-step I / 4) x the half's queries;
//         the two A fragments of the next k-step are read from LDS in the first slot of every k-step, the
//         first ones of the next tile (next_lds) in that of the last.
//   SCAN: two registers of the finished set Y.  Slots 0..15 cover sub-tile 0 (slot j: query half j % 2,
//         registers 2 (j / 2) and the next), slots 16..31 sub-tile 1, so every query half sees its rows in
//         ascending order.  Register 0 goes through plain C++ so that the compiler, which cannot see into
//         the asm, places the wait states a read of a fresh MFMA result needs (the MFMA that produced an
//         accumulator was issued before those of the accumulators read later).
// sched_barrier pins the interleaving: an MFMA keeps the matrix pipe busy for 32 cycles, the six VALU
// instructions behind it take 24.
template <bool F16, bool MFMA, bool SCAN, int I>
__device__ __forceinline__ void qs_tile_step(f32x16 (&X)[2][2], const f32x16 (&Y)[2][2], bf16x8 (&af)[2][2],
                                             const bf16_t* frag_lds, const bf16_t* next_lds,
                                             const bf16x8 (&bfrag)[2][8], float (&best)[2], int (&pos)[2]) {
  if constexpr (I < 32) {
    constexpr int ks = I >> 2, mi = (I >> 1) & 1, ni = I & 1;
    if constexpr (MFMA) {
      if constexpr ((I & 3) == 0) {
        if constexpr (ks < 7) {
          af[(ks + 1) & 1][0] = *reinterpret_cast<const bf16x8*>(frag_lds + (ks + 1) * 16);
          af[(ks + 1) & 1][1] = *reinterpret_cast<const bf16x8*>(frag_lds + 32 * kQsLd + (ks + 1) * 16);
        } else {
          af[0][0] = *reinterpret_cast<const bf16x8*>(next_lds);
          af[0][1] = *reinterpret_cast<const bf16x8*>(next_lds + 32 * kQsLd);
        }
      }
      if constexpr (ks == 0) {
        f32x16 z;
#pragma unroll
        for (int r = 0; r < 16; ++r) z[r] = 0.f;
        X[mi][ni] = mfma32<F16>(af[0][mi], bfrag[ni][0], z);
      } else {
        X[mi][ni] = mfma32<F16>(af[ks & 1][mi], bfrag[ni][ks], X[mi][ni]);
      }
    }
    if constexpr (SCAN) {
      constexpr int smi = I >> 4, sni = I & 1, r = 2 * ((I & 15) >> 1);
      if constexpr (r == 0) {
        const bool gt = Y[smi][sni][0] > best[sni];
        best[sni] = gt ? Y[smi][sni][0] : best[sni];
        pos[sni] = gt ? qs_row(smi, 0) : pos[sni];
        argmax_step<qs_row(smi, 1)>(best[sni], pos[sni], Y[smi][sni][1]);
      } else {
        argmax_step2<qs_row(smi, r), qs_row(smi, r + 1)>(best[sni], pos[sni], Y[smi][sni][r], Y[smi][sni][r + 1]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    qs_tile_step<F16, MFMA, SCAN, I + 1>(X, Y, af, frag_lds, next_lds, bfrag, best, pos);
  }
}

template <bool F16>
__global__ __launch_bounds__(512) void qhash_stream_kernel(const bf16_t* __restrict__ A,
                                                           const bf16_t* __restrict__ q,
                                                           int32_t* __restrict__ hash_out, int C, int Sq) {
  __shared__ __attribute__((aligned(16))) bf16_t sA[3][64 * kQsLd];
  const int h = blockIdx.y;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const bf16_t* Ah = A + int64_t(h) * C * 128;
  const bf16_t* qh = q + int64_t(h) * Sq * 128;
  const int i0 = blockIdx.x * 512 + w * 64;

  bf16x8 bfrag[2][8];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int i = i0 + ni * 32 + (l & 31);
    const bool ok = i < Sq;
    const uint4* pq = reinterpret_cast<const uint4*>(qh + int64_t(ok ? i : 0) * 128 + (l >> 5) * 8);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      union {
        uint4 u;
        bf16x8 b;
      } cvt;
      cvt.u = ok ? pq[2 * ks] : make_uint4(0, 0, 0, 0);
      bfrag[ni][ks] = cvt.b;
    }
  }
  float best[2] = {-INFINITY, -INFINITY};
  int pos[2] = {0, 0}, btile[2] = {0, 0};

  const int ntiles = (C + 63) / 64;
  // rows past C repeat row 0: an equal score later in the order never replaces the running maximum
  uint4 st0, st1;  // a tile on its way from global memory to LDS: rows tid/16 and 32 + tid/16
  auto fetch = [&](int t) {
    const int r0 = t * 64 + (tid >> 4), r1 = r0 + 32;
    st0 = reinterpret_cast<const uint4*>(Ah + int64_t(r0 < C ? r0 : 0) * 128)[tid & 15];
    st1 = reinterpret_cast<const uint4*>(Ah + int64_t(r1 < C ? r1 : 0) * 128)[tid & 15];
  };
  auto stash = [&](int buf) {
    *reinterpret_cast<uint4*>(&sA[buf][(tid >> 4) * kQsLd + (tid & 15) * 8]) = st0;
    *reinterpret_cast<uint4*>(&sA[buf][(32 + (tid >> 4)) * kQsLd + (tid & 15) * 8]) = st1;
  };
  // LDS address of this lane's A fragment 0 of sub-tile 0 of the tile in buffer buf (sub-tile 1: 32 rows on)
  auto frag_ptr = [&](int buf) -> const bf16_t* { return &sA[buf][(l & 31) * kQsLd + (l >> 5) * 8]; };
  // Three buffers: while tile t is multiplied, tile t + 1 is in place (its first fragments are read at the
  // end of the step) and tile t + 2 is written; tile t + 3 is on its way from memory in registers.
  fetch(0);
  stash(0);
  if (ntiles > 1) {
    fetch(1);
    stash(1);
  }
  if (ntiles > 2) fetch(2);
  __syncthreads();

  f32x16 acc[2][2][2];  // [set][sub-tile][query half]
  bf16x8 af[2][2];      // [k-step parity][sub-tile]
  af[0][0] = *reinterpret_cast<const bf16x8*>(frag_ptr(0));
  af[0][1] = *reinterpret_cast<const bf16x8*>(frag_ptr(0) + 32 * kQsLd);
  int buf = 0;  // t % 3
  // step t: the MFMAs of tile t into set XS, the scan of tile t - 1 in the other set
  auto tile = [&](int t, auto XS_, auto SCAN_) {
    constexpr int XS = decltype(XS_)::value;
    constexpr bool SCAN = decltype(SCAN_)::value;
    const int buf1 = buf == 2 ? 0 : buf + 1, buf2 = buf1 == 2 ? 0 : buf1 + 1;
    if (t + 2 < ntiles) stash(buf2);  // fetched a step ago; the buffer's last reads (tile t - 1) were before the barrier
    if (t + 3 < ntiles) fetch(t + 3);
    const float b0 = best[0], b1 = best[1];
    // (past the last tile the fragment reads at the end of the step fetch stale rows that nothing uses)
    qs_tile_step<F16, true, SCAN, 0>(acc[XS], acc[1 - XS], af, frag_ptr(buf), frag_ptr(buf1), bfrag, best, pos);
    if (best[0] != b0) btile[0] = t - 1;
    if (best[1] != b1) btile[1] = t - 1;
    buf = buf1;
    __syncthreads();
  };
  auto last_scan = [&](auto YS_) {
    constexpr int YS = decltype(YS_)::value;
    const float b0 = best[0], b1 = best[1];
    qs_tile_step<F16, false, true, 0>(acc[1 - YS], acc[YS], af, nullptr, nullptr, bfrag, best, pos);
    if (best[0] != b0) btile[0] = ntiles - 1;
    if (best[1] != b1) btile[1] = ntiles - 1;
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  tile(0, I0{}, std::false_type{});
  int t = 1;
  for (; t + 1 < ntiles; t += 2) {
    tile(t, I1{}, std::true_type{});
    tile(t + 1, I0{}, std::true_type{});
  }
  if (t < ntiles) {
    tile(t, I1{}, std::true_type{});
    last_scan(I1{});
  } else {
    last_scan(I0{});
  }
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    int idx = btile[ni] * 64 + pos[ni] + 4 * (l >> 5);
    float b = best[ni];
    if (b == -INFINITY) idx = 0x7fffffff;  // nothing seen (only NaN or -inf scores): handled below
    const float ob = __shfl_xor(b, 32);
    const int oi = __shfl_xor(idx, 32);
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ob > b || (ob == b && oi < idx))) {
      b = ob;
      idx = oi;
    }
    const int i = i0 + ni * 32 + (l & 31);
    if (l < 32 && i < Sq) hash_out[int64_t(h) * Sq + i] = idx == 0x7fffffff ? 0 : idx;
  }
}

}  // namespace fm

extern "C" int fm_project(const void* A, const void* K, float* Y, int H, int C, int N, int d,
                          int64_t ldy, int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 0 && C >= 1 && N >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG,
             "fm_project: H=%d C=%d N=%d d=%d", H, C, N, d);
  FM_REQUIRE(ldy >= N && ldy < (int64_t(1) << 29), FM_ERR_ARG, "fm_project: ldy=%lld, N=%d", (long long)ldy, N);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_project: dtype=%d", dtype);
  if (H == 0) return FM_OK;
  FM_REQUIRE(A && K && Y, FM_ERR_ARG, "fm_project: null pointer");
  FM_REQUIRE(H <= 65535, FM_ERR_UNSUPPORTED, "fm_project: H=%d > 65535", H);
  hipStream_t st = as_stream(stream);
  const bool h16 = dtype == FM_BF16 || dtype == FM_F16;  // 16-bit elements: MFMA kernels
  if (h16 && d == 128) {
    constexpr int kBT = 1, kKT = 4;  // 32 buckets per wave, 128 keys per step: 512 contiguous bytes per row and step
    constexpr int kSlab = 4 * 32 * kBT, kKeys = 32 * kKT;
    FM_REQUIRE(ceil_div(C, kSlab) <= 65535, FM_ERR_UNSUPPORTED, "fm_project: C too large");
    // enough key ranges for ~4 workgroups per CU, each at least 8 steps long
    const int64_t n_steps = ceil_div(N, kKeys);
    const int64_t slabs = int64_t(ceil_div(C, kSlab)) * H;
    int64_t ranges = std::max<int64_t>(1, std::min<int64_t>(ceil_div(1024, slabs), ceil_div(n_steps, 8)));
    const int steps_per_wg = int(ceil_div(n_steps, ranges));
    ranges = ceil_div(n_steps, steps_per_wg);
    const dim3 grid = dim3(unsigned(ranges), unsigned(ceil_div(C, kSlab)), unsigned(H));
    if (dtype == FM_F16)
      hipLaunchKernelGGL((project_stream_bf16_d128_kernel<kBT, kKT, true>), grid, dim3(256), 0, st, (const bf16_t*)A,
                         (const bf16_t*)K, Y, C, N, ldy, steps_per_wg);
    else
      hipLaunchKernelGGL((project_stream_bf16_d128_kernel<kBT, kKT, false>), grid, dim3(256), 0, st, (const bf16_t*)A,
                         (const bf16_t*)K, Y, C, N, ldy, steps_per_wg);
  } else if (h16 && d % 16 == 0) {
    FM_REQUIRE(ceil_div(C, 128) <= 65535, FM_ERR_UNSUPPORTED, "fm_project: C too large");
    size_t lds = std::max(size_t(2) * 128 * (d + 8) * sizeof(bf16_t), size_t(128) * kProjYLd * sizeof(float));
    FM_ALLOW_LDS(project_bf16_kernel<false>, 2 * 128 * (FM_MAX_D + 8) * sizeof(bf16_t), "fm_project: lds");
    FM_ALLOW_LDS(project_bf16_kernel<true>, 2 * 128 * (FM_MAX_D + 8) * sizeof(bf16_t), "fm_project: lds");
    dim3 grid = dim3(unsigned(ceil_div(N, 128)), unsigned(ceil_div(C, 128)), unsigned(H));
    if (dtype == FM_F16)
      hipLaunchKernelGGL(project_bf16_kernel<true>, grid, dim3(256), lds, st, (const bf16_t*)A, (const bf16_t*)K, Y, C,
                         N, d, ldy);
    else
      hipLaunchKernelGGL(project_bf16_kernel<false>, grid, dim3(256), lds, st, (const bf16_t*)A, (const bf16_t*)K, Y, C,
                         N, d, ldy);
  } else {
    size_t lds = size_t(64) * (d + 1) * sizeof(float);
    dim3 grid = dim3(unsigned(ceil_div(N, 64)), unsigned(H));
    FM_ALLOW_LDS(project_generic_kernel<float>, 64 * (FM_MAX_D + 1) * 4, "fm_project: lds");
    FM_ALLOW_LDS(project_generic_kernel<bf16_t>, 64 * (FM_MAX_D + 1) * 4, "fm_project: lds");
    FM_ALLOW_LDS(project_generic_kernel<f16_t>, 64 * (FM_MAX_D + 1) * 4, "fm_project: lds");
    if (dtype == FM_F32)
      hipLaunchKernelGGL(project_generic_kernel<float>, grid, dim3(256), lds, st, (const float*)A,
                         (const float*)K, Y, C, N, d, ldy);
    else if (dtype == FM_BF16)
      hipLaunchKernelGGL(project_generic_kernel<bf16_t>, grid, dim3(256), lds, st,
                         (const bf16_t*)A, (const bf16_t*)K, Y, C, N, d, ldy);
    else
      hipLaunchKernelGGL(project_generic_kernel<f16_t>, grid, dim3(256), lds, st,
                         (const f16_t*)A, (const f16_t*)K, Y, C, N, d, ldy);
  }
  return launch_status("fm_project");
}

extern "C" int fm_qhash(const void* A, const void* q, int32_t* hash_out, float* scores_out, int H,
                        int C, int Sq, int d, int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 0 && C >= 1 && Sq >= 0 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG,
             "fm_qhash: H=%d C=%d Sq=%d d=%d", H, C, Sq, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_qhash: dtype=%d", dtype);
  if (H == 0 || Sq == 0) return FM_OK;
  FM_REQUIRE(A && q && hash_out, FM_ERR_ARG, "fm_qhash: null pointer");
  FM_REQUIRE(H <= 65535, FM_ERR_UNSUPPORTED, "fm_qhash: H=%d > 65535", H);
  hipStream_t st = as_stream(stream);
  const bool h16 = dtype == FM_BF16 || dtype == FM_F16;  // 16-bit elements: MFMA kernels
  if (h16 && d == 128 && !scores_out) {
    dim3 grid = dim3(unsigned(ceil_div(Sq, 512)), unsigned(H));
    if (dtype == FM_F16)
      hipLaunchKernelGGL(qhash_stream_kernel<true>, grid, dim3(512), 0, st, (const bf16_t*)A, (const bf16_t*)q,
                         hash_out, C, Sq);
    else
      hipLaunchKernelGGL(qhash_stream_kernel<false>, grid, dim3(512), 0, st, (const bf16_t*)A, (const bf16_t*)q,
                         hash_out, C, Sq);
  } else if (h16 && d % 16 == 0) {
    size_t lds = size_t(2) * 128 * (d + 8) * sizeof(bf16_t);
    FM_ALLOW_LDS(qhash_bf16_kernel<false>, 2 * 128 * (FM_MAX_D + 8) * sizeof(bf16_t), "fm_qhash: lds");
    FM_ALLOW_LDS(qhash_bf16_kernel<true>, 2 * 128 * (FM_MAX_D + 8) * sizeof(bf16_t), "fm_qhash: lds");
    dim3 grid = dim3(unsigned(ceil_div(Sq, 128)), unsigned(H));
    if (dtype == FM_F16)
      hipLaunchKernelGGL(qhash_bf16_kernel<true>, grid, dim3(256), lds, st, (const bf16_t*)A, (const bf16_t*)q,
                         hash_out, scores_out, C, Sq, d);
    else
      hipLaunchKernelGGL(qhash_bf16_kernel<false>, grid, dim3(256), lds, st, (const bf16_t*)A, (const bf16_t*)q,
                         hash_out, scores_out, C, Sq, d);
  } else {
    size_t lds = size_t(64) * (d + 1) * sizeof(float);
    FM_ALLOW_LDS(qhash_generic_kernel<float>, 64 * (FM_MAX_D + 1) * 4, "fm_qhash: lds");
    FM_ALLOW_LDS(qhash_generic_kernel<bf16_t>, 64 * (FM_MAX_D + 1) * 4, "fm_qhash: lds");
    FM_ALLOW_LDS(qhash_generic_kernel<f16_t>, 64 * (FM_MAX_D + 1) * 4, "fm_qhash: lds");
    dim3 grid = dim3(unsigned(ceil_div(Sq, 64)), unsigned(H));
    if (dtype == FM_F32)
      hipLaunchKernelGGL(qhash_generic_kernel<float>, grid, dim3(256), lds, st, (const float*)A,
                         (const float*)q, hash_out, scores_out, C, Sq, d);
    else if (dtype == FM_BF16)
      hipLaunchKernelGGL(qhash_generic_kernel<bf16_t>, grid, dim3(256), lds, st, (const bf16_t*)A,
                         (const bf16_t*)q, hash_out, scores_out, C, Sq, d);
    else
      hipLaunchKernelGGL(qhash_generic_kernel<f16_t>, grid, dim3(256), lds, st, (const f16_t*)A,
                         (const f16_t*)q, hash_out, scores_out, C, Sq, d);
  }
  return launch_status("fm_qhash");
}
