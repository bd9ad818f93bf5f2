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
// the bucket rows of A through a double-buffered LDS tile of 64 rows.  One query
// per lane column: the running maximum and its position are per-lane registers,
// updated with three VALU instructions per accumulator register (compare, select
// value, select the row number as an inline constant); buckets arrive in
// ascending order, so "strictly greater" keeps the first maximum.  The loop is
// software-pipelined in half tiles: while the MFMAs of one 32-row sub-tile run,
// the finished sub-tile before it is scanned and the A fragments of the next are
// read from LDS.  On this hardware VALU and MFMA time of a SIMD add up rather
// than overlap, so the scan costs about as much as the products.  The scores are
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

// position of accumulator register R of the 32-row sub-tile MI inside the 64-row tile, for
// lanes 0..31 (lanes 32..63 hold the rows 4 further down)
constexpr int qs_row(int MI, int R) { return MI * 32 + 8 * (R >> 2) + (R & 3); }

// Elements E and E+1 (of 32: query column half E/16, register E%16) of a finished sub-tile.
// Register 0 of each half goes through plain C++ so that the compiler, which cannot see into the
// asm, places the wait states a read of a fresh MFMA result needs; the MFMA that produced a half
// was issued before those of anything read later.
template <int MI, int E>
__device__ __forceinline__ void argmax_pair(float (&best)[2], int (&pos)[2], const f32x16 (&acc)[2]) {
  constexpr int NI = E >> 4, R = E & 15;
  if constexpr (R == 0) {
    const bool gt = acc[NI][0] > best[NI];
    best[NI] = gt ? acc[NI][0] : best[NI];
    pos[NI] = gt ? qs_row(MI, 0) : pos[NI];
  } else {
    argmax_step<qs_row(MI, R)>(best[NI], pos[NI], acc[NI][R]);
  }
  argmax_step<qs_row(MI, R + 1)>(best[NI], pos[NI], acc[NI][R + 1]);
}

// One half step of the pipeline: the 16 MFMAs of sub-tile (MM) of one tile, with the running
// argmax over the finished sub-tile (ME) of the tile before it and the LDS reads of the next
// half step's A fragments spread between them.  sched_barrier pins the interleaving: an MFMA
// keeps the matrix pipe busy for 32 cycles, the six VALU instructions behind it take 24.
template <bool F16, int ME, bool MFMA, bool PREFETCH, int I>
__device__ __forceinline__ void qs_half_step(f32x16 (&accM)[2], const f32x16 (&accE)[2], const bf16x8 (&af)[8],
                                             bf16x8 (&af_next)[8], const bf16_t* next_lds,
                                             const bf16x8 (&bfrag)[2][8], float (&best)[2], int (&pos)[2]) {
  if constexpr (I < 16) {
    constexpr int ks = I >> 1, ni = I & 1;
    if constexpr (MFMA) {
      if constexpr (ks == 0) {
        f32x16 z;
#pragma unroll
        for (int r = 0; r < 16; ++r) z[r] = 0.f;
        accM[ni] = mfma32<F16>(af[ks], bfrag[ni][ks], z);
      } else {
        accM[ni] = mfma32<F16>(af[ks], bfrag[ni][ks], accM[ni]);
      }
    }
    if constexpr (PREFETCH && ni == 0) af_next[ks] = *reinterpret_cast<const bf16x8*>(next_lds + ks * 16);
    argmax_pair<ME, 2 * I>(best, pos, accE);
    __builtin_amdgcn_sched_barrier(0);
    qs_half_step<F16, ME, MFMA, PREFETCH, I + 1>(accM, accE, af, af_next, next_lds, bfrag, best, pos);
  }
}

template <bool F16>
__global__ __launch_bounds__(512) void qhash_stream_kernel(const bf16_t* __restrict__ A,
                                                           const bf16_t* __restrict__ q,
                                                           int32_t* __restrict__ hash_out, int C, int Sq) {
  __shared__ __attribute__((aligned(16))) bf16_t sA[2][64 * kQsLd];
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
  // LDS address of this lane's A fragment 0 of sub-tile mi of the tile in buffer buf
  auto frag_ptr = [&](int buf, int mi) -> const bf16_t* {
    return &sA[buf][(mi * 32 + (l & 31)) * kQsLd + (l >> 5) * 8];
  };
  fetch(0);
  stash(0);
  if (ntiles > 1) {
    fetch(1);
    stash(1);
  }
  __syncthreads();

  // Pipeline over half steps: sub-tile 0 of tile t+1 is multiplied while sub-tile 1 of tile t
  // is scanned, and the other way round; tile t+2 travels global -> registers -> LDS meanwhile.
  f32x16 acc[2][2];
  bf16x8 af0[8], af1[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) af0[ks] = *reinterpret_cast<const bf16x8*>(frag_ptr(0, 0) + ks * 16);
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.f;
    acc[0][0] = mfma32<F16>(af0[ks], bfrag[0][ks], ks ? acc[0][0] : z);
    acc[0][1] = mfma32<F16>(af0[ks], bfrag[1][ks], ks ? acc[0][1] : z);
    af1[ks] = *reinterpret_cast<const bf16x8*>(frag_ptr(0, 1) + ks * 16);
  }
  for (int t = 0; t < ntiles; ++t) {
    const bool more = t + 1 < ntiles;
    if (t + 2 < ntiles) fetch(t + 2);
    {
      const float b0 = best[0], b1 = best[1];
      if (more)
        qs_half_step<F16, 0, true, true, 0>(acc[1], acc[0], af1, af0, frag_ptr((t + 1) & 1, 0), bfrag, best, pos);
      else
        qs_half_step<F16, 0, true, false, 0>(acc[1], acc[0], af1, af0, nullptr, bfrag, best, pos);
      if (best[0] != b0) btile[0] = t;
      if (best[1] != b1) btile[1] = t;
    }
    {
      const float b0 = best[0], b1 = best[1];
      if (more)
        qs_half_step<F16, 1, true, true, 0>(acc[0], acc[1], af0, af1, frag_ptr((t + 1) & 1, 1), bfrag, best, pos);
      else
        qs_half_step<F16, 1, false, false, 0>(acc[0], acc[1], af0, af1, nullptr, bfrag, best, pos);
      if (best[0] != b0) btile[0] = t;
      if (best[1] != b1) btile[1] = t;
    }
    if (t + 2 < ntiles) stash(t & 1);  // the buffer of tile t: its last reads were a tile ago
    __syncthreads();
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
