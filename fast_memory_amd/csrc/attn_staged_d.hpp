// bf16 / fp16 bucket-gathered attention forward with a bucket's rows staged in LDS, for the head dimensions
// beside 128 that the MFMA path takes: D = 64 and D = 256 (triton_kernel.py:137-272; the reference kernel is
// generic in d_head, triton_kernel.py:141-147).  D = 128 has kernels of its own (attn_staged.hpp, attn_ring.hpp);
// this is their arithmetic and operand layout with every extent a function of D, and instantiated for 128
// too it gives the same bits (a test compares the two).
//
// One workgroup (4 waves) per work item (up to 64 queries of one bucket); wave w carries queries 16w .. 16w+15
// over ALL keys of the bucket, so the waves never merge.  Tiles of 64 keys go global -> registers (in flight
// during the previous tile's arithmetic) -> LDS: K rows as they are (row stride D + 8 elements: the 16 rows a
// lane group reads start 4 banks apart), V transposed on the way ( Vt[dim][key], stride 72 ), its key columns in
// the order in which the score registers hold the keys.
//   S^T = K.Q^T    v_mfma_f32_16x16x32, D / 32 contraction steps; lane (g,c) gets the scores of keys 4g..4g+3
//                  of each 16-key tile for query c
//   O^T += Vt.P^T  the same instruction over 32 keys, D / 16 output tiles; lane (g,c) holds
//                  O[query c][16t + 4g .. 16t + 4g + 3]
// Softmax as in the reference kernel (triton_kernel.py:248-263): base 2 with sm_scale*log2(e), fp32 running
// maximum and denominator, denominator from unrounded p, p rounded to the input type before P.V.
// Rows are addressed by 32-bit byte offsets: N * 2 D < 2^32 (checked by the host).
#pragma once
#include <type_traits>

#include "attn_staged.hpp"

namespace fm {

template <int D>
struct StagedD {
  static constexpr int kCPR = D / 8;                  // 16-byte chunks per row
  static constexpr int kKld = D + 8;                  // K tile row stride in LDS (elements)
  static constexpr int kVld = 72;                     // Vt row stride (elements): 64 keys + 8
  static constexpr int kSteps = D / 32;               // contraction steps of S^T = K.Q^T
  static constexpr int kOT = D / 16;                  // 16-dim output tiles
  static constexpr int kKLoads = kCPR / 4;            // K chunks a thread stages per tile (64 rows x kCPR / 256)
  static constexpr int kKRowStep = 256 / kCPR;        // rows between a thread's K chunks
  static constexpr int kVUnits = kCPR >= 16 ? kCPR / 16 : 1;  // (4 keys x 1 chunk) units a thread transposes per tile
  static constexpr int kRowShift = D == 64 ? 7 : D == 128 ? 8 : 9;  // log2 of a row's bytes
  static constexpr size_t kLdsBytes = size_t(64 * kKld + D * kVld) * sizeof(bf16_t);
  static_assert(D == 64 || D == 128 || D == 256, "head dimensions of the MFMA path");
};

template <int D, bool F16>
__device__ __forceinline__ void attend_staged_d(const bf16_t* __restrict__ Qb, const int* __restrict__ q_rows, int n_q,
                                                const bf16_t* __restrict__ Kb, const bf16_t* __restrict__ Vb,
                                                const int32_t* __restrict__ idx, int cnt, int N, float scale2,
                                                bf16_t* __restrict__ Ob, float* __restrict__ Lb,
                                                bf16_t* __restrict__ st_lds) {
  using S = StagedD<D>;
  bf16_t* const sK = st_lds;
  bf16_t* const sVt = st_lds + 64 * S::kKld;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int g = l >> 4, c = l & 15;
  const int ntiles = (cnt + 63) >> 6;

  // ---- this lane's query (column c of wave w's tile) ----
  const int jq = 16 * w + c;
  const bool q_ok = jq < n_q;
  const bool wave_on = 16 * w < n_q;
  const int64_t qrow = q_ok ? q_rows[jq] : 0;
  uint4 qf[S::kSteps];
  {
    const uint4* pq = reinterpret_cast<const uint4*>(Qb + qrow * D + 8 * g);
#pragma unroll
    for (int s = 0; s < S::kSteps; ++s) qf[s] = q_ok ? pq[4 * s] : make_uint4(0, 0, 0, 0);
  }
  f32x4 O[S::kOT];
#pragma unroll
  for (int t = 0; t < S::kOT; ++t) O[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;

  // ---- staging: key rows of tile t are idx[64t + lane] in every wave ----
  auto rows_of = [&](int t) -> int {
    const int kp = t * 64 + l;
    return kp < cnt ? idx[kp] : 0;  // positions past the end read row 0: their scores are masked, their p is 0
  };
  // K: chunk tid % kCPR of rows tid / kCPR + kKRowStep u.  V: keys 4j .. 4j+3 (j = lane % 16) of chunk
  // 4 wave + lane / 16 (+ 16 per further unit); with D = 64 only the chunks below 8 exist (waves 0 and 1).
  const int kchunk = tid % S::kCPR, krow = tid / S::kCPR;
  const int vj = l & 15, vc = 4 * w + (l >> 4);
  const bool v_on = vc < S::kCPR;
  // The staging registers are separate variables (tk0 .. tk7 for up to eight K chunks, tvUE for key E of unit
  // U): declared as arrays they are placed in scratch memory, and every access becomes a memory instruction
  // whose wait also waits for the tile's loads.  Those beyond what D needs are never touched.
  uint4 tk0, tk1, tk2, tk3, tk4, tk5, tk6, tk7;
  uint4 tv00, tv01, tv02, tv03, tv10, tv11, tv12, tv13;
  const char* Kc = reinterpret_cast<const char*>(Kb) + 16 * kchunk;
  const char* Vc = reinterpret_cast<const char*>(Vb) + 16 * vc;
#define FM_STD_K(u) \
  if constexpr (S::kKLoads > u) \
    tk##u = *reinterpret_cast<const uint4*>(Kc + (uint32_t(__shfl(rows_, krow + S::kKRowStep * u)) << S::kRowShift))
#define FM_STD_V(e)                                                                                        \
  do {                                                                                                     \
    const uint32_t off_ = uint32_t(__shfl(rows_, 4 * vj + e)) << S::kRowShift;                             \
    tv0##e = v_on ? *reinterpret_cast<const uint4*>(Vc + off_) : make_uint4(0, 0, 0, 0);                   \
    if constexpr (S::kVUnits > 1) tv1##e = *reinterpret_cast<const uint4*>(Vc + off_ + 256);               \
  } while (0)
#define FM_STD_LOAD_TILE(rows_raw)                    \
  do {                                                \
    const int rows_ = min(max((rows_raw), 0), N - 1); \
    FM_STD_K(0);                                      \
    FM_STD_K(1);                                      \
    FM_STD_K(2);                                      \
    FM_STD_K(3);                                      \
    FM_STD_K(4);                                      \
    FM_STD_K(5);                                      \
    FM_STD_K(6);                                      \
    FM_STD_K(7);                                      \
    FM_STD_V(0);                                      \
    FM_STD_V(1);                                      \
    FM_STD_V(2);                                      \
    FM_STD_V(3);                                      \
  } while (0)
  // keys 4j..4j+3 of the tile: 32-key half j/8, key tile (j/4)%2 of the half, lane group j%4
  const int pos0 = 32 * (vj >> 3) + 8 * (vj & 3) + 4 * ((vj >> 2) & 1);
  auto vt_pair = [&](int chunk, uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, int e) {
    uint2 lo, hi;  // dims e (low halves) and e + 1 (high halves) of the four keys
    lo.x = (a0 & 0xffffu) | (a1 << 16);
    lo.y = (a2 & 0xffffu) | (a3 << 16);
    hi.x = (a0 >> 16) | (a1 & 0xffff0000u);
    hi.y = (a2 >> 16) | (a3 & 0xffff0000u);
    *reinterpret_cast<uint2*>(&sVt[(8 * chunk + e) * S::kVld + pos0]) = lo;
    *reinterpret_cast<uint2*>(&sVt[(8 * chunk + e + 1) * S::kVld + pos0]) = hi;
  };
#define FM_STD_STASH_K(u) \
  if constexpr (S::kKLoads > u) *reinterpret_cast<uint4*>(&sK[(krow + S::kKRowStep * u) * S::kKld + kchunk * 8]) = tk##u
#define FM_STD_STASH_TILE()                                   \
  do {                                                        \
    FM_STD_STASH_K(0);                                        \
    FM_STD_STASH_K(1);                                        \
    FM_STD_STASH_K(2);                                        \
    FM_STD_STASH_K(3);                                        \
    FM_STD_STASH_K(4);                                        \
    FM_STD_STASH_K(5);                                        \
    FM_STD_STASH_K(6);                                        \
    FM_STD_STASH_K(7);                                        \
    if (v_on) {                                               \
      vt_pair(vc, tv00.x, tv01.x, tv02.x, tv03.x, 0);         \
      vt_pair(vc, tv00.y, tv01.y, tv02.y, tv03.y, 2);         \
      vt_pair(vc, tv00.z, tv01.z, tv02.z, tv03.z, 4);         \
      vt_pair(vc, tv00.w, tv01.w, tv02.w, tv03.w, 6);         \
      if constexpr (S::kVUnits > 1) {                         \
        vt_pair(vc + 16, tv10.x, tv11.x, tv12.x, tv13.x, 0);  \
        vt_pair(vc + 16, tv10.y, tv11.y, tv12.y, tv13.y, 2);  \
        vt_pair(vc + 16, tv10.z, tv11.z, tv12.z, tv13.z, 4);  \
        vt_pair(vc + 16, tv10.w, tv11.w, tv12.w, tv13.w, 6);  \
      }                                                       \
    }                                                         \
  } while (0)

  auto compute_tile = [&](int t) {
    const int kp0 = t * 64;
    // ---- S^T for the four 16-key tiles (contraction step outermost: consecutive MFMAs go to different
    // accumulators) ----
    f32x4 s[4];
#pragma unroll
    for (int st = 0; st < S::kSteps; ++st) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const uint4 a = *reinterpret_cast<const uint4*>(&sK[(kt * 16 + c) * S::kKld + 8 * g + 32 * st]);
        s[kt] = Mma<F16>::m16(a, qf[st], st == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[kt]);
      }
    }
    {  // (a branch follows: see mfma_settle in mma16.hpp)
      f32x4(&s1)[1][4] = reinterpret_cast<f32x4(&)[1][4]>(s);
      mfma_settle_scores<1>(s1);
    }
    if (kp0 + 64 > cnt) {  // the bucket's last, ragged tile
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (kp0 + 16 * kt + 4 * g + r >= cnt) s[kt][r] = -INFINITY;
    }
    // ---- online softmax; the four lane groups of a column share the query ----
    float mx = st_max3(s[0][0], s[0][1], s[0][2]);
    mx = st_max3(mx, s[0][3], s[1][0]);
    mx = st_max3(mx, s[1][1], s[1][2]);
    mx = st_max3(mx, s[1][3], s[2][0]);
    mx = st_max3(mx, s[2][1], s[2][2]);
    mx = st_max3(mx, s[2][3], s[3][0]);
    mx = st_max3(mx, s[3][1], s[3][2]);
    mx = st_max_lane_groups(st_max(mx, s[3][3])) * scale2;  // scale2 > 0: scaling commutes with the maximum
    const float m_new = fmaxf(m, mx);
    const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;  // a query that sees no key yet
    if (__any(m_new != m)) {
      const float alpha = __builtin_amdgcn_exp2f(m - m_sub);
      lsum *= alpha;
#pragma unroll
      for (int t8 = 0; t8 < S::kOT; ++t8) {
        O[t8][0] *= alpha;
        O[t8][1] *= alpha;
        O[t8][2] *= alpha;
        O[t8][3] *= alpha;
      }
      m = m_new;
    }
    uint4 pf[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      float p[8];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        p[r] = __builtin_amdgcn_exp2f(fmaf(s[2 * h][r], scale2, -m_sub));
        p[4 + r] = __builtin_amdgcn_exp2f(fmaf(s[2 * h + 1][r], scale2, -m_sub));
      }
#pragma unroll
      for (int r = 0; r < 8; ++r) lsum += p[r];
      pf[h] = make_uint4(Mma<F16>::pack2(p[0], p[1]), Mma<F16>::pack2(p[2], p[3]), Mma<F16>::pack2(p[4], p[5]),
                         Mma<F16>::pack2(p[6], p[7]));
    }
    // ---- O^T += Vt.P^T (32-key half outermost) ----
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int t8 = 0; t8 < S::kOT; ++t8) {
        const uint4 a = *reinterpret_cast<const uint4*>(&sVt[(16 * t8 + c) * S::kVld + 8 * g + 32 * h]);
        O[t8] = Mma<F16>::m16(a, pf[h], O[t8]);
      }
    }
  };

  // one tile buffer: the registers hold tile t + 1 while tile t is computed, two barriers per tile; the list
  // rows of tile t + 2 are requested while tile t is computed (two registers in turn)
  int rows_a = 0, rows_b = 0;
  if (ntiles > 0) {
    FM_STD_LOAD_TILE(rows_of(0));
    rows_a = rows_of(1);
    FM_STD_STASH_TILE();
  }
  // (the wait for the query fragments here, in front of the loop, not in front of every tile's first MFMA)
#pragma unroll
  for (int s = 0; s < S::kSteps; ++s) asm volatile("" ::"v"(qf[s].x), "v"(qf[s].y), "v"(qf[s].z), "v"(qf[s].w));
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const bool more = t + 1 < ntiles;
    if (more) {
      const int use = (t & 1) ? rows_b : rows_a;
      const int nxt = rows_of(t + 2);
      if (t & 1)
        rows_a = nxt;
      else
        rows_b = nxt;
      FM_STD_LOAD_TILE(use);  // lands while this tile is computed
    }
    if (wave_on) compute_tile(t);
    __syncthreads();  // every wave has read tile t
    if (more) FM_STD_STASH_TILE();
    __syncthreads();  // tile t + 1 is in place
  }
#undef FM_STD_K
#undef FM_STD_V
#undef FM_STD_LOAD_TILE
#undef FM_STD_STASH_K
#undef FM_STD_STASH_TILE

  // ---- finish: lane (g,c) holds dims 16t + 4g + r of query c ----
  float ltot = lsum + __shfl_xor(lsum, 16);
  ltot += __shfl_xor(ltot, 32);
  const bool empty = (m == -INFINITY);  // the query saw no key at all
  const float inv = empty ? 0.f : 1.f / ltot;
  if (q_ok) {
    bf16_t* po = Ob + qrow * D + 4 * g;
#pragma unroll
    for (int t8 = 0; t8 < S::kOT; ++t8) {
      uint2 o;
      o.x = Mma<F16>::pack2(O[t8][0] * inv, O[t8][1] * inv);
      o.y = Mma<F16>::pack2(O[t8][2] * inv, O[t8][3] * inv);
      *reinterpret_cast<uint2*>(po + 16 * t8) = o;
    }
    if (g == 0) Lb[qrow] = empty ? -FLT_MAX : (m + __builtin_amdgcn_logf(ltot)) * kLn2;
  }
}

}  // namespace fm
