// bf16 / fp16 bucket-gathered attention forward for head dimension 128 (gfx950) with a bucket's rows
// staged in LDS (triton_kernel.py:137-272).  The kernel of every launch that has work items enough
// to fill the chip or buckets with many queries (the register-gather kernel of attn_mfma.hip keeps
// the launches with few, small items): from the HBM-bound shapes (16 queries per bucket over a
// million keys) to the shape of the reference's own performance harness (triton_kernel.py:507-528,
// 128 queries per bucket), where the arithmetic is the larger part.
//
// Work decomposition.  One workgroup (4 waves) per work item (up to 64 queries of one bucket), or
// per two consecutive items of a bucket; wave w carries 16 (or 32) of the queries over ALL keys of
// the bucket, so the waves never merge.  The bucket's rows are gathered once per workgroup: tiles
// of 64 keys go global -> registers (in flight during the previous tile's arithmetic) -> LDS, V
// transposed on the way ( Vt[d][key] ), and every wave reads its MFMA operands from there.
// 154 registers and 35 KiB of LDS per workgroup with one item (three workgroups per CU), 251 and
// 70 KiB with two (two per CU): one wave's softmax runs under another's MFMAs.
//   S^T = K.Q^T    v_mfma_f32_16x16x32_bf16, A = 16 K rows from LDS, B = Q^T fragments resident
//                  in registers; lane (g,c) gets the scores of keys 4g..4g+3 of each 16-key
//                  tile for query c.
//   O^T += Vt.P^T  same instruction over 32 keys: the scores of key tiles 2h and 2h+1 in a lane
//                  are the B operand if contraction slot 8g+e stands for key 4g+e of tile 2h
//                  (e < 4) or key 4g+e-4 of tile 2h+1; Vt is stored with its key columns in
//                  that order, so neither P nor V is shuffled.  Lane (g,c) holds
//                  O[query c][16t + 4g .. 16t + 4g + 3], t = 0..7.
// Softmax as in the reference kernel (triton_kernel.py:248-263): base 2 with sm_scale*log2(e),
// fp32 running max and denominator, denominator from unrounded p, p rounded to the input type before P.V.
//
// Roofline: HBM for the algorithmic bytes (cnt*(2*128*2+4) per bucket), MFMA for 4*128 flops per
// query-key pair; at 128 queries per bucket the two are within a factor of three of each other.
#pragma once
#include "mma16.hpp"

namespace fm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kSD = 128;    // head dimension
constexpr int kSK = 64;     // keys per tile
constexpr int kSKld = 136;  // K tile row stride in LDS (elements): rows 16 banks apart
constexpr int kSVld = 72;   // Vt row stride in LDS (elements): 64 keys + 8

__device__ __forceinline__ uint32_t st_pack_bf16(float lo, float hi) {
  f32x2 x = {lo, hi};
  bf16x2 y = __builtin_convertvector(x, bf16x2);  // v_cvt_pk_bf16_f32, round to nearest even
  return *reinterpret_cast<uint32_t*>(&y);
}

// Maxima as single instructions: fmaxf() first quiets each operand with an instruction of its own,
// which the MFMA results here do not need.
__device__ __forceinline__ float st_max(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float st_max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// Maximum over the four lanes l, l^16, l^32, l^48 with the gfx950 row swaps (no LDS round trip):
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its
// second, v_permlane32_swap the upper half of the first with the lower half of the second; with
// both operands equal, each lane finds its own value in one result and its partner's in the other.
__device__ __forceinline__ float st_max_lane_groups(float x) {
  const unsigned u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned v = __float_as_uint(st_max(__uint_as_float(a[0]), __uint_as_float(a[1])));
  const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return st_max(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ bf16x8 st_as_bf16x8(uint4 u) {
  union {
    uint4 u;
    bf16x8 b;
  } x;
  x.u = u;
  return x.b;
}


constexpr size_t kStagedTileBytes = size_t(kSK * kSKld + kSD * kSVld) * sizeof(bf16_t);

// The staged attention of one work item: n_q queries (rows q_rows[0..n_q) of Qb / Ob / Lb; q_rows may
// point to global memory or LDS) over the cnt keys idx[0..cnt) of one bucket.  Called by all 256
// threads of a workgroup; lds holds NQW tile buffers of kStagedTileBytes.  NQW = 16-query tiles per
// wave: the workgroup takes up to 64 * NQW queries.
// BIGN: rows are addressed by 64-bit byte offsets (memories of more than 2^24 keys; a few more address
// instructions per tile), otherwise by 32-bit ones (N * 256 B < 4 GiB).
template <int NQW, bool F16 = false, bool BIGN = false>
__device__ __forceinline__ void attend_staged(
    const bf16_t* __restrict__ Qb, const int* __restrict__ q_rows, int n_q, const bf16_t* __restrict__ Kb,
    const bf16_t* __restrict__ Vb, const int32_t* __restrict__ idx, int cnt, int N, float scale2,
    bf16_t* __restrict__ Ob, float* __restrict__ Lb, bf16_t* __restrict__ st_lds) {
  // NQW tile buffers (K rows, then Vt) each: with two, tile t + 1 is written while tile t is read
  constexpr int NBUF = NQW;
  bf16_t* const sK = st_lds;
  bf16_t* const sVt = st_lds + NBUF * kSK * kSKld;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int g = l >> 4, c = l & 15;
  const int ntiles = (cnt + kSK - 1) / kSK;

  // ---- this lane's queries (column c of each of wave w's NQW tiles) ----
  const int nqt_w = min(max((n_q - 16 * NQW * w + 15) >> 4, 0), NQW);  // tiles of this wave that hold queries
  const bool wave_on = nqt_w > 0;
  bool q_ok[NQW];
  int64_t qrow[NQW];
  uint4 qf[NQW][4];
#pragma unroll
  for (int qt = 0; qt < NQW; ++qt) {
    const int jq = 16 * (NQW * w + qt) + c;
    q_ok[qt] = jq < n_q;
    qrow[qt] = q_ok[qt] ? q_rows[jq] : 0;
    const uint4* pq = reinterpret_cast<const uint4*>(Qb + qrow[qt] * kSD + 8 * g);
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[qt][s] = q_ok[qt] ? pq[4 * s] : make_uint4(0, 0, 0, 0);
  }
  f32x4 O[NQW][8];
  float m[NQW], lsum[NQW];
#pragma unroll
  for (int qt = 0; qt < NQW; ++qt) {
    m[qt] = -INFINITY;
    lsum[qt] = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) O[qt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- tiles: key rows of tile t are idx[64t + lane] of every wave ----
  // (fetched two tiles ahead and clamped only when used: nothing waits for the fetch in between)
  auto rows_of = [&](int t) -> int {
    const int kp = t * kSK + l;
    return kp < cnt ? idx[kp] : 0;
  };
  // staging registers of the next tile, as separate variables (an array here ends up in LDS):
  // K rows tid/16 + 16u, 16-byte chunk tid%16; V rows 4j..4j+3 (j = lane%16), chunk 4*wave + lane/16
  // (16 consecutive lanes then write 16 different key groups of one Vt row: every LDS bank once)
  uint4 tk0, tk1, tk2, tk3, tv0, tv1, tv2, tv3;
  const int vj = l & 15, vc = 4 * w + (l >> 4);
  const int kchunk = tid & 15, krow = tid >> 4;
  // (positions past the end of the list read row 0: their scores are masked, their p is 0)
  // (row offsets as unsigned 32-bit byte offsets from the uniform bases unless BIGN: N * 256 < 2^32, checked by the host)
  const char* Kc = reinterpret_cast<const char*>(Kb) + 16 * kchunk;
  const char* Vc = reinterpret_cast<const char*>(Vb) + 16 * vc;
  auto k_row = [&](int rows, int p) {
    if constexpr (BIGN)
      return *reinterpret_cast<const uint4*>(Kc + (uint64_t(uint32_t(__shfl(rows, p))) << 8));
    else
      return *reinterpret_cast<const uint4*>(Kc + (uint32_t(__shfl(rows, p)) << 8));
  };
  auto v_row = [&](int rows, int p) {
    if constexpr (BIGN)
      return *reinterpret_cast<const uint4*>(Vc + (uint64_t(uint32_t(__shfl(rows, p))) << 8));
    else
      return *reinterpret_cast<const uint4*>(Vc + (uint32_t(__shfl(rows, p)) << 8));
  };
#define FM_STAGED_LOAD_TILE(rows_raw)                      \
  do {                                                     \
    const int rows_ = min(max((rows_raw), 0), N - 1);      \
    tk0 = k_row(rows_, krow);                              \
    tk1 = k_row(rows_, krow + 16);                         \
    tk2 = k_row(rows_, krow + 32);                         \
    tk3 = k_row(rows_, krow + 48);                         \
    tv0 = v_row(rows_, 4 * vj);                            \
    tv1 = v_row(rows_, 4 * vj + 1);                        \
    tv2 = v_row(rows_, 4 * vj + 2);                        \
    tv3 = v_row(rows_, 4 * vj + 3);                        \
  } while (0)
  // keys 4j..4j+3 of the tile: 32-key half j/8, key tile (j/4)%2 of the half, lane group j%4
  const int pos0 = 32 * (vj >> 3) + 8 * (vj & 3) + 4 * ((vj >> 2) & 1);
  auto vt_pair = [&](bf16_t* sVt, uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, int e) {
    uint2 lo, hi;  // dims e (low halves) and e + 1 (high halves) of the four keys
    lo.x = (a0 & 0xffffu) | (a1 << 16);
    lo.y = (a2 & 0xffffu) | (a3 << 16);
    hi.x = (a0 >> 16) | (a1 & 0xffff0000u);
    hi.y = (a2 >> 16) | (a3 & 0xffff0000u);
    *reinterpret_cast<uint2*>(&sVt[(8 * vc + e) * kSVld + pos0]) = lo;
    *reinterpret_cast<uint2*>(&sVt[(8 * vc + e + 1) * kSVld + pos0]) = hi;
  };
  auto stash_tile = [&](int buf) {
    bf16_t* const bK = sK + buf * (kSK * kSKld);
    bf16_t* const bV = sVt + buf * (kSD * kSVld);
    *reinterpret_cast<uint4*>(&bK[(krow + 0) * kSKld + kchunk * 8]) = tk0;
    *reinterpret_cast<uint4*>(&bK[(krow + 16) * kSKld + kchunk * 8]) = tk1;
    *reinterpret_cast<uint4*>(&bK[(krow + 32) * kSKld + kchunk * 8]) = tk2;
    *reinterpret_cast<uint4*>(&bK[(krow + 48) * kSKld + kchunk * 8]) = tk3;
    vt_pair(bV, tv0.x, tv1.x, tv2.x, tv3.x, 0);
    vt_pair(bV, tv0.y, tv1.y, tv2.y, tv3.y, 2);
    vt_pair(bV, tv0.z, tv1.z, tv2.z, tv3.z, 4);
    vt_pair(bV, tv0.w, tv1.w, tv2.w, tv3.w, 6);
  };

  auto compute_tile = [&](int t, int buf) {
    const int kp0 = t * kSK;
    const bf16_t* const bK = sK + buf * (kSK * kSKld);
    const bf16_t* const bV = sVt + buf * (kSD * kSVld);
    // ---- S^T for the four 16-key tiles; an operand read from LDS serves every query tile ----
    // (contraction step outermost: consecutive MFMAs go to different accumulators, none waits for
    // the one before it)
    f32x4 s[NQW][4];
#pragma unroll
    for (int st = 0; st < 4; ++st) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const uint4 a = *reinterpret_cast<const uint4*>(&bK[(kt * 16 + c) * kSKld + 8 * g + 32 * st]);
#pragma unroll
        for (int qt = 0; qt < NQW; ++qt)
          s[qt][kt] = Mma<F16>::m16(a, qf[qt][st], st == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[qt][kt]);
      }
    }
    mfma_settle_scores<NQW>(s);  // (a branch follows: see mma16.hpp)
    if (kp0 + kSK > cnt) {  // the bucket's last, ragged tile
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (kp0 + 16 * kt + 4 * g + r >= cnt) {
#pragma unroll
            for (int qt = 0; qt < NQW; ++qt) s[qt][kt][r] = -INFINITY;
          }
    }
    // ---- online softmax; the four lane groups of a column share the query ----
    uint4 pf[NQW][2];
#pragma unroll
    for (int qt = 0; qt < NQW; ++qt) {
      float mx = st_max3(s[qt][0][0], s[qt][0][1], s[qt][0][2]);
      mx = st_max3(mx, s[qt][0][3], s[qt][1][0]);
      mx = st_max3(mx, s[qt][1][1], s[qt][1][2]);
      mx = st_max3(mx, s[qt][1][3], s[qt][2][0]);
      mx = st_max3(mx, s[qt][2][1], s[qt][2][2]);
      mx = st_max3(mx, s[qt][2][3], s[qt][3][0]);
      mx = st_max3(mx, s[qt][3][1], s[qt][3][2]);
      mx = st_max_lane_groups(st_max(mx, s[qt][3][3])) * scale2;  // scale2 > 0: scaling commutes with the maximum
      const float m_new = fmaxf(m[qt], mx);
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;  // a query that sees no key yet
      // lists are sorted by descending projection, so after the first tiles the running maximum
      // rarely moves: rescale only when it moved for some query of the wave
      if (__any(m_new != m[qt])) {
        const float alpha = __builtin_amdgcn_exp2f(m[qt] - m_sub);
        lsum[qt] *= alpha;
#pragma unroll
        for (int t8 = 0; t8 < 8; ++t8) {
          O[qt][t8][0] *= alpha;
          O[qt][t8][1] *= alpha;
          O[qt][t8][2] *= alpha;
          O[qt][t8][3] *= alpha;
        }
        m[qt] = m_new;
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float p[8];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[r] = __builtin_amdgcn_exp2f(fmaf(s[qt][2 * h][r], scale2, -m_sub));
          p[4 + r] = __builtin_amdgcn_exp2f(fmaf(s[qt][2 * h + 1][r], scale2, -m_sub));
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) lsum[qt] += p[r];
        pf[qt][h] = make_uint4(Mma<F16>::pack2(p[0], p[1]), Mma<F16>::pack2(p[2], p[3]), Mma<F16>::pack2(p[4], p[5]),
                               Mma<F16>::pack2(p[6], p[7]));
      }
    }
    // ---- O^T += Vt.P^T (32-key half outermost, for the same reason) ----
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int t8 = 0; t8 < 8; ++t8) {
        const uint4 a = *reinterpret_cast<const uint4*>(&bV[(16 * t8 + c) * kSVld + 8 * g + 32 * h]);
#pragma unroll
        for (int qt = 0; qt < NQW; ++qt) O[qt][t8] = Mma<F16>::m16(a, pf[qt][h], O[qt][t8]);
      }
    }
  };

  // The list rows of tile t + 2 are requested while tile t is computed and first looked at one tile
  // later; the two registers alternate (a single one, copied at the end of the iteration, makes the
  // copy wait for the request just issued).
  int rows_a = 0, rows_b = 0;
  if (ntiles > 0) {
    FM_STAGED_LOAD_TILE(rows_of(0));
    rows_a = rows_of(1);
    stash_tile(0);
    if (NBUF == 2 && ntiles > 1) {
      FM_STAGED_LOAD_TILE(rows_a);
      rows_b = rows_of(2);
    }
  }
  // The query fragments are first read inside the loop; reading them here puts the wait for their
  // loads in front of the loop instead of in front of the first MFMA of every tile (where it would
  // also wait for the tile loads just issued).
#pragma unroll
  for (int qt = 0; qt < NQW; ++qt)
#pragma unroll
    for (int s = 0; s < 4; ++s)
      asm volatile("" ::"v"(qf[qt][s].x), "v"(qf[qt][s].y), "v"(qf[qt][s].z), "v"(qf[qt][s].w));
  __syncthreads();
  if (NBUF == 1) {
    // one buffer: the registers hold tile t + 1 while tile t is computed, two barriers per tile
#define FM_STAGED_STEP(t_, rows_use, rows_fetch)                                   \
  do {                                                                             \
    const bool more_ = (t_) + 1 < ntiles;                                          \
    if (more_) {                                                                   \
      rows_fetch = rows_of((t_) + 2);                                              \
      FM_STAGED_LOAD_TILE(rows_use); /* lands while this tile is computed */       \
    }                                                                              \
    if (wave_on) compute_tile(t_, 0);                                              \
    __syncthreads(); /* every wave has read tile t */                              \
    if (more_) stash_tile(0);                                                      \
    __syncthreads(); /* tile t + 1 is in place */                                  \
  } while (0)
    for (int t = 0; t < ntiles; t += 2) {
      FM_STAGED_STEP(t, rows_a, rows_b);
      if (t + 1 >= ntiles) break;
      FM_STAGED_STEP(t + 1, rows_b, rows_a);
    }
#undef FM_STAGED_STEP
  } else {
    // two buffers: tile t + 1 (requested a whole tile ago) goes from the registers into the buffer that
    // tile t - 1 was read from, the request for tile t + 2 follows, then tile t is computed; one
    // barrier per tile
#define FM_STAGED_STEP(t_, rows_use, rows_fetch)                                   \
  do {                                                                             \
    if ((t_) + 1 < ntiles) stash_tile(((t_) + 1) & 1);                             \
    if ((t_) + 2 < ntiles) {                                                       \
      rows_fetch = rows_of((t_) + 3);                                              \
      FM_STAGED_LOAD_TILE(rows_use);                                               \
    }                                                                              \
    if (wave_on) compute_tile(t_, (t_) & 1);                                       \
    __syncthreads();                                                               \
  } while (0)
    for (int t = 0; t < ntiles; t += 2) {
      FM_STAGED_STEP(t, rows_b, rows_a);
      if (t + 1 >= ntiles) break;
      FM_STAGED_STEP(t + 1, rows_a, rows_b);
    }
#undef FM_STAGED_STEP
  }

  // ---- finish: lane (g,c) holds dims 16t + 4g + r of query c of each tile ----
#undef FM_STAGED_LOAD_TILE
#pragma unroll
  for (int qt = 0; qt < NQW; ++qt) {
    float ltot = lsum[qt] + __shfl_xor(lsum[qt], 16);
    ltot += __shfl_xor(ltot, 32);
    const bool empty = (m[qt] == -INFINITY);  // the query saw no key at all
    const float inv = empty ? 0.f : 1.f / ltot;
    if (q_ok[qt]) {
      bf16_t* po = Ob + qrow[qt] * kSD + 4 * g;
#pragma unroll
      for (int t8 = 0; t8 < 8; ++t8) {
        uint2 o;
        o.x = Mma<F16>::pack2(O[qt][t8][0] * inv, O[qt][t8][1] * inv);
        o.y = Mma<F16>::pack2(O[qt][t8][2] * inv, O[qt][t8][3] * inv);
        *reinterpret_cast<uint2*>(po + 16 * t8) = o;
      }
      if (g == 0) Lb[qrow[qt]] = empty ? -FLT_MAX : (m[qt] + __builtin_amdgcn_logf(ltot)) * kLn2;
    }
  }
}

}  // namespace fm
