// bf16 bucket-gathered attention forward for head dimension 128 (gfx950), the form for
// launches whose work items are mostly full (many queries per bucket, e.g. the shape of the
// reference's own performance harness, triton_kernel.py:507-528: 128 queries per bucket).
// There the arithmetic, not the gather, is the larger part, and the register-gather kernel
// (attn_mfma.hip) runs one wave per SIMD with every MFMA, softmax and load of a wave in series.
//
// Work decomposition.  One workgroup (4 waves) per work item (up to 64 queries of one bucket);
// wave w carries queries 16w..16w+15 over ALL keys of the bucket, so the waves never merge.
// The bucket's rows are gathered once per workgroup: tiles of 64 keys go global -> registers
// (in flight during the previous tile's arithmetic) -> LDS, V transposed on the way
// ( Vt[d][key] ), and every wave reads its MFMA operands from there.  About 100 registers per
// wave and 36 KiB of LDS per workgroup: four workgroups share a CU, one wave's softmax runs
// under another's MFMAs.
//   S^T = K.Q^T    v_mfma_f32_16x16x32_bf16, A = 16 K rows from LDS, B = Q^T fragments resident
//                  in registers; lane (g,c) gets the scores of keys 4g..4g+3 of each 16-key
//                  tile for query c.
//   O^T += Vt.P^T  same instruction over 32 keys: the scores of key tiles 2h and 2h+1 in a lane
//                  are the B operand if contraction slot 8g+e stands for key 4g+e of tile 2h
//                  (e < 4) or key 4g+e-4 of tile 2h+1; Vt is stored with its key columns in
//                  that order, so neither P nor V is shuffled.  Lane (g,c) holds
//                  O[query c][16t + 4g .. 16t + 4g + 3], t = 0..7.
// Softmax as in the reference kernel (triton_kernel.py:248-263): base 2 with sm_scale*log2(e),
// fp32 running max and denominator, denominator from unrounded p, p rounded to bf16 before P.V.
//
// Roofline: HBM for the algorithmic bytes (cnt*(2*128*2+4) per bucket), MFMA for 4*128 flops per
// query-key pair; at 128 queries per bucket the two are within a factor of three of each other.
#include "common.hpp"

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


__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void hash_attn_staged_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2) {
  __shared__ __attribute__((aligned(16))) bf16_t sK[kSK * kSKld];
  __shared__ __attribute__((aligned(16))) bf16_t sVt[kSD * kSVld];
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int g = l >> 4, c = l & 15;
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int cnt = bucket_cnt[bkt];
  const int32_t* idx = k_idx + bucket_off[bkt];
  const bf16_t* Kb = k + int64_t(it.row) * N * kSD;
  const bf16_t* Vb = v + int64_t(it.row) * N * kSD;
  const int64_t qbase = int64_t(it.row) * Sq;
  const int ntiles = (cnt + kSK - 1) / kSK;

  // ---- this lane's query (column c of wave w's 16) ----
  const int jq = 16 * w + c;
  const bool q_ok = jq < it.n_q;
  const bool wave_on = 16 * w < it.n_q;
  const int64_t qrow = q_ok ? q_perm[it.q_start + jq] : 0;
  uint4 qf[4];
  {
    const uint4* pq = reinterpret_cast<const uint4*>(q + (qbase + qrow) * kSD + 8 * g);
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = q_ok ? pq[4 * s] : make_uint4(0, 0, 0, 0);
  }
  f32x4 O[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) O[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;

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
  auto k_row = [&](int rows, int p) {
    return reinterpret_cast<const uint4*>(Kb + int64_t(__shfl(rows, p)) * kSD)[kchunk];
  };
  auto v_row = [&](int rows, int p) {
    return reinterpret_cast<const uint4*>(Vb + int64_t(__shfl(rows, p)) * kSD)[vc];
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
  auto vt_pair = [&](uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, int e) {
    uint2 lo, hi;  // dims e (low halves) and e + 1 (high halves) of the four keys
    lo.x = (a0 & 0xffffu) | (a1 << 16);
    lo.y = (a2 & 0xffffu) | (a3 << 16);
    hi.x = (a0 >> 16) | (a1 & 0xffff0000u);
    hi.y = (a2 >> 16) | (a3 & 0xffff0000u);
    *reinterpret_cast<uint2*>(&sVt[(8 * vc + e) * kSVld + pos0]) = lo;
    *reinterpret_cast<uint2*>(&sVt[(8 * vc + e + 1) * kSVld + pos0]) = hi;
  };
  auto stash_tile = [&]() {
    *reinterpret_cast<uint4*>(&sK[(krow + 0) * kSKld + kchunk * 8]) = tk0;
    *reinterpret_cast<uint4*>(&sK[(krow + 16) * kSKld + kchunk * 8]) = tk1;
    *reinterpret_cast<uint4*>(&sK[(krow + 32) * kSKld + kchunk * 8]) = tk2;
    *reinterpret_cast<uint4*>(&sK[(krow + 48) * kSKld + kchunk * 8]) = tk3;
    vt_pair(tv0.x, tv1.x, tv2.x, tv3.x, 0);
    vt_pair(tv0.y, tv1.y, tv2.y, tv3.y, 2);
    vt_pair(tv0.z, tv1.z, tv2.z, tv3.z, 4);
    vt_pair(tv0.w, tv1.w, tv2.w, tv3.w, 6);
  };

  auto compute_tile = [&](int t) {
    const int kp0 = t * kSK;
    // ---- S^T for the four 16-key tiles ----
    f32x4 s[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* pa = &sK[(kt * 16 + c) * kSKld + 8 * g];
#pragma unroll
      for (int st = 0; st < 4; ++st)
        s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(pa + 32 * st),
                                                        st_as_bf16x8(qf[st]), s[kt], 0, 0, 0);
    }
    if (kp0 + kSK > cnt) {  // the bucket's last, ragged tile
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
    // lists are sorted by descending projection, so after the first tiles the running maximum
    // rarely moves: rescale only when it moved for some query of the wave
    if (__any(m_new != m)) {
      const float alpha = __builtin_amdgcn_exp2f(m - m_sub);
      lsum *= alpha;
#pragma unroll
      for (int t8 = 0; t8 < 8; ++t8) {
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
      pf[h] = make_uint4(st_pack_bf16(p[0], p[1]), st_pack_bf16(p[2], p[3]), st_pack_bf16(p[4], p[5]),
                         st_pack_bf16(p[6], p[7]));
    }
    // ---- O^T += Vt.P^T ----
#pragma unroll
    for (int t8 = 0; t8 < 8; ++t8) {
      const bf16_t* pv = &sVt[(16 * t8 + c) * kSVld + 8 * g];
#pragma unroll
      for (int h = 0; h < 2; ++h)
        O[t8] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(pv + 32 * h),
                                                        st_as_bf16x8(pf[h]), O[t8], 0, 0, 0);
    }
  };

  int rows_next = 0;
  if (ntiles > 0) {
    FM_STAGED_LOAD_TILE(rows_of(0));
    rows_next = rows_of(1);
    stash_tile();
  }
  // The query fragments are first read inside the loop; reading them here puts the wait for their
  // loads in front of the loop instead of in front of the first MFMA of every tile (where it would
  // also wait for the tile loads just issued).
#pragma unroll
  for (int s = 0; s < 4; ++s) asm volatile("" ::"v"(qf[s].x), "v"(qf[s].y), "v"(qf[s].z), "v"(qf[s].w));
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const bool more = t + 1 < ntiles;
    if (more) {
      const int rows_after = rows_of(t + 2);
      FM_STAGED_LOAD_TILE(rows_next);  // lands while this tile is computed
      rows_next = rows_after;
    }
    if (wave_on) compute_tile(t);
    __syncthreads();  // every wave has read tile t
    if (more) stash_tile();
    __syncthreads();  // tile t + 1 is in place
  }

  // ---- finish: lane (g,c) holds dims 16t + 4g + r of query c ----
  float ltot = lsum + __shfl_xor(lsum, 16);
  ltot += __shfl_xor(ltot, 32);
  const bool empty = (m == -INFINITY);  // the query saw no key at all
  const float inv = empty ? 0.f : 1.f / ltot;
#undef FM_STAGED_LOAD_TILE
  if (q_ok) {
    bf16_t* po = out + (qbase + qrow) * kSD + 4 * g;
#pragma unroll
    for (int t8 = 0; t8 < 8; ++t8) {
      uint2 o;
      o.x = st_pack_bf16(O[t8][0] * inv, O[t8][1] * inv);
      o.y = st_pack_bf16(O[t8][2] * inv, O[t8][3] * inv);
      *reinterpret_cast<uint2*>(po + 16 * t8) = o;
    }
    if (g == 0) lse[qbase + qrow] = empty ? -FLT_MAX : (m + __builtin_amdgcn_logf(ltot)) * kLn2;
  }
}

int hash_attn_mfma_staged(const void* q, const void* k, const void* v, const int32_t* k_idx,
                          const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                          const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                          float* lse, int Sq, int N, int C, float sm_scale, hipStream_t st) {
  hipLaunchKernelGGL(hash_attn_staged_kernel, dim3(unsigned(max_items)), dim3(256), 0, st, (const bf16_t*)q,
                     (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items,
                     (bf16_t*)out, lse, Sq, N, C, sm_scale * kLog2e);
  return launch_status("fm_hash_attn_fwd(mfma, staged)");
}

}  // namespace fm
