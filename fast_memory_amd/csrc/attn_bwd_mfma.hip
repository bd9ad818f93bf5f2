// Backward of the bucket-gathered attention on MFMA: bf16, head dimension 128
// (gfx950).  Same mathematics as the generic kernel in attn_bwd.hip.
//
// One workgroup (4 waves) per (work item, 16-query tile): the tile's rows of Q
// and dO stay in registers, the bucket's 32-key blocks are dealt round-robin to
// the waves, K and V rows go from global memory straight into MFMA operand
// registers (one block in flight behind the one being computed).  Per block a
// wave forms the 16 x 32 score tile twice, once per orientation, because the
// three gradients contract over different indices and an accumulator can only
// be fed back as the operand whose contraction index it holds in registers:
//   keys on accumulator rows (S^T = K.Q^T, dP^T = V.dO^T): lane (g,c) holds
//     query c, keys 4g+r -- exactly the B operand of  dQ^T += K^T . dS^T
//     (contraction over keys; K^T comes from coalesced loads repacked per lane,
//     as V does in the forward kernel);
//   queries on accumulator rows (S = Q.K^T, dP = dO.V^T): lane (g,c) holds key
//     c, queries 4g+r -- exactly the A operand of  dV = P^T . dO  and
//     dK = dS^T . Q  (v_mfma_f32_16x16x16_bf16, contraction over the 16
//     queries; dO^T and Q^T fragments, the B operands, are loaded once per tile).
// dQ partial sums of the four waves are added through LDS and written once.  dK
// and dV tiles (keys on rows, d on columns) leave the wave as fp32 atomic adds
// into the keys' rows (a key belongs to many buckets): per instruction and lane
// group 16 consecutive floats of one row.
//
// Roofline: the atomic traffic, 2 * d * 4 bytes per gathered (item tile, key)
// pair, on top of the forward's gather traffic.
#include "common.hpp"

namespace fm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4s;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bbf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float bf32x2;

constexpr int kBD = 128;

__device__ __forceinline__ bf16x8 b_as_bf16x8(uint4 u) {
  union {
    uint4 u;
    bf16x8 b;
  } x;
  x.u = u;
  return x.b;
}
__device__ __forceinline__ bf16x4s b_as_bf16x4(uint2 u) {
  union {
    uint2 u;
    bf16x4s b;
  } x;
  x.u = u;
  return x.b;
}
__device__ __forceinline__ uint32_t b_pack(float lo, float hi) {
  bf32x2 x = {lo, hi};
  bbf16x2 y = __builtin_convertvector(x, bbf16x2);  // round to nearest even
  return *reinterpret_cast<uint32_t*>(&y);
}

struct BwdBlock {
  uint4 k[2][4];   // K rows as MFMA operand: [key tile][contraction step], lane (g,c): key c, columns 32s+8g..
  uint4 vk[2][4];  // V rows in the same layout
  uint4 kc[2][4];  // K rows coalesced: [key tile][key 4g+j], lane (g,c): 16-byte chunk c
  int rk[2];       // key row of lane's column c in each key tile
};

__device__ __forceinline__ void bwd_load_block(BwdBlock& r, const bf16_t* __restrict__ Kb,
                                               const bf16_t* __restrict__ Vb, int rows, int g, int c) {
#pragma unroll
  for (int kt = 0; kt < 2; ++kt) {
    const int rk = __shfl(rows, kt * 16 + c);
    r.rk[kt] = rk;
    const uint4* pk = reinterpret_cast<const uint4*>(Kb + int64_t(rk) * kBD + 8 * g);
    const uint4* pv = reinterpret_cast<const uint4*>(Vb + int64_t(rk) * kBD + 8 * g);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      r.k[kt][s] = pk[4 * s];
      r.vk[kt][s] = pv[4 * s];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rv = __shfl(rows, kt * 16 + 4 * g + j);
      r.kc[kt][j] = *reinterpret_cast<const uint4*>(Kb + int64_t(rv) * kBD + 8 * c);
    }
  }
}

__global__ __launch_bounds__(256) void hash_attn_bwd_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off, const int32_t* __restrict__ bucket_cnt,
    const int32_t* __restrict__ q_perm, const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    const bf16_t* __restrict__ out, const float* __restrict__ lse, const bf16_t* __restrict__ dout,
    bf16_t* __restrict__ dq, float* __restrict__ dk, float* __restrict__ dv, int Sq, int N, int C, float sm_scale) {
  __shared__ __attribute__((aligned(16))) float red[4 * 8 * 4 * 64];  // dQ partials [wave][t][r][lane]
  __shared__ int q_rows[16];
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int q0 = int(blockIdx.y) * 16;  // this workgroup's query tile inside the item
  if (q0 >= it.n_q) return;
  const int n_q = min(16, it.n_q - q0);
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int cnt = bucket_cnt[bkt];
  if (threadIdx.x < 16) q_rows[threadIdx.x] = threadIdx.x < n_q ? q_perm[it.q_start + q0 + threadIdx.x] : -1;
  __syncthreads();
  const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int g = l >> 4, c = l & 15;
  const int64_t qbase = int64_t(it.row) * Sq;
  const bf16_t* Kb = k + int64_t(it.row) * N * kBD;
  const bf16_t* Vb = v + int64_t(it.row) * N * kBD;
  float* dKb = dk + int64_t(it.row) * N * kBD;
  float* dVb = dv + int64_t(it.row) * N * kBD;
  const int32_t* idx = k_idx + bucket_off[bkt];
  const float scale2 = sm_scale * kLog2e;

  // ---- the tile's Q, dO rows: operand fragments in both orientations, lse and D ----
  const int myq = q_rows[c];  // query of lane column c (-1: none)
  uint4 qf[4], dof[4];
  float Dc = 0.f;
  {
    const int64_t row = qbase + max(myq, 0);
    const uint4* pq = reinterpret_cast<const uint4*>(q + row * kBD + 8 * g);
    const uint4* pd = reinterpret_cast<const uint4*>(dout + row * kBD + 8 * g);
    const uint4* po = reinterpret_cast<const uint4*>(out + row * kBD + 8 * g);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bool ok = myq >= 0;
      qf[s] = ok ? pq[4 * s] : make_uint4(0, 0, 0, 0);
      dof[s] = ok ? pd[4 * s] : make_uint4(0, 0, 0, 0);
      const uint4 o4 = ok ? po[4 * s] : make_uint4(0, 0, 0, 0);
      const uint32_t dw[4] = {dof[s].x, dof[s].y, dof[s].z, dof[s].w};
      const uint32_t ow[4] = {o4.x, o4.y, o4.z, o4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        Dc = fmaf(__uint_as_float(dw[e] << 16), __uint_as_float(ow[e] << 16), Dc);
        Dc = fmaf(__uint_as_float(dw[e] & 0xffff0000u), __uint_as_float(ow[e] & 0xffff0000u), Dc);
      }
    }
  }
  Dc += __shfl_xor(Dc, 16);
  Dc += __shfl_xor(Dc, 32);  // D of query c, in all four lane groups
  // a lane column without a query gets lse = +inf: every probability is 0
  const float lse2c = myq >= 0 ? lse[qbase + myq] * kLog2e : INFINITY;
  float Dq[4], lse2q[4];  // the same for queries 4g+r (the other orientation)
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    Dq[r] = __shfl(Dc, 4 * g + r);
    lse2q[r] = __shfl(lse2c, 4 * g + r);
  }
  // transposed fragments: lane (g,c) holds rows (queries) 4g..4g+3 at column 16t + c
  uint2 qT[8], doT[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    uint32_t qa[4], da[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int qq = q_rows[4 * g + j];
      const int64_t row = qbase + max(qq, 0);
      qa[j] = qq >= 0 ? uint32_t(q[row * kBD + 16 * t + c]) : 0u;
      da[j] = qq >= 0 ? uint32_t(dout[row * kBD + 16 * t + c]) : 0u;
    }
    qT[t] = make_uint2(qa[0] | (qa[1] << 16), qa[2] | (qa[3] << 16));
    doT[t] = make_uint2(da[0] | (da[1] << 16), da[2] | (da[3] << 16));
  }

  f32x4 dQ[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) dQ[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int nblk = (cnt + 31) / 32;
  auto rows_of = [&](int b) -> int {
    const int kp = b * 32 + (l & 31);
    int r = 0;
    if (kp < cnt) r = idx[kp];
    return min(max(r, 0), N - 1);
  };

  auto compute = [&](const BwdBlock& kv, int b) {
    const int kp0 = b * 32;
    // K^T fragments for the eight output tiles of dQ: element t of the eight coalesced loads
    uint4 kf[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int dw = t >> 1;
      uint32_t a[8];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint4 x = kv.kc[kt][j];
          a[kt * 4 + j] = dw == 0 ? x.x : dw == 1 ? x.y : dw == 2 ? x.z : x.w;
        }
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o[e] = (t & 1) ? ((a[2 * e] >> 16) | (a[2 * e + 1] & 0xffff0000u))
                       : ((a[2 * e] & 0xffffu) | (a[2 * e + 1] << 16));
      kf[t] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    // ---- keys on rows: S^T, dP^T -> dS^T -> dQ ----
    {
      f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0, p0 = s0, p1 = s0;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_as_bf16x8(kv.k[0][s]), b_as_bf16x8(qf[s]), s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_as_bf16x8(kv.k[1][s]), b_as_bf16x8(qf[s]), s1, 0, 0, 0);
        p0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_as_bf16x8(kv.vk[0][s]), b_as_bf16x8(dof[s]), p0, 0, 0, 0);
        p1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_as_bf16x8(kv.vk[1][s]), b_as_bf16x8(dof[s]), p1, 0, 0, 0);
      }
      float ds[8];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float pa = (kp0 + 4 * g + r < cnt) ? __builtin_amdgcn_exp2f(fmaf(s0[r], scale2, -lse2c)) : 0.f;
        const float pb = (kp0 + 16 + 4 * g + r < cnt) ? __builtin_amdgcn_exp2f(fmaf(s1[r], scale2, -lse2c)) : 0.f;
        ds[r] = pa * (p0[r] - Dc) * sm_scale;
        ds[4 + r] = pb * (p1[r] - Dc) * sm_scale;
      }
      const uint4 pf = make_uint4(b_pack(ds[0], ds[1]), b_pack(ds[2], ds[3]), b_pack(ds[4], ds[5]), b_pack(ds[6], ds[7]));
#pragma unroll
      for (int t = 0; t < 8; ++t)
        dQ[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_as_bf16x8(kf[t]), b_as_bf16x8(pf), dQ[t], 0, 0, 0);
    }
    // ---- queries on rows: S, dP -> P, dS -> dV, dK tiles, added to the keys' rows ----
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      f32x4 sN = {0.f, 0.f, 0.f, 0.f}, pN = sN;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        sN = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_as_bf16x8(qf[s]), b_as_bf16x8(kv.k[kt][s]), sN, 0, 0, 0);
        pN = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_as_bf16x8(dof[s]), b_as_bf16x8(kv.vk[kt][s]), pN, 0, 0, 0);
      }
      const bool key_ok = kp0 + 16 * kt + c < cnt;
      float pr[4], dsr[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pr[r] = key_ok ? __builtin_amdgcn_exp2f(fmaf(sN[r], scale2, -lse2q[r])) : 0.f;
        dsr[r] = pr[r] * (pN[r] - Dq[r]) * sm_scale;
      }
      // P and dS as the A operand (lane (g,c): row = key c, contraction = queries 4g..4g+3), dO^T and
      // Q^T fragments as B: the output tile has keys on rows and d on columns, so that one atomic
      // instruction covers, per lane group, 16 consecutive floats (a 64-byte line) of one key's row
      const bf16x4s pA = b_as_bf16x4(make_uint2(b_pack(pr[0], pr[1]), b_pack(pr[2], pr[3])));
      const bf16x4s dsA = b_as_bf16x4(make_uint2(b_pack(dsr[0], dsr[1]), b_pack(dsr[2], dsr[3])));
      int64_t rowoff[4];
      bool rok[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        rowoff[r] = int64_t(__shfl(kv.rk[kt], 4 * g + r)) * kBD + c;
        rok[r] = kp0 + 16 * kt + 4 * g + r < cnt;
      }
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
        const f32x4 tv = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pA, b_as_bf16x4(doT[t]), z, 0, 0, 0);
        const f32x4 tk = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(dsA, b_as_bf16x4(qT[t]), z, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (rok[r]) {
            unsafeAtomicAdd(dVb + rowoff[r] + 16 * t, tv[r]);
            unsafeAtomicAdd(dKb + rowoff[r] + 16 * t, tk[r]);
          }
      }
    }
  };

  // ---- main loop: this wave's blocks w, w+4, ..., one block in flight ----
  BwdBlock ra, rb;
  int b = w;
  if (b < nblk) bwd_load_block(ra, Kb, Vb, rows_of(b), g, c);
  while (b < nblk) {
    const int b1 = b + 4, b2 = b + 8;
    if (b1 < nblk) bwd_load_block(rb, Kb, Vb, rows_of(b1), g, c);
    compute(ra, b);
    if (b1 >= nblk) break;
    if (b2 < nblk) bwd_load_block(ra, Kb, Vb, rows_of(b2), g, c);
    compute(rb, b1);
    b = b2;
  }

  // ---- dQ: add the four waves' partial sums, write the tile's rows ----
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((w * 8 + t) * 4 + r) * 64 + l] = dQ[t][r];
  __syncthreads();
  // wave w finalises accumulator row r = w: columns 32g + 8w + (0..7) of query c
  float o[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    float a = 0.f;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) a += red[((ww * 8 + t) * 4 + w) * 64 + l];
    o[t] = a;
  }
  if (myq >= 0)
    *reinterpret_cast<uint4*>(dq + (qbase + myq) * kBD + 32 * g + 8 * w) =
        make_uint4(b_pack(o[0], o[1]), b_pack(o[2], o[3]), b_pack(o[4], o[5]), b_pack(o[6], o[7]));
}

bool hash_attn_bwd_mfma_supported(int d, int dtype) { return d == kBD && dtype == FM_BF16; }

int hash_attn_bwd_mfma(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                       const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                       int64_t max_items, const void* out, const float* lse, const void* dout, void* dq, float* dk,
                       float* dv, int Sq, int N, int C, float sm_scale, hipStream_t st) {
  dim3 grid = dim3(unsigned(max_items), unsigned(FM_QTILE / 16));
  hipLaunchKernelGGL(hash_attn_bwd_mfma_kernel, grid, dim3(256), 0, st, (const bf16_t*)q, (const bf16_t*)k,
                     (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, (const bf16_t*)out, lse,
                     (const bf16_t*)dout, (bf16_t*)dq, dk, dv, Sq, N, C, sm_scale);
  return launch_status("fm_hash_attn_bwd(mfma)");
}

}  // namespace fm
