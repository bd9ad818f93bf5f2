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
#include <atomic>

#include "common.hpp"
#include "attn_ring.hpp"
#include "mma16.hpp"

namespace fm {

extern std::atomic<int> g_force_generic;  // attn_api.hip; 9: the staged backward loads its blocks into registers

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4s;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bbf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float bf32x2;

constexpr int kBD = 128;
constexpr int kPartLd = 2 * kBD;  // a list position's partial rows lie side by side: [dK row | dV row], 512 bytes

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

constexpr int kStLd = 136;  // bf16 elements per staged partial row (128 + 8: 16-byte aligned, banks spread)

// Sum of two rows of eight bf16, rounded to nearest even.
__device__ __forceinline__ uint4 add_bf16x8(uint4 a, uint4 b) {
  const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    o[e] = b_pack(__uint_as_float(aw[e] << 16) + __uint_as_float(bw[e] << 16),
                  __uint_as_float(aw[e] & 0xffff0000u) + __uint_as_float(bw[e] & 0xffff0000u));
  return make_uint4(o[0], o[1], o[2], o[3]);
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

// One 16-query tile of a bucket: q_list[0..n_q) are the tile's query rows (inside row `qbase / Sq`).
// STAGED = false: dK and dV contributions are added atomically into the keys' rows of dKb / dVb (fp32).
// STAGED = true:  they go to the bucket's own partial rows dkp / dvp [list position][128] in bf16, one row
//                 per listed key, stored (first tile of the bucket) or added to what the earlier tiles
//                 left (the workgroup owns the bucket, so no atomics); a second kernel sums every key's
//                 partial rows over the buckets that list it.
//
// TILES = 2 or 4 (staged form only): q_list holds up to TILES tiles, n_q <= 16 * TILES.  With two, waves
// 0,1 take the first and waves 2,3 the second, and waves w and w^2 walk the same key blocks (parity w&1)
// in step; with four, every wave has a tile of its own and all walk every block.  What the tiles add to
// a block's partial rows is summed through the waves' LDS slabs before it is stored, so the bucket's K
// and V rows are gathered and its partial rows written once for all the tiles of the pass.  The sums are
// those of single-tile passes in tile order (bf16 rows added and rounded one by one).
//
// LDSBLK (two-tile staged form, first pass only): a block's K and V rows do not come into registers straight
// from memory when the block is needed; they are requested a block ahead with loads that write LDS directly
// (no registers in between), and the waves fill their operand registers from there.  The gather then runs
// beside the arithmetic and the stores of the block before it.  blk: 32 KB, [block parity][K | V][32 rows of 256 B],
// 16-byte chunk q of row r at position q ^ f(r) (no padding, no bank conflicts for either read pattern).
template <bool STAGED, bool FIRST_TILE, int TILES = 1, bool LDSBLK = false, bool F16 = false>
__device__ __forceinline__ void bwd_tile(const bf16_t* __restrict__ q, const bf16_t* __restrict__ out,
                                         const float* __restrict__ lse, const bf16_t* __restrict__ dout,
                                         const float* __restrict__ dlse, const int32_t* __restrict__ q_list, int n_q, int64_t qbase,
                                         const bf16_t* __restrict__ Kb, const bf16_t* __restrict__ Vb,
                                         const int32_t* __restrict__ idx, int cnt, int N, float sm_scale,
                                         bf16_t* __restrict__ dq, float* __restrict__ dKb, float* __restrict__ dVb,
                                         bf16_t* dkp, bf16_t* dvp, bf16_t* dump, float* red, int* q_rows,
                                         bf16_t* stage, unsigned char* blk = nullptr) {
  static_assert(!LDSBLK || (STAGED && FIRST_TILE && TILES == 2), "the LDS block form is the first two-tile pass");
  using M = Mma<F16>;  // the 16-bit type of q, k, v, out, dout and dq (F16: fp16, else bf16); partial rows are bf16
  if (threadIdx.x < 16 * TILES) q_rows[threadIdx.x] = threadIdx.x < n_q ? q_list[threadIdx.x] : -1;
  __syncthreads();
  const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int g = l >> 4, c = l & 15;
  const float scale2 = sm_scale * kLog2e;
  constexpr bool PAIR = TILES == 2, QUAD = TILES == 4;
  const int tw = PAIR ? (w >> 1) : QUAD ? w : 0;  // this wave's tile of the pass
  q_rows += 16 * tw;
  auto lds_barrier = [] {  // workgroup barrier that orders LDS only (global stores stay in flight)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  };

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
        Dc = fmaf(M::lo(dw[e]), M::lo(ow[e]), Dc);
        Dc = fmaf(M::hi(dw[e]), M::hi(ow[e]), Dc);
      }
    }
  }
  Dc += __shfl_xor(Dc, 16);
  Dc += __shfl_xor(Dc, 32);  // D of query c, in all four lane groups
  // a gradient of the log-sum-exp enters dS = P (dP - D) as dS += P dlse: fold it into D
  if (dlse != nullptr && myq >= 0) Dc -= dlse[qbase + myq];
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
  // Nothing in the block loop branches around a memory instruction: loads past the end of the list are
  // clamped to its last entry and stores of the staged form are redirected to a dump row, so the
  // compiler knows how many memory operations follow each load and the wait for a prefetched block does
  // not drain the stores behind it (loads and stores share one completion counter).
  auto rows_of = [&](int b) -> int {
    const int kp = min(b * 32 + (l & 31), max(cnt - 1, 0));
    return min(max(idx[kp], 0), N - 1);
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
        s0 = M::m16(kv.k[0][s], qf[s], s0);
        s1 = M::m16(kv.k[1][s], qf[s], s1);
        p0 = M::m16(kv.vk[0][s], dof[s], p0);
        p1 = M::m16(kv.vk[1][s], dof[s], p1);
      }
      float ds[8];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float pa = (kp0 + 4 * g + r < cnt) ? __builtin_amdgcn_exp2f(fmaf(s0[r], scale2, -lse2c)) : 0.f;
        const float pb = (kp0 + 16 + 4 * g + r < cnt) ? __builtin_amdgcn_exp2f(fmaf(s1[r], scale2, -lse2c)) : 0.f;
        ds[r] = pa * (p0[r] - Dc) * sm_scale;
        ds[4 + r] = pb * (p1[r] - Dc) * sm_scale;
      }
      const uint4 pf = make_uint4(M::pack2(ds[0], ds[1]), M::pack2(ds[2], ds[3]), M::pack2(ds[4], ds[5]), M::pack2(ds[6], ds[7]));
#pragma unroll
      for (int t = 0; t < 8; ++t)
        dQ[t] = M::m16(kf[t], pf, dQ[t]);
    }
    // ---- queries on rows: S, dP -> P, dS -> dV, dK tiles, added to the keys' rows ----
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      f32x4 sN = {0.f, 0.f, 0.f, 0.f}, pN = sN;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        sN = M::m16(qf[s], kv.k[kt][s], sN);
        pN = M::m16(dof[s], kv.vk[kt][s], pN);
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
      const uint2 pA = make_uint2(M::pack2(pr[0], pr[1]), M::pack2(pr[2], pr[3]));
      const uint2 dsA = make_uint2(M::pack2(dsr[0], dsr[1]), M::pack2(dsr[2], dsr[3]));
      if (STAGED) {
        // The transposed tiles (the same registers with the operands swapped): lane (g,c) holds key c and
        // the four consecutive columns 16t + 4g .. +3.  They go through a slab of LDS private to the wave
        // ([dV | dK][16 keys][136]) and leave as whole rows: 16 adjacent lanes store the 256 bytes of one
        // key's partial row, an instruction 1 KB of consecutive list positions.
        bf16_t* slab = stage + w * (2 * 16 * kStLd);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const f32x4 z = {0.f, 0.f, 0.f, 0.f};
          const f32x4 tv = M::m16k16(doT[t], pA, z);
          const f32x4 tk = M::m16k16(qT[t], dsA, z);
          *reinterpret_cast<uint2*>(slab + c * kStLd + 16 * t + 4 * g) =
              make_uint2(b_pack(tv[0], tv[1]), b_pack(tv[2], tv[3]));
          *reinterpret_cast<uint2*>(slab + (16 + c) * kStLd + 16 * t + 4 * g) =
              make_uint2(b_pack(tk[0], tk[1]), b_pack(tk[2], tk[3]));
        }
        if (QUAD) {
          // the four tiles' slabs of this key tile are complete; wave 0 stores dV rows 0-7, wave 1 dV rows
          // 8-15, waves 2 and 3 the dK rows likewise, each the sum of the four slabs in tile order
          lds_barrier();
          const int mat = w >> 1;  // 0: dV, 1: dK
#pragma unroll
          for (int ii = 0; ii < 2; ++ii) {
            const int rr = 4 * (2 * (w & 1) + ii) + g;
            const bf16_t* src = stage + mat * (16 * kStLd) + rr * kStLd + 8 * c;
            uint4 x = *reinterpret_cast<const uint4*>(src);
#pragma unroll
            for (int j = 1; j < 4; ++j) x = add_bf16x8(x, *reinterpret_cast<const uint4*>(src + j * (2 * 16 * kStLd)));
            const int pos = kp0 + 16 * kt + rr;
            const bool ok = pos < cnt;
            bf16_t* base = mat == 0 ? dvp : dkp;
            uint4* px = reinterpret_cast<uint4*>((ok ? base + int64_t(pos) * kPartLd : dump + (4 * mat + g) * kBD) + 8 * c);
            if (!FIRST_TILE) x = add_bf16x8(x, *px);
            *px = x;
          }
          lds_barrier();  // slabs read before the next key tile's writes
        } else if (PAIR) {
          // both tiles' slabs of this key tile are complete; waves of the first tile store the dV rows,
          // waves of the second the dK rows, each the sum of the two slabs
          lds_barrier();
          const bf16_t* slab_a = stage + (w & 1) * (2 * 16 * kStLd) + tw * (16 * kStLd);        // first tile's wave
          const bf16_t* slab_b = stage + ((w & 1) + 2) * (2 * 16 * kStLd) + tw * (16 * kStLd);  // second tile's wave
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int rr = 4 * i + g;
            uint4 x = add_bf16x8(*reinterpret_cast<const uint4*>(slab_a + rr * kStLd + 8 * c),
                                 *reinterpret_cast<const uint4*>(slab_b + rr * kStLd + 8 * c));
            const int pos = kp0 + 16 * kt + rr;
            const bool ok = pos < cnt;
            bf16_t* base = tw == 0 ? dvp : dkp;
            uint4* px = reinterpret_cast<uint4*>((ok ? base + int64_t(pos) * kPartLd : dump + (4 * tw + g) * kBD) + 8 * c);
            if (!FIRST_TILE) x = add_bf16x8(x, *px);
            *px = x;
          }
          lds_barrier();  // slabs read before the next key tile's writes
        } else {
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront", "local");  // LDS only: the wave's writes before its reads below
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int rr = 4 * i + g;  // key row of the tile; lane chunk c = 16 bytes of it
          uint4 xv = *reinterpret_cast<const uint4*>(slab + rr * kStLd + 8 * c);
          uint4 xk = *reinterpret_cast<const uint4*>(slab + (16 + rr) * kStLd + 8 * c);
          const int pos = kp0 + 16 * kt + rr;
          const bool ok = pos < cnt;
          uint4* pv = reinterpret_cast<uint4*>((ok ? dvp + int64_t(pos) * kPartLd : dump + g * kBD) + 8 * c);
          uint4* pk = reinterpret_cast<uint4*>((ok ? dkp + int64_t(pos) * kPartLd : dump + (4 + g) * kBD) + 8 * c);
          if (!FIRST_TILE) {  // (compile time: a load here, even skipped, would make every store wait)
            xv = add_bf16x8(xv, *pv);
            xk = add_bf16x8(xk, *pk);
          }
          *pv = xv;
          *pk = xk;
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront", "local");  // reads done before the next tile's writes
        }
      } else {
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
          const f32x4 tv = M::m16k16(pA, doT[t], z);
          const f32x4 tk = M::m16k16(dsA, qT[t], z);
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (rok[r]) {
              unsafeAtomicAdd(dVb + rowoff[r] + 16 * t, tv[r]);
              unsafeAtomicAdd(dKb + rowoff[r] + 16 * t, tk[r]);
            }
        }
      }
    }
  };

  // ---- main loop: this wave's blocks w, w+4, ..., one block in flight ----
  if (STAGED) {
    // Two workgroups share a CU (the kernel is held to 256 registers per lane): while one wave waits
    // for its block, the waves of the other workgroup compute.  A wave keeps one block in registers
    // and has the list rows of its next block on the way.
    BwdBlock ra;
    if (QUAD) {
      int rows_nx = rows_of(0);
      for (int b = 0; b < nblk; ++b) {
        const int rows = rows_nx;
        rows_nx = rows_of(b + 1);
        bwd_load_block(ra, Kb, Vb, rows, g, c);
        compute(ra, b);
      }
    } else if (PAIR && LDSBLK) {
      const int par = w & 1;  // the parity of this wave's blocks; waves par and par + 2 walk them together
      const lds_char_t* const blk_l = (lds_char_t*)blk;
      const uint32_t blk0 = __builtin_amdgcn_readfirstlane(uint32_t(uintptr_t(blk_l)));
      const uint32_t kbuf = uint32_t(par) * 16384u, vbuf = kbuf + 8192u;  // byte offsets inside blk
      // wave par brings the K rows of a block, wave par + 2 its V rows: 8 loads of 4 rows each
      const bf16_t* src = ring_uniform_ptr(w < 2 ? Kb : Vb);
      const uint32_t dst = blk0 + (w < 2 ? kbuf : vbuf);
      auto swz = [](int r) { return ((r & 7) << 1) | ((r >> 3) & 1); };
      auto issue = [&](int rows) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int r = 4 * j + g;  // row of the block this lane's 16 bytes belong to; its position in the row: c
          const uint32_t key = uint32_t(__shfl(rows, r));
          ring_load16(dst + uint32_t(j) * 1024u, key * 256u + uint32_t((c ^ swz(r & 15)) * 16), src);
        }
      };
      auto rd = [&](uint32_t a) {
        const ring_u32x4 x = *reinterpret_cast<const __attribute__((address_space(3))) ring_u32x4*>(blk_l + a);
        return make_uint4(x.x, x.y, x.z, x.w);
      };
      auto fill = [&](BwdBlock& r, int rows) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          const uint32_t row = uint32_t(kt * 16 + c) * 256u;
          const int f = swz(c);
#pragma unroll
          for (int s2 = 0; s2 < 4; ++s2) {
            const uint32_t at = row + uint32_t(((4 * s2 + g) ^ f) * 16);
            r.k[kt][s2] = rd(kbuf + at);
            r.vk[kt][s2] = rd(vbuf + at);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int r2 = kt * 16 + 4 * g + j;
            r.kc[kt][j] = rd(kbuf + uint32_t(r2) * 256u + uint32_t((c ^ swz(r2 & 15)) * 16));
          }
          r.rk[kt] = __shfl(rows, kt * 16 + c);
        }
      };
      const int nb2 = (nblk + 1) & ~1;
      int rows_nx = rows_of(par + 2);
      {
        const int rows0 = rows_of(par);
        issue(rows0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        ring_barrier();
        fill(ra, rows0);
      }
      for (int b = par; b < nb2; b += 2) {
        const int rows_nx2 = rows_of(b + 4);  // (an ordinary load: older than the block's loads below)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's operands have left LDS ...
        ring_barrier();                                      // ... and so have the other waves'
        issue(rows_nx);  // block b + 2 (past the end: clamped rows, never used)
        compute(ra, b);
        // the block's loads are older than the eight partial-row stores of compute(): they have landed once at
        // most eight operations are outstanding (a wave's vector memory operations complete in order)
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        ring_barrier();
        fill(ra, rows_nx);
        rows_nx = rows_nx2;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else if (PAIR) {
      // every wave makes the same number of trips (the barriers inside): a block past the end is
      // clamped, contributes zeros and stores to the dump rows
      int rows_nx = rows_of(w & 1);
      for (int b = w & 1; b < ((nblk + 1) & ~1); b += 2) {
        const int rows = rows_nx;
        rows_nx = rows_of(b + 2);
        bwd_load_block(ra, Kb, Vb, rows, g, c);
        compute(ra, b);
      }
    } else {
      int rows_nx = rows_of(w);
      for (int b = w; b < nblk; b += 4) {
        const int rows = rows_nx;
        rows_nx = rows_of(b + 4);
        bwd_load_block(ra, Kb, Vb, rows, g, c);
        compute(ra, b);
      }
    }
  } else {
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
  }

  // ---- dQ: add the four waves' partial sums, write the tile's rows ----
  if (STAGED) __syncthreads();  // red shares its LDS with the waves' staging slabs: every wave is past its blocks
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((w * 8 + t) * 4 + r) * 64 + l] = dQ[t][r];
  __syncthreads();
  if (QUAD) {
    // a wave holds all of its tile's sums
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float o[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) o[t] = red[((w * 8 + t) * 4 + r) * 64 + l];
      if (myq >= 0)
        *reinterpret_cast<uint4*>(dq + (qbase + myq) * kBD + 32 * g + 8 * r) =
            make_uint4(M::pack2(o[0], o[1]), M::pack2(o[2], o[3]), M::pack2(o[4], o[5]), M::pack2(o[6], o[7]));
    }
    return;
  }
  if (PAIR) {
    // the two waves of a tile add their sums; wave parity p finalises accumulator rows 2p and 2p+1
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      const int r = 2 * (w & 1) + rr;
      float o[8];
#pragma unroll
      for (int t = 0; t < 8; ++t)
        o[t] = red[(((2 * tw) * 8 + t) * 4 + r) * 64 + l] + red[(((2 * tw + 1) * 8 + t) * 4 + r) * 64 + l];
      if (myq >= 0)
        *reinterpret_cast<uint4*>(dq + (qbase + myq) * kBD + 32 * g + 8 * r) =
            make_uint4(M::pack2(o[0], o[1]), M::pack2(o[2], o[3]), M::pack2(o[4], o[5]), M::pack2(o[6], o[7]));
    }
    return;
  }
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
        make_uint4(M::pack2(o[0], o[1]), M::pack2(o[2], o[3]), M::pack2(o[4], o[5]), M::pack2(o[6], o[7]));
}

// grid (items, FM_QTILE / 16): one workgroup per (work item, 16-query tile); dK, dV by atomic adds.
// F16: q, k, v, out, dout and dq are fp16 (else bf16).
template <bool F16>
__global__ __launch_bounds__(256) void hash_attn_bwd_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off, const int32_t* __restrict__ bucket_cnt,
    const int32_t* __restrict__ q_perm, const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    const bf16_t* __restrict__ out, const float* __restrict__ lse, const bf16_t* __restrict__ dout,
    const float* __restrict__ dlse, bf16_t* __restrict__ dq, float* __restrict__ dk, float* __restrict__ dv, int Sq, int N, int C, float sm_scale) {
  __shared__ __attribute__((aligned(16))) float red[4 * 8 * 4 * 64];  // dQ partials [wave][t][r][lane]
  __shared__ int q_rows[16];
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int q0 = int(blockIdx.y) * 16;  // this workgroup's query tile inside the item
  if (q0 >= it.n_q) return;
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  bwd_tile<false, true, 1, false, F16>(q, out, lse, dout, dlse, q_perm + it.q_start + q0, min(16, it.n_q - q0), int64_t(it.row) * Sq,
                  k + int64_t(it.row) * N * kBD, v + int64_t(it.row) * N * kBD, k_idx + bucket_off[bkt],
                  bucket_cnt[bkt], N, sm_scale, dq, dk + int64_t(it.row) * N * kBD, dv + int64_t(it.row) * N * kBD,
                  nullptr, nullptr, nullptr, red, q_rows, nullptr);
}

// grid (C, rows): one workgroup per (row, bucket) takes the bucket's query tiles one after the other;
// dK, dV partial rows of the bucket go to dkp / dvp + (flat list position - pos0) * kPartLd (dvp = dkp + kBD:
// the two rows of a position are 512 contiguous bytes, which the reduction reads together); dump: 8 rows of
// 128 bf16 that take the stores of a block's positions past the end of a list.
// MAXT: the most tiles a pass takes (2 or 4).  The four-tile form costs registers in every path of the
// kernel that holds it, so it is only launched where buckets receive more than 24 queries on average.
constexpr int kStagedMaxQ = 256;  // queries of a bucket that go through its bf16 partial rows

// LDSBLK: the kernel whose two-tile first pass takes its blocks through LDS.  The two-tile kernels have a compute
// unit to themselves (one workgroup of four waves, all the registers a lane can have, nothing spilled): with two
// workgroups at 256 registers each their 96 / 138 spilled registers cost more than the second workgroup hides
// (c5: 94.5 against 91.8 ms; c4: 11.4 against 10.9 ms).  The four-tile kernel keeps two workgroups per CU
// (c2: 1.3 against 1.6 ms).
template <int MAXT, bool LDSBLK, bool F16 = false>
__global__ __launch_bounds__(256, MAXT == 4 ? 2 : 1) void hash_attn_bwd_staged_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off, const int32_t* __restrict__ bucket_cnt,
    const int32_t* __restrict__ q_perm, const int32_t* __restrict__ bin_off, const int32_t* __restrict__ bin_count,
    const bf16_t* __restrict__ out, const float* __restrict__ lse, const bf16_t* __restrict__ dout,
    const float* __restrict__ dlse, bf16_t* __restrict__ dq, bf16_t* dkp, bf16_t* dvp, bf16_t* dump, int64_t pos0, int row0, int Sq, int N, int C,
    float sm_scale) {
  // the waves' staging slabs ([wave][dV | dK][16][kStLd] bf16) during a tile's blocks, then the dQ partial
  // sums ([wave][t][r][lane] fp32) at its end
  __shared__ __attribute__((aligned(16))) unsigned char lds_buf[4 * 2 * 16 * kStLd * sizeof(bf16_t)];
  static_assert(sizeof(lds_buf) >= 4 * 8 * 4 * 64 * sizeof(float), "dQ partials fit the staging slabs");
  __shared__ int q_rows[16 * MAXT];
  __shared__ __attribute__((aligned(16))) unsigned char blk[LDSBLK ? 32768 : 16];
  float* red = reinterpret_cast<float*>(lds_buf);
  bf16_t* stage = reinterpret_cast<bf16_t*>(lds_buf);
  const int row = row0 + blockIdx.y;
  const int64_t bkt = int64_t(row) * C + blockIdx.x;
  const int nq = bin_count[bkt];
  const int64_t off = bucket_off[bkt];
  if (nq <= 0) {  // nobody hashed here: the bucket contributes zero rows
    const int64_t n16 = int64_t(bucket_cnt[bkt]) * (kPartLd * sizeof(bf16_t) / 16);
    uint4* z = reinterpret_cast<uint4*>(dkp + (off - pos0) * kPartLd);
    for (int64_t i = threadIdx.x; i < n16; i += 256) z[i] = make_uint4(0, 0, 0, 0);
    return;
  }
  const int32_t* ql = q_perm + bin_off[bkt];
  const bf16_t* Kb = k + int64_t(row) * N * kBD;
  const bf16_t* Vb = v + int64_t(row) * N * kBD;
  const int cnt = bucket_cnt[bkt];
  bf16_t* dkb = dkp + (off - pos0) * kPartLd;
  bf16_t* dvb = dvp + (off - pos0) * kPartLd;
  // the first pass stores the bucket's partial rows, the others add to them; a pass takes up to MAXT tiles.
  // The partial rows are bf16 and every pass after the first rounds them again, so only the first
  // kStagedMaxQ queries of a bucket go through them; a bucket that receives more (a heavily skewed hash)
  // adds the rest straight into dK / dV with fp32 atomic adds (hash_attn_bwd_excess_kernel).
  const int nq_staged = min(nq, kStagedMaxQ);
  for (int q0 = 0; q0 < nq_staged; q0 += 16 * MAXT) {
    if (q0) __syncthreads();  // red and q_rows are reused
    const int left = nq_staged - q0;
#define FM_BWD_PASS(FIRST, NT)                                                                                        \
  bwd_tile<true, FIRST, NT, false, F16>(q, out, lse, dout, dlse, ql + q0, min(16 * NT, left), int64_t(row) * Sq, Kb, Vb, k_idx + off,  \
                            cnt, N, sm_scale, dq, nullptr, nullptr, dkb, dvb, dump, red, q_rows, stage)
    if (MAXT == 4 && left > 32) {
      if (q0 == 0)
        FM_BWD_PASS(true, MAXT);  // (MAXT, not 4: the two-tile kernel does not instantiate this form)
      else
        FM_BWD_PASS(false, MAXT);
    } else if (LDSBLK && q0 == 0 && left > 16) {
      // the first pass of a bucket with 17 to 32 queries, its rows through LDS
      bwd_tile<true, true, 2, LDSBLK, F16>(q, out, lse, dout, dlse, ql, min(32, left), int64_t(row) * Sq, Kb, Vb, k_idx + off,
                                      cnt, N, sm_scale, dq, nullptr, nullptr, dkb, dvb, dump, red, q_rows, stage, blk);
    } else if (left > 16) {
      if (q0 == 0)
        FM_BWD_PASS(true, 2);
      else
        FM_BWD_PASS(false, 2);
    } else {
      if (q0 == 0)
        FM_BWD_PASS(true, 1);
      else
        FM_BWD_PASS(false, 1);
    }
#undef FM_BWD_PASS
  }
}

// grid (C, rows): the queries of a bucket beyond the first kStagedMaxQ, 16 at a time, with atomic adds into
// dK / dV; a workgroup whose bucket has no such query (nearly all of them) reads one word and leaves.
template <bool F16>
__global__ __launch_bounds__(256) void hash_attn_bwd_excess_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off, const int32_t* __restrict__ bucket_cnt,
    const int32_t* __restrict__ q_perm, const int32_t* __restrict__ bin_off, const int32_t* __restrict__ bin_count,
    const bf16_t* __restrict__ out, const float* __restrict__ lse, const bf16_t* __restrict__ dout,
    const float* __restrict__ dlse, bf16_t* __restrict__ dq, float* __restrict__ dk, float* __restrict__ dv, int row0,
    int Sq, int N, int C, float sm_scale) {
  __shared__ __attribute__((aligned(16))) float red[4 * 8 * 4 * 64];
  __shared__ int q_rows[16];
  const int row = row0 + blockIdx.y;
  const int64_t bkt = int64_t(row) * C + blockIdx.x;
  const int nq = bin_count[bkt];
  if (nq <= kStagedMaxQ) return;
  const int32_t* ql = q_perm + bin_off[bkt];
  for (int q0 = kStagedMaxQ; q0 < nq; q0 += 16) {
    if (q0 > kStagedMaxQ) __syncthreads();  // red and q_rows are reused
    bwd_tile<false, true, 1, false, F16>(q, out, lse, dout, dlse, ql + q0, min(16, nq - q0), int64_t(row) * Sq,
                          k + int64_t(row) * N * kBD, v + int64_t(row) * N * kBD, k_idx + bucket_off[bkt],
                          bucket_cnt[bkt], N, sm_scale, dq, dk + int64_t(row) * N * kBD, dv + int64_t(row) * N * kBD,
                          nullptr, nullptr, nullptr, red, q_rows, nullptr);
  }
}

bool hash_attn_bwd_mfma_supported(int d, int dtype) { return d == kBD && (dtype == FM_BF16 || dtype == FM_F16); }

int hash_attn_bwd_mfma(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                       const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                       int64_t max_items, const void* out, const float* lse, const void* dout, const float* dlse, void* dq,
                       float* dk, float* dv, int Sq, int N, int C, float sm_scale, bool f16, hipStream_t st) {
  dim3 grid = dim3(unsigned(max_items), unsigned(FM_QTILE / 16));
  if (f16)
    hipLaunchKernelGGL(hash_attn_bwd_mfma_kernel<true>, grid, dim3(256), 0, st, (const bf16_t*)q, (const bf16_t*)k,
                       (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, (const bf16_t*)out, lse,
                       (const bf16_t*)dout, dlse, (bf16_t*)dq, dk, dv, Sq, N, C, sm_scale);
  else
    hipLaunchKernelGGL(hash_attn_bwd_mfma_kernel<false>, grid, dim3(256), 0, st, (const bf16_t*)q, (const bf16_t*)k,
                       (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, (const bf16_t*)out, lse,
                       (const bf16_t*)dout, dlse, (bf16_t*)dq, dk, dv, Sq, N, C, sm_scale);
  return launch_status("fm_hash_attn_bwd(mfma)");
}

int hash_attn_bwd_staged_partials(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                  const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                                  const int32_t* bin_off, const int32_t* bin_count, const void* out, const float* lse,
                                  const void* dout, const float* dlse, void* dq, void* dkp, void* dvp, void* dump, int64_t pos0,
                                  int row0, int rows, int Sq, int N, int C, float sm_scale, float* dk, float* dv,
                                  bool f16, hipStream_t st) {
#define FM_BWD_STAGED(MAXT, LB)                                                                                    \
  do {                                                                                                             \
  if (f16)                                                                                                         \
    hipLaunchKernelGGL((hash_attn_bwd_staged_kernel<MAXT, LB, true>), dim3(unsigned(C), unsigned(rows)), dim3(256), 0, st, \
                       (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm,  \
                       bin_off, bin_count, (const bf16_t*)out, lse, (const bf16_t*)dout, dlse, (bf16_t*)dq, (bf16_t*)dkp,  \
                       (bf16_t*)dvp, (bf16_t*)dump, pos0, row0, Sq, N, C, sm_scale);                                  \
  else                                                                                                             \
  hipLaunchKernelGGL((hash_attn_bwd_staged_kernel<MAXT, LB, false>), dim3(unsigned(C), unsigned(rows)), dim3(256), 0, st, \
                     (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm,  \
                     bin_off, bin_count, (const bf16_t*)out, lse, (const bf16_t*)dout, dlse, (bf16_t*)dq, (bf16_t*)dkp,  \
                     (bf16_t*)dvp, (bf16_t*)dump, pos0, row0, Sq, N, C, sm_scale);                                    \
  } while (0)
  if (int64_t(Sq) > 24 * int64_t(C))  // more than 24 queries per bucket on average
    FM_BWD_STAGED(4, false);
  else if (N < (1 << 24) && int64_t(Sq) > 12 * int64_t(C) && g_force_generic != 9)
    // rows addressed by 32-bit byte offsets in the loads that write LDS; and enough buckets with more than 16
    // queries to pay for the registers the extra form costs the others (12 queries per bucket on average: a
    // fifth of the buckets of evenly hashed queries; at 8 the form costs 2 %, at 16 it gains 8 %)
    FM_BWD_STAGED(2, true);
  else
    FM_BWD_STAGED(2, false);
#undef FM_BWD_STAGED
  if (Sq > kStagedMaxQ) {  // some bucket may hold more queries than go through its partial rows
    if (f16)
      hipLaunchKernelGGL(hash_attn_bwd_excess_kernel<true>, dim3(unsigned(C), unsigned(rows)), dim3(256), 0, st,
                         (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm,
                         bin_off, bin_count, (const bf16_t*)out, lse, (const bf16_t*)dout, dlse, (bf16_t*)dq, dk, dv, row0,
                         Sq, N, C, sm_scale);
    else
      hipLaunchKernelGGL(hash_attn_bwd_excess_kernel<false>, dim3(unsigned(C), unsigned(rows)), dim3(256), 0, st,
                         (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm,
                         bin_off, bin_count, (const bf16_t*)out, lse, (const bf16_t*)dout, dlse, (bf16_t*)dq, dk, dv, row0,
                         Sq, N, C, sm_scale);
  }
  return launch_status("fm_hash_attn_bwd_staged(partials)");
}

}  // namespace fm
