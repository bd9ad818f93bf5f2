// bf16 / fp16 bucket-gathered attention forward for head dimension 128 (gfx950), the form for buckets
// that receive many queries (triton_kernel.py:137-272; the shape of the reference's own performance
// harness, triton_kernel.py:507-528, has 128 queries per bucket).  Same arithmetic and operand layout
// as attn_staged.hpp; what differs is how a bucket's rows reach LDS.
//
// In attn_staged.hpp a tile's rows wait in registers between their load and their place in LDS (32
// registers a thread) and V is transposed on the way with VALU work.
// Here the rows go from global memory straight into LDS (global_load_lds_dwordx4: lane i of a wave's
// load writes 16 bytes at M0 + 16 i):
//   * LDS holds two tiles of 64 keys (K and V, 64 rows x 256 B each): the one being read and the next,
//     on its way while this one is computed.  One barrier per tile.
//   * Rows are stored unpadded (a wave's load writes 1 KiB = 4 whole rows), so bank conflicts are
//     avoided by position instead: 16-byte chunk q of row r sits at position q ^ f(r),
//     f(r) = ((r & 7) << 1) | ((r >> 3) & 1).  The lane that loads position p of row r asks global memory
//     for chunk p ^ f(r).  The 16 lanes that read one chunk column of 16 consecutive rows (the K operand)
//     then hit 16 different positions, and the 8 consecutive rows x 32 B that half a wave reads for
//     the V operand cover all banks once.
//   * V stays row-major: ds_read_b64_tr_b16 hands the MFMA its V^T operand.  Within each group of 16
//     lanes, lane i names 8 bytes (4 elements); lane j receives element j % 4 of the rows named by lanes
//     j / 4 + {0, 4, 8, 12}.  With lane i naming elements 4 (i % 4) .. + 3 (of a 16-wide slice of the
//     head dimension) of key i / 4 of the group's 4 keys, lane j holds element j of the slice for
//     those 4 keys: the A operand of O^T += V^T P^T, with no transposition in registers.
//   * The list entries (row numbers) of a tile also travel by such a load (global_load_lds_dword, one
//     per wave and tile into two 256-byte buffers of the wave's own), one tile ahead of the rows.
//   * The compiler knows nothing of these loads, which is why they are inline assembly: for its own
//     LDS-writing loads it waits for all of them before any LDS read, here also before the reads of
//     the tile being computed.  The one wait there is (vmcnt(0) in front of the barrier) is written by hand.
//
// Per tile t: wait for this wave's loads, barrier (tile t is in place; every wave has finished tile
// t - 1, whose buffers are free), request tile t + 1 and the list entries of tile t + 2, then
// S^T = K Q^T, the softmax and O^T += V^T P^T.
//
// A wave takes up to three tiles of 16 queries (a workgroup 192 queries: three consecutive work items of a
// bucket), dealt to the waves in turn so that their shares differ by one tile at most, and runs a copy of the
// loop compiled for the number of tiles it has.  250 registers, none spilled: a spill inside the loop would be
// reloaded by a vector-memory instruction, and the wait for it would also wait for the rows on their way.
//
// Measured at the reference's harness shape (fp16, 128 queries per bucket on average, half of the buckets
// above 128, 3072 keys): 2.51 ms against 3.05 ms for the staged kernel with two items per workgroup (2.62 ms
// with two tiles per wave, where a bucket of 129-192 queries was swept by two workgroups).
#pragma once
#include <type_traits>

#include "attn_staged.hpp"

namespace fm {

typedef __attribute__((address_space(3))) char lds_char_t;
typedef short ring_short4 __attribute__((ext_vector_type(4)));
typedef unsigned int ring_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kRSlotBytes = 64 * 256;  // 64 rows of 128 two-byte elements
constexpr int kRIdsBytes = 4 * 2 * 256;  // four waves, two tiles of list entries each
constexpr size_t kRingLdsBytes = size_t(kRIdsBytes) + 4 * kRSlotBytes;

// s_barrier alone (no wait for outstanding loads); the compiler may not move memory accesses across it
__device__ __forceinline__ void ring_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// M0 is written inside the statements below and is not on their clobber lists: it is a reserved register of
// the AMDGPU backend, which keeps no value live in it across an asm statement (it rewrites M0 right in front
// of each of its own uses) and rejects it as a clobber with a warning per statement.
// lane i of the wave: 16 bytes from base + voff(i) to LDS byte address lds_addr + 16 i
__device__ __forceinline__ void ring_load16(uint32_t lds_addr, uint32_t voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(base)
               : "memory");
}
// lane i of the wave: 4 bytes from base + voff(i) to LDS byte address lds_addr + 4 i
__device__ __forceinline__ void ring_load4(uint32_t lds_addr, uint32_t voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(base)
               : "memory");
}

template <typename T>
__device__ __forceinline__ const T* ring_uniform_ptr(const T* p) {
  const uint64_t u = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(uint32_t(u)), hi = __builtin_amdgcn_readfirstlane(uint32_t(u >> 32));
  return reinterpret_cast<const T*>(uint64_t(lo) | (uint64_t(hi) << 32));
}

// The attention of n_q <= 64 NQW queries (rows q_rows[0..n_q) of Qb / Ob / Lb) over the cnt keys
// idx[0..cnt) of one bucket; called by all 256 threads of a workgroup (a wave takes up to NQW <= 3 tiles of
// 16 queries), lds = kRingLdsBytes of LDS.
// Rows are addressed by 32-bit byte offsets: N * 256 < 2^32 (checked by the host).
template <int NQW, bool F16>
__device__ __forceinline__ void attend_ring(const bf16_t* __restrict__ Qb, const int* __restrict__ q_rows, int n_q,
                                            const bf16_t* Kb, const bf16_t* Vb, const int32_t* idx, int cnt, int N,
                                            float scale2, bf16_t* __restrict__ Ob, float* __restrict__ Lb,
                                            bf16_t* lds_generic, int rot) {
  lds_char_t* const lds = (lds_char_t*)lds_generic;
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane(uint32_t(uintptr_t(lds)));
  const int tid = threadIdx.x, l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = l >> 4, c = l & 15;
  const int ntiles = (cnt + 63) >> 6;
  Kb = ring_uniform_ptr(Kb);
  Vb = ring_uniform_ptr(Vb);
  idx = ring_uniform_ptr(idx);
  auto swz = [](int r) { return ((r & 7) << 1) | ((r >> 3) & 1); };

  // ---- this lane's queries (column c of each of wave w's NQW tiles) ----
  // The 16-query tiles are dealt to the waves in turn, tile j to wave (j + rot) % 4 as its tile j / 4, so a
  // wave's share differs from another's by one tile at most (9 tiles: 3, 2, 2, 2), and `rot` (the caller
  // passes the bucket number) moves the wave with the extra tile, and with it the SIMD, from bucket to bucket.
  const int wl = (w - rot) & 3;
  const int n_qt = (n_q + 15) >> 4;
  const int nqt_w = min(max((n_qt - wl + 3) >> 2, 0), NQW);  // tiles of this wave that hold queries
  uint4 qf[NQW][4];
#pragma unroll
  for (int qt = 0; qt < NQW; ++qt) {
    const int jq = 16 * (wl + 4 * qt) + c;
    const bool ok = jq < n_q;
    const int64_t qrow = ok ? q_rows[jq] : 0;
    const uint4* pq = reinterpret_cast<const uint4*>(Qb + qrow * kSD + 8 * g);
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[qt][s] = ok ? pq[4 * s] : make_uint4(0, 0, 0, 0);
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

  // (the wait for the query fragments goes here, in front of the rows' loads: one placed after them would
  // wait for those too)
#pragma unroll
  for (int qt = 0; qt < NQW; ++qt)
#pragma unroll
    for (int s = 0; s < 4; ++s)
      asm volatile("" ::"v"(qf[qt][s].x), "v"(qf[qt][s].y), "v"(qf[qt][s].z), "v"(qf[qt][s].w));

  // ---- loads: K or V of a tile is 16 loads of 4 rows; wave w issues loads w, w + 4, ..: lane l takes position
  // l % 16 of row 16 u + 4 w + l / 16 ----
  const int lr = 4 * w + (l >> 4);                                // the row modulo 16
  const uint32_t ld_chunk = uint32_t(((l & 15) ^ swz(lr)) << 4);  // byte offset of the chunk this lane asks for
  const uint32_t ids_lds = lds0 + uint32_t(w) * 512u;
  const uint32_t ring_lds = lds0 + kRIdsBytes;
  auto issue_ids = [&](int t) {
    const int kp = min(t * 64 + l, cnt - 1);  // entries past the end of the list repeat the last one (their scores are masked)
    ring_load4(ids_lds + uint32_t(t & 1) * 256u, uint32_t(kp) * 4u, idx);
  };
  uint32_t rows[4];  // byte offsets of this lane's four rows of a tile
  auto read_rows = [&](int t) {
    const lds_char_t* p = lds + (2 * w + (t & 1)) * 256 + lr * 4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int a = *reinterpret_cast<const __attribute__((address_space(3))) int*>(p + 64 * u);
      rows[u] = (uint32_t(min(max(a, 0), N - 1)) << 8) | ld_chunk;  // (a list may hold any int: clamp, as the other kernels do)
    }
  };
  // K and V of a tile into buffer pair `par` (slots 2 par and 2 par + 1)
  auto issue_tile = [&](int par) {
    const uint32_t dst = ring_lds + uint32_t(2 * par) * kRSlotBytes + uint32_t(w) * 1024u;
#pragma unroll
    for (int u = 0; u < 4; ++u) ring_load16(dst + uint32_t(u) * 4096u, rows[u], Kb);
#pragma unroll
    for (int u = 0; u < 4; ++u) ring_load16(dst + kRSlotBytes + uint32_t(u) * 4096u, rows[u], Vb);
  };

  // ---- operand addresses: K row 16 kt + c, chunk 4 st + g; V key 4 g + c / 4 of a 16-key tile ----
  const int kbase = c * 256 + ((g ^ swz(c)) << 4);  // ^ (st << 6): swz(c) < 16, and 4 st only has bits 2, 3
  const int vrl = 4 * g + (c >> 2);
  const int vbase = vrl * 256 + ((((c & 3) >> 1) ^ swz(vrl)) << 4) + (c & 1) * 8;  // ^ (t8 << 5)
  const lds_char_t* const ring = lds + kRIdsBytes;

  // (T_ = std::integral_constant: the number of this wave's query tiles the call works on)
  // (kb, vb: kbase and vbase through an empty asm statement of the caller, once per tile, so that the
  // 12 operand addresses are formed again with an XOR each instead of living in registers through the loop)
  auto scores = [&](auto T_, int t, int slot, int kb, f32x4 (&s)[NQW][4]) {
    constexpr int T = decltype(T_)::value;
    const lds_char_t* const bK = ring + slot * kRSlotBytes;
#pragma unroll
    for (int st = 0; st < 4; ++st) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const ring_u32x4 a_ =
            *reinterpret_cast<const __attribute__((address_space(3))) ring_u32x4*>(bK + kt * 4096 + (kb ^ (st << 6)));
        const uint4 a = make_uint4(a_[0], a_[1], a_[2], a_[3]);
#pragma unroll
        for (int qt = 0; qt < T; ++qt)
          s[qt][kt] = Mma<F16>::m16(a, qf[qt][st], st == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[qt][kt]);
      }
    }
    mfma_settle_scores<T>(s);  // (a branch follows: see mma16.hpp)
    const int kp0 = t * 64;
    if (kp0 + 64 > cnt) {  // the bucket's last, ragged tile
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (kp0 + 16 * kt + 4 * g + r >= cnt) {
#pragma unroll
            for (int qt = 0; qt < T; ++qt) s[qt][kt][r] = -INFINITY;
          }
    }
  };
  // online softmax as in attn_staged.hpp (triton_kernel.py:248-263)
  auto softmax = [&](auto T_, f32x4 (&s)[NQW][4], uint4 (&pf)[NQW][2]) {
    constexpr int T = decltype(T_)::value;
#pragma unroll
    for (int qt = 0; qt < T; ++qt) {
      float mx = st_max3(s[qt][0][0], s[qt][0][1], s[qt][0][2]);
      mx = st_max3(mx, s[qt][0][3], s[qt][1][0]);
      mx = st_max3(mx, s[qt][1][1], s[qt][1][2]);
      mx = st_max3(mx, s[qt][1][3], s[qt][2][0]);
      mx = st_max3(mx, s[qt][2][1], s[qt][2][2]);
      mx = st_max3(mx, s[qt][2][3], s[qt][3][0]);
      mx = st_max3(mx, s[qt][3][1], s[qt][3][2]);
      mx = st_max_lane_groups(st_max(mx, s[qt][3][3])) * scale2;
      const float m_new = fmaxf(m[qt], mx);
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
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
  };
  auto weighted_values = [&](auto T_, int slot, int vb, const uint4 (&pf)[NQW][2]) {
    constexpr int T = decltype(T_)::value;
    const lds_char_t* const bV = ring + slot * kRSlotBytes;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int t8 = 0; t8 < 8; ++t8) {
        // contraction slots 8g .. 8g+3: keys 4g .. 4g+3 of key tile 2h; slots 8g+4 .. 8g+7: the same of key tile 2h+1
        const lds_char_t* p = bV + h * 8192 + (vb ^ (t8 << 5));
        const ring_short4 lo =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ring_short4*)p);
        const ring_short4 hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ring_short4*)(p + 4096));
        union {
          ring_short4 s4[2];
          uint4 u;
        } a;
        a.s4[0] = lo;
        a.s4[1] = hi;
#pragma unroll
        for (int qt = 0; qt < T; ++qt) O[qt][t8] = Mma<F16>::m16(a.u, pf[qt][h], O[qt][t8]);
      }
    }
  };

  // The work of a wave that has T of its NQW query tiles: the loop over the bucket's tiles and the
  // write-out, compiled once for every T so that a wave runs neither MFMAs nor softmax for tiles it does
  // not have (the waves of a workgroup meet at the barriers all the same: every copy has one per tile).
  auto run = [&](auto T_) {
    constexpr int T = decltype(T_)::value;
    if (ntiles > 0) {
      // ---- prologue: list entries of tile 0, then tile 0 and the list entries of tile 1 ----
      issue_ids(0);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      read_rows(0);
      if (ntiles > 1) issue_ids(1);
      issue_tile(0);
      // two tiles per round, so that the buffers are compile-time constants
      for (int t0 = 0; t0 < ntiles; t0 += 2) {
#pragma unroll
        for (int par = 0; par < 2; ++par) {
          const int t = t0 + par;
          if (t >= ntiles) break;
          f32x4 s_[NQW][4];
          uint4 pf_[NQW][2];
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          ring_barrier();  // tile t is in place (and this wave's list entries of tile t + 1); every wave has finished tile t - 1
          if (t + 1 < ntiles) {
            read_rows(t + 1);
            if (t + 2 < ntiles) issue_ids(t + 2);
            issue_tile(1 - par);
          }
          if (T > 0) {
            constexpr int TT = T > 0 ? T : 1;
            int kb = kbase, vb = vbase;
            asm volatile("" : "+v"(kb), "+v"(vb));
            scores(std::integral_constant<int, TT>{}, t, 2 * par, kb, s_);
            softmax(std::integral_constant<int, TT>{}, s_, pf_);
            weighted_values(std::integral_constant<int, TT>{}, 2 * par + 1, vb, pf_);
          }
        }
      }
    }
    // ---- finish: lane (g,c) holds dims 16t + 4g + r of query c of each tile ----
#pragma unroll
    for (int qt = 0; qt < T; ++qt) {
      float ltot = lsum[qt] + __shfl_xor(lsum[qt], 16);
      ltot += __shfl_xor(ltot, 32);
      const bool empty = (m[qt] == -INFINITY);
      const float inv = empty ? 0.f : 1.f / ltot;
      const int jq = 16 * (wl + 4 * qt) + c;  // (looked up again rather than kept in registers through the loop)
      if (jq < n_q) {
        const int64_t qrow = q_rows[jq];
        bf16_t* po = Ob + qrow * kSD + 4 * g;
#pragma unroll
        for (int t8 = 0; t8 < 8; ++t8) {
          uint2 o;
          o.x = Mma<F16>::pack2(O[qt][t8][0] * inv, O[qt][t8][1] * inv);
          o.y = Mma<F16>::pack2(O[qt][t8][2] * inv, O[qt][t8][3] * inv);
          *reinterpret_cast<uint2*>(po + 16 * t8) = o;
        }
        if (g == 0) Lb[qrow] = empty ? -FLT_MAX : (m[qt] + __builtin_amdgcn_logf(ltot)) * kLn2;
      }
    }
  };
  if (nqt_w == NQW)
    run(std::integral_constant<int, NQW>{});
  else if (NQW > 1 && nqt_w == NQW - 1)
    run(std::integral_constant<int, (NQW > 1 ? NQW - 1 : 0)>{});
  else if (NQW > 2 && nqt_w == NQW - 2)
    run(std::integral_constant<int, (NQW > 2 ? NQW - 2 : 0)>{});
  else
    run(std::integral_constant<int, 0>{});
}

}  // namespace fm
