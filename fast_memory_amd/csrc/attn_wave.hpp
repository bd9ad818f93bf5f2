// bf16 / fp16 bucket-gathered attention forward for head dimension 128 (gfx950), the form for long lists
// that receive few queries each (triton_kernel.py:137-272): one WAVE per work item instead of one workgroup.
// Same arithmetic as attn_ring.hpp, same loads from global memory straight into LDS, same swizzled rows and
// the same V^T operand from ds_read_b64_tr_b16; what differs is who shares what.
//
// With 16 queries per bucket a workgroup of attn_ring.hpp has one wave that computes and four that load, and a
// compute unit sweeps two buckets at a time.  When every key row is listed in many buckets and the lists are
// in ascending key order, the buckets that are swept at the same time behind one L2 meet at the same rows: of
// the requests for a row, all but the first within a short time are answered by the L2.  How many they are is
// the number of buckets in flight behind that L2 times the share of the keys a bucket lists; two per compute
// unit leave most requests to the fabric.  Here every wave sweeps a bucket of its own: eight per compute unit,
// four times as many meetings.
//
//   * A wave owns 16.5 KiB of LDS: two buffers of 64 list entries and two tiles of 16 keys (K and V, 16 rows x
//     256 B each), the one being read and the next, on its way while this one is computed.
//   * No barriers: a wave waits for its own loads (s_waitcnt vmcnt(0), written by hand as in attn_ring.hpp)
//     and for nothing else.
//   * A tile's K is four loads of 4 rows: lane l takes position l % 16 of row 4 u + l / 16 and asks global
//     memory for chunk (l % 16) ^ f(row), f as in attn_ring.hpp.
//   * S^T = K Q^T is four v_mfma_f32_16x16x32 per 16 queries (the head dimension in four steps); the tile has
//     16 keys, so O^T += V^T P^T contracts over 16 and uses v_mfma_f32_16x16x16 (eight per 16 queries), whose B
//     operand is the S^T accumulator of the lane as it stands: four keys of one query.
//   * The list entries come 64 at a time (four tiles), two tiles or more before their first use.
//
// A wave takes up to three tiles of 16 queries and runs a copy of the loop compiled for the number it has; the
// caller sweeps an item of more than 48 queries twice.
#pragma once
#include "attn_ring.hpp"

namespace fm {

constexpr int kWTileBytes = 16 * 256;                  // 16 rows of 128 two-byte elements
constexpr int kWWaveBytes = 512 + 4 * kWTileBytes;     // two buffers of list entries, two tiles of K and V
constexpr size_t kWaveLdsBytes = size_t(4) * kWWaveBytes;

// Pacing of the sweeps.  The requests of two buckets for one row meet in the L2 only while that row is still
// there, and the 4 MB of an L2 hold the rows of about 8000 consecutive keys: the waves behind one L2 have to
// sweep the key range within that distance of each other.  Left alone they do not -- entry i of a sorted list
// lies where the list's own density puts it (a standard deviation of 4000 keys in the middle of 16384 entries
// among 2^20 keys), and a wave with more queries takes longer per tile.  Talking to each other costs the waves
// more than it wins (a line that 256 waves read and write).  They share a clock, though (s_memrealtime, 100
// MHz, the same for every wave of the device): a launch has a schedule, key x is due t0 + x * ticks_per_key,
// and a wave asks for a tile only once its first key is due (less a margin).  Waves that are behind run free,
// waves that are ahead wait, and if the schedule is one the launch can keep, all of them sweep the key range
// together and the launch ends on schedule -- sooner than it ends unpaced (2^20 keys, 2048 buckets of 16384:
// 1.32 ms per launch unpaced, 0.94 ms on a schedule of 0.93 ms; on a schedule it cannot keep, a fifth to a half
// longer than unpaced: the waves that get behind no longer find their rows in the L2 and get further behind).
// Which schedule a launch can keep is found by trying (WavePaceSlot in attn_mfma_wave.hip).  A wait ends after kWaveGateTicks at the
// latest and a wave stops pacing after kWaveLongWaits such waits or kWaveSpinLimit looks at the clock in all
// (lists that do not ascend; a clock that stands still), so every wave ends whatever the clock says.  The
// clock only delays loads: results do not depend on it.
struct WaveClock {
  uint64_t t0;          // the launch's start
  float ticks_per_key;  // 0: unpaced
};
constexpr int kWaveMarginKeys = 2048;   // how far ahead of the schedule a wave may ask
constexpr int kWaveGateTicks = 2000;    // 20 us: the longest single wait
constexpr int kWaveLongWaits = 4;
constexpr int kWaveSpinLimit = 40000;

// (the slots an MFMA's result needs before a vector instruction may touch it: mfma_settle in mma16.hpp)
template <int T>
__device__ __forceinline__ void wave_mfma_settle(f32x4 (&x)[T]) {
  static_assert(T >= 1 && T <= 3, "one to three accumulators");
  if constexpr (T == 1)
    mfma_settle(x[0]);
  else if constexpr (T == 2)
    mfma_settle(x[0], x[1]);
  else
    mfma_settle(x[0], x[1], x[2]);
}

// The attention of n_q <= 16 NQW queries (rows q_rows[0..n_q) of Qb / Ob / Lb) over the cnt keys idx[0..cnt)
// of one bucket; called by the 64 lanes of one wave, lds_wave = kWWaveBytes of LDS that no other wave touches.
// Rows are addressed by 32-bit byte offsets: N * 256 <= 2^32 (checked by the host).
template <int NQW, bool F16>
__device__ __forceinline__ void attend_wave(const bf16_t* __restrict__ Qb, const int* __restrict__ q_rows, int n_q,
                                            const bf16_t* Kb, const bf16_t* Vb, const int32_t* idx, int cnt, int N,
                                            float scale2, bf16_t* __restrict__ Ob, float* __restrict__ Lb,
                                            lds_char_t* lds, const WaveClock clk) {
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane(uint32_t(uintptr_t(lds)));
  const int l = threadIdx.x & 63;
  const int g = l >> 4, c = l & 15;
  const int ntiles = (cnt + 15) >> 4;
  const int nblk = (cnt + 63) >> 6;  // blocks of 64 list entries
  Kb = ring_uniform_ptr(Kb);
  Vb = ring_uniform_ptr(Vb);
  idx = ring_uniform_ptr(idx);
  auto swz = [](int r) { return ((r & 7) << 1) | ((r >> 3) & 1); };

  // ---- this lane's queries (column c of each of the NQW tiles) ----
  const int n_qt = __builtin_amdgcn_readfirstlane(min((n_q + 15) >> 4, NQW));
  uint4 qf[NQW][4];
#pragma unroll
  for (int qt = 0; qt < NQW; ++qt) {
    const int jq = 16 * qt + c;
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

  // ---- loads: K or V of a tile is 4 loads of 4 rows; lane l takes position l % 16 of row 4 u + l / 16 ----
  const int la = l >> 4;
  const uint32_t ld_chunk = uint32_t(((l & 15) ^ swz(la)) << 4);  // for u = 0; f(4 u + a) = f(a) ^ 8 (u & 1) ^ (u >> 1)
  const uint32_t tiles_lds = lds0 + 512u;
  auto issue_ids = [&](int b) {
    const int kp = min(b * 64 + l, cnt - 1);  // entries past the end of the list repeat the last one (their scores are masked)
    ring_load4(lds0 + uint32_t(b & 1) * 256u, uint32_t(kp) * 4u, idx);
  };
  uint32_t rows[4];  // byte offsets of this lane's four rows of a tile
  int first_key = 0;  // the tile's first key (lane 0 reads entry 0 of the tile)
  auto read_rows = [&](int t) {
    const lds_char_t* p = lds + ((t >> 2) & 1) * 256 + (t & 3) * 64 + la * 4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int a = min(max(*reinterpret_cast<const __attribute__((address_space(3))) int*>(p + 16 * u), 0), N - 1);
      const uint32_t cu = uint32_t(((u & 1) << 3) | (u >> 1)) << 4;
      rows[u] = (uint32_t(a) << 8) | (ld_chunk ^ cu);  // (a list may hold any int: clamp)
      if (u == 0) first_key = __builtin_amdgcn_readfirstlane(a);
    }
  };
  // ---- pacing (see WaveClock): wait until the tile's first key is due ----
  int looks_left = clk.ticks_per_key > 0.f ? kWaveSpinLimit : 0, long_waits = 0;
  auto gate = [&]() {
    if (looks_left > 0) {
      const uint64_t due = clk.t0 + uint64_t(float(max(first_key - kWaveMarginKeys, 0)) * clk.ticks_per_key);
      uint64_t now = __builtin_amdgcn_s_memrealtime();
      const uint64_t give_up = now + kWaveGateTicks;
      while (now < due) {
        if (now >= give_up) {
          if (++long_waits >= kWaveLongWaits) looks_left = 0;
          break;
        }
        if (--looks_left <= 0) break;
        __builtin_amdgcn_s_sleep(8);
        now = __builtin_amdgcn_s_memrealtime();
      }
    }
  };
  // K and V of a tile into buffer `par`
  auto issue_tile = [&](int par) {
    const uint32_t dst = tiles_lds + uint32_t(2 * par) * kWTileBytes;
#pragma unroll
    for (int u = 0; u < 4; ++u) ring_load16(dst + uint32_t(u) * 1024u, rows[u], Kb);
#pragma unroll
    for (int u = 0; u < 4; ++u) ring_load16(dst + kWTileBytes + uint32_t(u) * 1024u, rows[u], Vb);
  };

  // ---- operand addresses: K row c, chunk 4 st + g; V key 4 g + c / 4 ----
  const int kbase = c * 256 + ((g ^ swz(c)) << 4);  // ^ (st << 6)
  const int vrl = 4 * g + (c >> 2);
  const int vbase = vrl * 256 + ((((c & 3) >> 1) ^ swz(vrl)) << 4) + (c & 1) * 8;  // ^ (t8 << 5)
  const lds_char_t* const tiles = lds + 512;

  auto run = [&](auto T_) {
    constexpr int T = decltype(T_)::value;
    if (ntiles > 0) {
      issue_ids(0);
      if (nblk > 1) issue_ids(1);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      read_rows(0);
      gate();
      issue_tile(0);
      // two tiles per trip of the loop, so that the buffers are compile-time constants
      for (int t0 = 0; t0 < ntiles; t0 += 2) {
#pragma unroll
        for (int par = 0; par < 2; ++par) {
          const int t = t0 + par;
          if (t >= ntiles) break;
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // tile t is in place, and every list entry asked for so far
          if (t + 1 < ntiles) {
            read_rows(t + 1);
            gate();
            // block b + 1 of the list entries takes the buffer of block b - 1, last read for tile 4 b - 1 (in iteration 4 b - 2)
            if (par == 0 && (t & 3) == 0 && t > 0 && (t >> 2) + 1 < nblk) issue_ids((t >> 2) + 1);
            issue_tile(1 - par);
          }
          const lds_char_t* const bK = tiles + 2 * par * kWTileBytes;
          const lds_char_t* const bV = bK + kWTileBytes;
          int kb = kbase, vb = vbase;
          asm volatile("" : "+v"(kb), "+v"(vb));
          // ---- S^T = K Q^T: keys 4 g + r of query c ----
          f32x4 s[T];
#pragma unroll
          for (int st = 0; st < 4; ++st) {
            const ring_u32x4 a_ = *reinterpret_cast<const __attribute__((address_space(3))) ring_u32x4*>(bK + (kb ^ (st << 6)));
            const uint4 a = make_uint4(a_[0], a_[1], a_[2], a_[3]);
#pragma unroll
            for (int qt = 0; qt < T; ++qt) s[qt] = Mma<F16>::m16(a, qf[qt][st], st == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[qt]);
          }
          wave_mfma_settle<T>(s);
          const int kp0 = t * 16;
          if (kp0 + 16 > cnt) {  // the bucket's last, ragged tile
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (kp0 + 4 * g + r >= cnt) {
#pragma unroll
                for (int qt = 0; qt < T; ++qt) s[qt][r] = -INFINITY;
              }
          }
          // ---- online softmax (triton_kernel.py:248-263) ----
          uint2 pf[T];
#pragma unroll
          for (int qt = 0; qt < T; ++qt) {
            float mx = st_max_lane_groups(st_max(st_max3(s[qt][0], s[qt][1], s[qt][2]), s[qt][3])) * scale2;
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
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(fmaf(s[qt][r], scale2, -m_sub));
            lsum[qt] += (p[0] + p[1]) + (p[2] + p[3]);
            pf[qt] = make_uint2(Mma<F16>::pack2(p[0], p[1]), Mma<F16>::pack2(p[2], p[3]));
          }
          // ---- O^T += V^T P^T ----
#pragma unroll
          for (int t8 = 0; t8 < 8; ++t8) {
            const ring_short4 a4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) ring_short4*)(bV + (vb ^ (t8 << 5))));
            const uint2 a = __builtin_bit_cast(uint2, a4);
#pragma unroll
            for (int qt = 0; qt < T; ++qt) O[qt][t8] = Mma<F16>::m16k16(a, pf[qt], O[qt][t8]);
          }
        }
      }
    }
    // ---- finish: lane (g,c) holds dims 16 t8 + 4g + r of query c of each tile ----
    {
      f32x4 last[T];
#pragma unroll
      for (int qt = 0; qt < T; ++qt) last[qt] = O[qt][7];
      wave_mfma_settle<T>(last);
#pragma unroll
      for (int qt = 0; qt < T; ++qt) O[qt][7] = last[qt];
    }
#pragma unroll
    for (int qt = 0; qt < T; ++qt) {
      float ltot = lsum[qt] + __shfl_xor(lsum[qt], 16);
      ltot += __shfl_xor(ltot, 32);
      const bool empty = (m[qt] == -INFINITY);
      const float inv = empty ? 0.f : 1.f / ltot;
      const int jq = 16 * qt + c;
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
  // A wave with more queries has more to do per tile and sets the pace of its launch: it goes first where it
  // shares a SIMD with a lighter one.
  if (n_qt >= 3)
    __builtin_amdgcn_s_setprio(3);
  else if (n_qt == 2)
    __builtin_amdgcn_s_setprio(1);
  if (n_qt <= 1)
    run(std::integral_constant<int, 1>{});
  else if (NQW >= 2 && n_qt == 2)
    run(std::integral_constant<int, (NQW >= 2 ? 2 : 1)>{});
  else if (NQW >= 3 && n_qt == 3)
    run(std::integral_constant<int, (NQW >= 3 ? 3 : 1)>{});
  else
    run(std::integral_constant<int, NQW>{});
  __builtin_amdgcn_s_setprio(0);
}

}  // namespace fm
