// Dense local attention for bf16 / fp16, head dimensions 64, 128 and 256 (gfx950): the attention over
// the most recent keys that the memory's output is merged with (call site
// memory.py:302; the reference leaves `attention_forward` undefined, the contract
// here is softmax(q.k^T * scale) v with a causal mask aligned bottom-right, output
// plus natural-log LSE).
//
// One workgroup (4 waves) per 128 consecutive queries of one query head, 32 queries
// per wave.  K and V tiles of 64 keys go global -> registers -> LDS, double buffered;
// V is transposed on the way ( Vt[d][key] ) because both MFMA operands want the
// contraction index contiguous per lane.
//   S^T = K.Q^T    v_mfma_f32_32x32x16_{bf16,f16}, A = K rows from LDS, B = Q^T fragments
//                  resident in registers.  Lane (query l%32, half l/32) ends up with
//                  the scores of keys 8*(r/4) + 4*(l/32) + r%4 of each 32-key block:
//                  one query per lane column, so the softmax statistics are per-lane
//                  registers and need one cross-half shuffle per tile.
//   O^T += Vt.P^T  same instruction; registers 8s..8s+7 of a score block are exactly
//                  the B operand of contraction step s if the 16 keys of the step are
//                  taken in the order [0..3, 8..11 | 4..7, 12..15]; Vt is stored in LDS
//                  with its key columns in that order, so neither P nor V is shuffled.
// Softmax as in the gather kernel (triton_kernel.py:248-263): base 2 with
// sm_scale*log2(e), fp32 running max and denominator, denominator from unrounded p,
// p rounded to the input type before P.V; the running maximum is followed lazily (see kLazy: p stays below
// 2^8, far inside fp16).  Head dimension 256 runs one workgroup per CU (141 KB of LDS, 128 output registers).
//
// Roofline: MFMA (4*d flops per visible query-key pair); the per-element softmax
// VALU work is of the same order as the MFMA time and does not overlap with it.
#include "common.hpp"
#include "mma16.hpp"

namespace fm {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

constexpr int kLQ = 128;    // queries per workgroup
constexpr int kLK = 64;     // keys per tile
constexpr int kLVld = 72;   // Vt row stride in LDS (elements): 64 keys + 8
constexpr float kLazy = 8.f;  // growth of a running maximum (in powers of two) that is left unfollowed

// F16: the 16-bit type is fp16 (else bf16); D: head dimension.  A row has CP = D / 8 16-byte chunks.  K: thread
// tid takes chunk tid % CP of rows tid / CP + (256 / CP) u.  V: a unit is (chunk c, four consecutive keys 4j..4j+3),
// 16 CP of them in a tile; unit u has c = u % 4 + 4 (u / 64), j = (u / 4) % 16 (four neighbouring lanes read 64
// contiguous bytes), thread tid takes units tid + 256 i.
template <bool F16, int D>
__global__ __launch_bounds__(256, D == 256 ? 1 : 2) void local_attn_dense_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    bf16_t* __restrict__ out, float* __restrict__ lse, int G, int S, int L, float scale2, int causal) {
  constexpr int kLD = D;
  constexpr int kLKld = D + 8;            // K tile row stride in LDS (elements)
  constexpr int CP = D / 8;               // 16-byte chunks of a row
  constexpr int KU = kLK * CP / 256;      // K chunks per thread
  constexpr int KR = 256 / CP;            // rows between a thread's K chunks
  constexpr int VUNITS = 16 * CP;         // (chunk, four keys) units of a V tile
  constexpr int VU = (VUNITS + 255) / 256;
  constexpr int NKS = D / 16, NDT = D / 32;
  using M = Mma<F16>;
  __shared__ __attribute__((aligned(16))) bf16_t sK[2][kLK * kLKld];
  __shared__ __attribute__((aligned(16))) bf16_t sVt[2][kLD * kLVld];
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int col = l & 31, hb = l >> 5;
  // Late query blocks see most keys: the launch hands out the last block of every head first, then the block
  // before it of every head, ..., so that what starts last is the shortest work and the launch ends evenly
  // (with the blocks of a head in a row, the longest workgroup of the last head would start near the end).
  const int hq = blockIdx.x, hk = hq / G;
  const int qb = int(gridDim.y) - 1 - int(blockIdx.y);
  const int i0 = qb * kLQ;
  const bf16_t* Kh = k + int64_t(hk) * L * kLD;
  const bf16_t* Vh = v + int64_t(hk) * L * kLD;
  const int64_t qrow0 = int64_t(hq) * S;

  // visible keys: query i sees keys [0, lim(i))
  auto lim_of = [&](int i) { return causal ? min(L, max(0, i + (L - S) + 1)) : L; };
  const int i_last = min(S, i0 + kLQ) - 1;
  const int wg_lim = lim_of(i_last);
  const int ntiles = (wg_lim + kLK - 1) / kLK;

  const int iq = i0 + w * 32 + col;  // this lane's query
  const bool q_ok = iq < S;
  const int my_lim = q_ok ? lim_of(iq) : 0;
  // (the same in every lane of a wave: read through one lane, so that the tests on them are scalar branches
  // and not per-lane selects that every tile would pay for)
  const int wq0 = i0 + __builtin_amdgcn_readfirstlane(w) * 32;
  const int wave_lim_hi = lim_of(min(S - 1, wq0 + 31));  // most keys any query of the wave sees
  const int wave_lim_lo = (wq0 + 31 < S) ? lim_of(wq0) : 0;  // fewest

  uint4 qf[NKS];
  {
    const uint4* pq = reinterpret_cast<const uint4*>(q + (qrow0 + (q_ok ? iq : 0)) * kLD + hb * 8);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qf[ks] = q_ok ? pq[2 * ks] : make_uint4(0, 0, 0, 0);
  }
  // The compiler's wait-count pass cannot see that these loads have landed by the time the loop starts (the path
  // that skips the first tile has no wait) and would otherwise wait, in front of every tile's first MFMA, for
  // all loads in flight: the next tile's, whose latency the double buffering is there to hide.  The empty
  // statements read the registers (the pass waits for the loads here, once) and count as their last writers.
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
    asm volatile("" : "+v"(qf[ks].x), "+v"(qf[ks].y), "+v"(qf[ks].z), "+v"(qf[ks].w));
  f32x16 O[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) O[dt][r] = 0.f;
  float m = -INFINITY, lsum = 0.f;

  uint4 trk[KU];      // K rows tid / CP + KR u, chunk tid % CP
  uint4 trv[VU][4];   // V unit tid + 256 i: rows 4j..4j+3, chunk c
  const int krow = tid / CP, kch = tid % CP;
  auto unit_c = [&](int i) { const int u = tid + 256 * i; return (u & 3) + 4 * (u >> 6); };
  auto unit_j = [&](int i) { return ((tid + 256 * i) >> 2) & 15; };
  auto unit_ok = [&](int i) { return VUNITS % 256 == 0 || tid + 256 * i < VUNITS; };
  const uint4* pk0 = reinterpret_cast<const uint4*>(Kh + int64_t(krow) * kLD) + kch;
  const uint4* pv0[VU];
#pragma unroll
  for (int i = 0; i < VU; ++i) pv0[i] = reinterpret_cast<const uint4*>(Vh + int64_t(4 * unit_j(i)) * kLD) + unit_c(i);
  auto load_tile = [&](int t) {
    const int kp0 = t * kLK;
    if (kp0 + kLK <= L) {  // a whole tile: no row of it lies past the keys
      const uint4* pk = pk0 + int64_t(kp0) * CP;
#pragma unroll
      for (int u = 0; u < KU; ++u) trk[u] = pk[KR * u * CP];
#pragma unroll
      for (int i = 0; i < VU; ++i) {
        if (!unit_ok(i)) continue;
        const uint4* pv = pv0[i] + int64_t(kp0) * CP;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) trv[i][kk] = pv[kk * CP];
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int row = kp0 + krow + KR * u;
      trk[u] = row < L ? reinterpret_cast<const uint4*>(Kh + int64_t(row) * kLD)[kch] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < VU; ++i) {
      if (!unit_ok(i)) continue;
      const int c = unit_c(i), j = unit_j(i);
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const int row = kp0 + 4 * j + kk;
        trv[i][kk] = row < L ? reinterpret_cast<const uint4*>(Vh + int64_t(row) * kLD)[c] : make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto stash_tile = [&](int buf) {
#pragma unroll
    for (int u = 0; u < KU; ++u)
      *reinterpret_cast<uint4*>(&sK[buf][(krow + KR * u) * kLKld + kch * 8]) = trk[u];
    // keys 4j..4j+3 of the tile keep their order; the groups of four inside each 16 are
    // stored in the order 0, 2, 1, 3
#pragma unroll
    for (int i = 0; i < VU; ++i) {
      if (!unit_ok(i)) continue;
      const int vc = unit_c(i), vj = unit_j(i);
      const int a = vj >> 2, g4 = vj & 3;
      const int pos0 = 16 * a + 4 * ((g4 & 1) * 2 + (g4 >> 1));
      const uint32_t w0[4] = {trv[i][0].x, trv[i][0].y, trv[i][0].z, trv[i][0].w};
      const uint32_t w1[4] = {trv[i][1].x, trv[i][1].y, trv[i][1].z, trv[i][1].w};
      const uint32_t w2[4] = {trv[i][2].x, trv[i][2].y, trv[i][2].z, trv[i][2].w};
      const uint32_t w3[4] = {trv[i][3].x, trv[i][3].y, trv[i][3].z, trv[i][3].w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int wi = e >> 1;
        uint2 o;
        if (e & 1) {
          o.x = (w0[wi] >> 16) | (w1[wi] & 0xffff0000u);
          o.y = (w2[wi] >> 16) | (w3[wi] & 0xffff0000u);
        } else {
          o.x = (w0[wi] & 0xffffu) | (w1[wi] << 16);
          o.y = (w2[wi] & 0xffffu) | (w3[wi] << 16);
        }
        *reinterpret_cast<uint2*>(&sVt[buf][(8 * vc + e) * kLVld + pos0]) = o;
      }
    }
  };

  auto compute_tile = [&](int t, int buf) {
    const int kp0 = t * kLK;
    if (kp0 >= wave_lim_hi) return;  // no query of this wave sees the tile
    // ---- S^T for the two 32-key blocks ----
    f32x16 s[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[sb][r] = 0.f;
    {
      const bf16_t* pa = &sK[buf][col * kLKld + hb * 8];
      // the two 32-key blocks in turn: neighbouring MFMAs do not wait for each other's sums
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
          s[sb] = M::m32(*reinterpret_cast<const uint4*>(pa + sb * 32 * kLKld + ks * 16), qf[ks], s[sb]);
    }
    // ---- mask (only tiles that reach past what some query of the wave sees; the empty statement keeps the
    // compiler from turning the branch into per-lane selects that every tile would execute) ----
    if (kp0 + kLK > wave_lim_lo) {
      asm volatile("");
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kp0 + sb * 32 + 8 * (r >> 2) + 4 * hb + (r & 3);
          if (key >= my_lim) s[sb][r] = -INFINITY;
        }
    }
    // ---- online softmax, one query per lane column ----
    float mx = s[0][0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[0][r]);
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[1][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32)) * scale2;  // scale2 > 0: scaling commutes with the maximum
    // The running maximum follows the scores only when some query's grew by more than 2^kLazy (or it sees
    // its first key): until then the weights are taken against the older maximum and stay below 2^kLazy,
    // which fp32 sums and the relative rounding of bf16 do not notice, and the 64 multiplications of the
    // accumulator are spared in most tiles.  The sums, the output and the LSE are the same function of the
    // scores either way.
    const float m_new = fmaxf(m, mx);
    if (__any(m_new > m + kLazy)) {
      const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m - m_to);
      lsum *= alpha;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) O[dt][r] *= alpha;
      m = m_new;
    }
    const float m_sub = (m == -INFINITY) ? 0.f : m;  // a query that sees no key yet
    uint4 pf[2][2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[r] = __builtin_amdgcn_exp2f(fmaf(s[sb][r], scale2, -m_sub));
        lsum += p[r];
      }
#pragma unroll
      for (int st = 0; st < 2; ++st)
        pf[sb][st] = make_uint4(M::pack2(p[8 * st + 0], p[8 * st + 1]), M::pack2(p[8 * st + 2], p[8 * st + 3]),
                                M::pack2(p[8 * st + 4], p[8 * st + 5]), M::pack2(p[8 * st + 6], p[8 * st + 7]));
    }
    // ---- O^T += Vt.P^T (the four 32-row blocks of the output in turn, for the same reason) ----
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
          const bf16_t* pv = &sVt[buf][(dt * 32 + col) * kLVld + hb * 8];
          O[dt] = M::m32(*reinterpret_cast<const uint4*>(pv + sb * 32 + st * 16), pf[sb][st], O[dt]);
        }
  };

  if (ntiles > 0) {
    load_tile(0);
    stash_tile(0);
  }
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    if (t + 1 < ntiles) load_tile(t + 1);
    compute_tile(t, t & 1);
    if (t + 1 < ntiles) stash_tile((t + 1) & 1);  // last read one tile ago, behind the barrier below
    __syncthreads();
  }

  // ---- finish: lane (query, half) holds d = 32*dt + 8*(r/4) + 4*half + r%4 ----
  const float ltot = lsum + __shfl_xor(lsum, 32);
  const bool empty = (m == -INFINITY);
  const float inv = empty ? 0.f : 1.f / ltot;
  if (q_ok) {
    bf16_t* po = out + (qrow0 + iq) * kLD;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        uint2 o;
        o.x = M::pack2(O[dt][4 * rq + 0] * inv, O[dt][4 * rq + 1] * inv);
        o.y = M::pack2(O[dt][4 * rq + 2] * inv, O[dt][4 * rq + 3] * inv);
        *reinterpret_cast<uint2*>(po + dt * 32 + 8 * rq + 4 * hb) = o;
      }
    if (hb == 0) lse[qrow0 + iq] = empty ? -FLT_MAX : (m + __builtin_amdgcn_logf(ltot)) * kLn2;
  }
}

template <bool F16, int D>
static void launch_local_dense(const void* q, const void* k, const void* v, void* out, float* lse, int H, int G, int S,
                               int L, float sm_scale, int causal, hipStream_t st) {
  dim3 grid = dim3(unsigned(H * G), unsigned(ceil_div(S, kLQ)));
  hipLaunchKernelGGL((local_attn_dense_kernel<F16, D>), grid, dim3(256), 0, st, (const bf16_t*)q, (const bf16_t*)k,
                     (const bf16_t*)v, (bf16_t*)out, lse, G, S, L, sm_scale * kLog2e, causal);
}

bool local_attn_dense_supported(int d, int dtype) {
  return (d == 64 || d == 128 || d == 256) && (dtype == FM_BF16 || dtype == FM_F16);
}

int local_attn_dense(const void* q, const void* k, const void* v, void* out, float* lse, int H, int G, int S,
                     int L, int d, bool f16, float sm_scale, int causal, hipStream_t st) {
#define FM_LOCAL_DENSE(F, DD) launch_local_dense<F, DD>(q, k, v, out, lse, H, G, S, L, sm_scale, causal, st)
  if (d == 64)
    f16 ? FM_LOCAL_DENSE(true, 64) : FM_LOCAL_DENSE(false, 64);
  else if (d == 128)
    f16 ? FM_LOCAL_DENSE(true, 128) : FM_LOCAL_DENSE(false, 128);
  else
    f16 ? FM_LOCAL_DENSE(true, 256) : FM_LOCAL_DENSE(false, 256);
#undef FM_LOCAL_DENSE
  return launch_status("fm_local_attn_fwd(dense)");
}

}  // namespace fm
