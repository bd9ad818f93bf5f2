// bf16 bucket-gathered attention forward on MFMA for head dimension 128 (gfx950)
// (triton_kernel.py:137-272), for grouped work items and for decode batches.
//
// Work decomposition.  One workgroup (4 waves) per work item = up to 64 queries
// that hashed to the same (row, bucket).  The bucket's key list is cut into
// blocks of 32 keys dealt round-robin to the four waves; every wave runs its own
// online softmax over its blocks for all the item's queries and the four partial
// (m, l, O) triples are merged through LDS at the end.  K and V rows of a bucket
// are therefore read from HBM once per item, whatever the number of queries.
//
// Data path.  No LDS in the main loop: gathered rows go from global memory
// straight into MFMA operand registers.
//   S^T = K.Q^T   v_mfma_f32_16x16x32_bf16, A = 16 gathered K rows (lane c of
//                 lane group g reads 16 bytes at column 32s+8g of row c), B =
//                 Q^T fragments kept in registers for the whole item.  Lane
//                 (g,c) ends up with scores of keys 4g..4g+3 for query c.
//   O^T += V^T.P^T  same instruction over a 32-key block: the accumulator
//                 layout of S^T is already the B-operand layout (keys along
//                 the contraction), so P needs no shuffle.  V rows are read
//                 fully coalesced (16 lanes x 16 B = one 256-byte row): lane
//                 (g,c) reads column chunk c of keys 4g..4g+3; transposing to
//                 the A-operand layout is a per-lane repack because output
//                 tile t takes column 8c+t of every chunk.  Lane (g,c) then
//                 holds O[query c][32g .. 32g+31].
// Softmax follows the reference kernel: base-2 with sm_scale*log2(e), fp32
// running max / denominator, denominator from unrounded p, p rounded to bf16
// before P.V (triton_kernel.py:248-263).
//
// Roofline: HBM.  Algorithmic bytes per item = cnt*(2*128*2 + 4) + n_q*(2*128*2
// + 4).  Per 32-key block a wave issues 16 KiB of loads and keeps one block in
// flight behind the one it is computing on.
#include "common.hpp"

namespace fm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kD = 128;
constexpr int kNQT = FM_QTILE / 16;  // query tiles of 16 per item
constexpr int kBlk = 32;             // keys per block (two MFMA key tiles)

struct KVRegs {
  uint4 k[2][4];  // [key tile][contraction step]
  uint4 v[2][4];  // [key tile][key 4g+j]
};

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 u) {
  union {
    uint4 u;
    bf16x8 b;
  } x;
  x.u = u;
  return x.b;
}

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  f32x2 x = {lo, hi};
  bf16x2 y = __builtin_convertvector(x, bf16x2);  // v_cvt_pk_bf16_f32, round to nearest even
  return *reinterpret_cast<uint32_t*>(&y);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Issues the loads of one 32-key block.  `rows` holds, in lanes 0..31 (and again
// in 32..63), the key row of block position lane%32 (already clamped to [0,N)).
__device__ __forceinline__ void load_block(KVRegs& r, const bf16_t* __restrict__ Kb,
                                           const bf16_t* __restrict__ Vb, int rows, int g, int c) {
#pragma unroll
  for (int kt = 0; kt < 2; ++kt) {
    const int rk = __shfl(rows, kt * 16 + c);
    const uint4* pk = reinterpret_cast<const uint4*>(Kb + int64_t(rk) * kD + 8 * g);
#pragma unroll
    for (int s = 0; s < 4; ++s) r.k[kt][s] = pk[4 * s];  // column 32s + 8g
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rv = __shfl(rows, kt * 16 + 4 * g + j);
      r.v[kt][j] = *reinterpret_cast<const uint4*>(Vb + int64_t(rv) * kD + 8 * c);
    }
  }
}

// NQ = number of 16-query tiles the instantiation carries (register footprint grows with it).
template <int NQ>
__device__ __forceinline__ void attend_item(
    const bf16_t* __restrict__ Qb,   // query rows of this item's row/head: [*, 128]
    const int* __restrict__ q_rows,  // LDS: row index (into Qb / out) of the item's queries
    int n_q, const bf16_t* __restrict__ Kb, const bf16_t* __restrict__ Vb,
    const int32_t* __restrict__ idx,  // bucket list; nullptr = keys 0..cnt-1
    int cnt, int N, float scale2, bf16_t* __restrict__ Ob, float* __restrict__ Lb, float* __restrict__ red) {
  const int l = lane_id(), w = threadIdx.x >> 6;
  const int g = l >> 4, c = l & 15;
  const int nqt = (n_q + 15) >> 4;

  // ---- Q^T fragments -------------------------------------------------------
  uint4 qf[NQ][4];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    const int j = qt * 16 + c;
    const bool ok = (qt < nqt) && (j < n_q);
    const uint4* pq = reinterpret_cast<const uint4*>(Qb + int64_t(ok ? q_rows[j] : 0) * kD + 8 * g);
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[qt][s] = ok ? pq[4 * s] : make_uint4(0, 0, 0, 0);
  }

  f32x4 O[NQ][8];
  float m[NQ], lsum[NQ];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    m[qt] = -INFINITY;
    lsum[qt] = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) O[qt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int nblk = (cnt + kBlk - 1) / kBlk;
  // (positions past the list read its last entry: the load is issued on every path, so the number of loads in
  // flight at any point of the loop below is known to the compiler, and so are the loads of the blocks)
  auto rows_of = [&](int b) -> int {
    const int kp = min(b * kBlk + (l & 31), cnt - 1);
    const int r = idx ? idx[max(kp, 0)] : kp;
    return min(max(r, 0), N - 1);
  };

  auto compute = [&](const KVRegs& kv, int b) {
    const int kp0 = b * kBlk;
    // V^T fragments for the 8 output tiles: element t of the 8 loads of this lane
    uint4 vf[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int dw = t >> 1;
      uint32_t a[8];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint4 x = kv.v[kt][j];
          a[kt * 4 + j] = dw == 0 ? x.x : dw == 1 ? x.y : dw == 2 ? x.z : x.w;
        }
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o[e] = (t & 1) ? ((a[2 * e] >> 16) | (a[2 * e + 1] & 0xffff0000u))
                       : ((a[2 * e] & 0xffffu) | (a[2 * e + 1] << 16));
      vf[t] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    const bool tail = kp0 + kBlk > cnt;
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
      if (qt < nqt) {
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kv.k[0][s]), as_bf16x8(qf[qt][s]), s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kv.k[1][s]), as_bf16x8(qf[qt][s]), s1, 0, 0, 0);
        }
        float x[8];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          x[r] = s0[r] * scale2;
          x[4 + r] = s1[r] * scale2;
        }
        if (tail) {
          const int lim = cnt;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if (kp0 + 4 * g + r >= lim) x[r] = -INFINITY;
            if (kp0 + 16 + 4 * g + r >= lim) x[4 + r] = -INFINITY;
          }
        }
        float mx = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])),
                         fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m[qt], mx);
        // a query that sees no key yet keeps m = -inf; subtract 0 instead of -inf
        const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
        // bucket lists are sorted by descending projection, so after the first blocks the
        // running maximum rarely moves: rescale only when it moved for some query of the tile
        if (__any(m_new != m[qt])) {
          const float alpha = fast_exp2(m[qt] - m_sub);
          lsum[qt] *= alpha;
#pragma unroll
          for (int t = 0; t < 8; ++t) {
            O[qt][t][0] *= alpha;
            O[qt][t][1] *= alpha;
            O[qt][t][2] *= alpha;
            O[qt][t][3] *= alpha;
          }
          m[qt] = m_new;
        }
        float p[8], ps = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          p[r] = fast_exp2(x[r] - m_sub);
          ps += p[r];
        }
        lsum[qt] += ps;
        const uint4 pf = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]),
                                    pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7]));
#pragma unroll
        for (int t = 0; t < 8; ++t)
          O[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf[t]), as_bf16x8(pf), O[qt][t], 0, 0, 0);
      }
    }
  };

  // ---- main loop: this wave's blocks w, w+4, ..., one block in flight -------
  KVRegs ra, rb;
  int b = w;
  // Key rows are fetched two blocks ahead of the block being computed, K/V one ahead.  The loads of the block
  // ahead go out whether or not there is one (past the end they fetch the list's last row again): with a load
  // that some path skips, the compiler's wait in front of a block's first MFMA has to be for every load in
  // flight, the block ahead included, and nothing is fetched ahead at all.
  if (cnt > 0) {  // (an empty list has no entry to read)
    load_block(ra, Kb, Vb, rows_of(b), g, c);
    int r1 = rows_of(b + 4);
    while (b < nblk) {
      const int b1 = b + 4, b2 = b + 8;
      const int r2 = rows_of(b2);
      load_block(rb, Kb, Vb, r1, g, c);
      compute(ra, b);
      if (b1 >= nblk) break;
      const int r3 = rows_of(b2 + 4);
      load_block(ra, Kb, Vb, r2, g, c);
      compute(rb, b1);
      r1 = r3;
      b = b2;
    }
  }

  // ---- merge the four waves ---------------------------------------------------
  // red layout (floats): O part [wave][qt][t][r][lane], then l [wave][qt][lane],
  // then m [wave][qt][16], with NQ query tiles: red_floats(NQ) floats
  float* redO = red;
  float* redL = red + 4 * NQ * 8 * 4 * 64;
  float* redM = redL + 4 * NQ * 64;
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    if (qt < nqt) {
#pragma unroll
      for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) redO[(((w * NQ + qt) * 8 + t) * 4 + r) * 64 + l] = O[qt][t][r];
      redL[(w * NQ + qt) * 64 + l] = lsum[qt];
      if (g == 0) redM[(w * NQ + qt) * 16 + c] = m[qt];
    }
  }
  __syncthreads();
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    if (qt < nqt) {
      float mw[4], mstar = -INFINITY;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) {
        mw[ww] = redM[(ww * NQ + qt) * 16 + c];
        mstar = fmaxf(mstar, mw[ww]);
      }
      const int j = qt * 16 + c;
      float f[4], lstar = 0.f;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) {
        f[ww] = (mw[ww] == -INFINITY) ? 0.f : fast_exp2(mw[ww] - mstar);
        float lw = 0.f;
#pragma unroll
        for (int gg = 0; gg < 4; ++gg) lw += redL[(ww * NQ + qt) * 64 + gg * 16 + c];
        lstar += f[ww] * lw;
      }
      const bool empty = (mstar == -INFINITY);  // the query saw no key at all
      const float inv = empty ? 0.f : 1.f / lstar;
      // wave w finalises accumulator row r = w: columns 32g + 8w + (0..7) of query c
      float o[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        float a = 0.f;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) a += f[ww] * redO[(((ww * NQ + qt) * 8 + t) * 4 + w) * 64 + l];
        o[t] = a * inv;
      }
      if (j < n_q) {
        const int64_t qr = q_rows[j];
        uint4 st = make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]),
                              pack_bf16(o[6], o[7]));
        *reinterpret_cast<uint4*>(Ob + qr * kD + 32 * g + 8 * w) = st;
        if (w == 0 && g == 0) Lb[qr] = empty ? -FLT_MAX : (mstar + __builtin_amdgcn_logf(lstar)) * kLn2;
      }
    }
  }
}

// floats of LDS the merge of the four waves needs for NQ query tiles
constexpr int red_floats(int nq) { return 4 * nq * 8 * 4 * 64 + 4 * nq * 64 + 4 * nq * 16; }
constexpr int kRedFloats = red_floats(kNQT);

__global__ __launch_bounds__(256) void hash_attn_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2) {
  extern __shared__ __attribute__((aligned(16))) float red[];
  __shared__ int q_rows[FM_QTILE];
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int cnt = bucket_cnt[bkt];
  if (threadIdx.x < it.n_q) q_rows[threadIdx.x] = q_perm[it.q_start + threadIdx.x];
  __syncthreads();
  const int64_t qbase = int64_t(it.row) * Sq;
  const bf16_t* Kb = k + int64_t(it.row) * N * kD;
  const bf16_t* Vb = v + int64_t(it.row) * N * kD;
  const int32_t* idx = k_idx + bucket_off[bkt];
  attend_item<kNQT>(q + qbase * kD, q_rows, it.n_q, Kb, Vb, idx, cnt, N, scale2, out + qbase * kD,
                     lse + qbase, red);
}

// Decode batch over memories of different sizes: G workgroups per row (one KV head
// of one sequence) with its G <= 16 queries.  Every workgroup of a row hashes the
// row's queries against the row's own A (first maximum wins; cheap, and it keeps the
// launch free of any host-side grouping); workgroup s then attends the s-th distinct
// bucket among the G hashes with the queries that chose it, or exits if there are
// fewer distinct buckets.  Each bucket is read once, and a row's buckets in parallel.  Rows are described by fm_rowdesc; A, K, V
// and the bucket lists of all rows are packed back to back.
// MODE 0: hash and attend in one launch; 1: hash only (one workgroup per row, writes hash_out); 2:
// attend only, on the hashes a MODE 1 launch left in hash_out.  Two launches take the hash off the
// path of the G workgroups of a row, which otherwise each repeat it before their first key load.
template <int MODE>
__global__ __launch_bounds__(256, 2) void decode_hash_attn_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ A_all, const bf16_t* __restrict__ K_all,
    const bf16_t* __restrict__ V_all, const int32_t* __restrict__ idx_all,
    const fm_rowdesc* __restrict__ desc, int G, float scale2, bf16_t* __restrict__ out,
    float* __restrict__ lse, int32_t* __restrict__ hash_out, float* __restrict__ scores_out) {
  extern __shared__ __attribute__((aligned(16))) float red[];
  __shared__ float s_best[4][16];
  __shared__ int s_besti[4][16];
  __shared__ int s_hash[16];
  __shared__ int q_rows[FM_QTILE];
  // the G workgroups of a row are neighbours in launch order: with descriptors given longest lists
  // first, the longest buckets of the whole batch start first
  const int row = MODE == 1 ? int(blockIdx.x) : int(blockIdx.x / unsigned(G));
  const int slot = MODE == 1 ? 0 : int(blockIdx.x % unsigned(G));
  const fm_rowdesc ds = desc[row];
  const int qrow = ds.q_row1 ? ds.q_row1 - 1 : row;  // where the row's queries and results live
  const int tid = threadIdx.x, l = tid & 63, w = tid >> 6;
  const bf16_t* qb = q + int64_t(qrow) * G * kD;
  if constexpr (MODE != 2) {
    // ---- hash on MFMA: 32 buckets x (G queries padded to 32) per v_mfma_f32_32x32x16_bf16 chain,
    //      buckets on the A operand and ascending contraction steps: the sums of the other hash
    //      kernels.  Wave w takes bucket chunks w, w+4, ...; lane (column l%32, half l/32) sees the
    //      scores of its query for 16 buckets of a chunk in ascending order.
    typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
    const int C = ds.n_buckets;
    const int col = l & 31, hb = l >> 5;
    bf16x8 bq[8];
    {
      const uint4* pq = reinterpret_cast<const uint4*>(qb + int64_t(col < G ? col : 0) * kD + hb * 8);
  #pragma unroll
      for (int ks = 0; ks < 8; ++ks) bq[ks] = as_bf16x8(col < G ? pq[2 * ks] : make_uint4(0, 0, 0, 0));
    }
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int c0 = 32 * w; c0 < C; c0 += 128) {
      const int cr = min(c0 + col, C - 1);
      const uint4* pa = reinterpret_cast<const uint4*>(A_all + (ds.a_off + cr) * kD + hb * 8);
      uint4 au[8];
  #pragma unroll
      for (int ks = 0; ks < 8; ++ks) au[ks] = pa[2 * ks];
      f32x16 acc;
  #pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  #pragma unroll
      for (int ks = 0; ks < 8; ++ks)
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(au[ks]), bq[ks], acc, 0, 0, 0);
  #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = c0 + 8 * (r >> 2) + 4 * hb + (r & 3);
        if (c < C && col < G) {
          if (scores_out && slot == 0) scores_out[(ds.a_off + c) * G + col] = acc[r];
          if (besti == 0x7fffffff || acc[r] > best) {  // buckets ascend per lane
            best = acc[r];
            besti = c;
          }
        }
      }
    }
    // the two lane halves of a column, then the four waves: larger score wins, equal scores keep the
    // lower bucket
    {
      const float ob = __shfl_xor(best, 32);
      const int oi = __shfl_xor(besti, 32);
      if (oi != 0x7fffffff && (besti == 0x7fffffff || ob > best || (ob == best && oi < besti))) {
        best = ob;
        besti = oi;
      }
      if (l < G) {
        s_best[w][l] = best;
        s_besti[w][l] = besti;
      }
    }
    __syncthreads();
    if (tid < G) {
      float b = s_best[0][tid];
      int bi = s_besti[0][tid];
      for (int ww = 1; ww < 4; ++ww) {
        const float ob = s_best[ww][tid];
        const int oi = s_besti[ww][tid];
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ob > b || (ob == b && oi < bi))) {
          b = ob;
          bi = oi;
        }
      }
      s_hash[tid] = bi;
      if (slot == 0) hash_out[int64_t(qrow) * G + tid] = bi;
    }
    __syncthreads();
  } else {
    if (tid < G) s_hash[tid] = hash_out[int64_t(qrow) * G + tid];
    __syncthreads();
  }
  if constexpr (MODE == 1) return;
  // ---- this workgroup's bucket: the slot-th distinct one among the G hashes ----
  const bf16_t* Kb = K_all + ds.k_off * kD;
  const bf16_t* Vb = V_all + ds.k_off * kD;
  int seen = 0, bkt = -1;
  for (int g0 = 0; g0 < G; ++g0) {  // uniform: every thread reads the same s_hash
    bool first = true;
    for (int g = 0; g < g0; ++g) first = first && (s_hash[g] != s_hash[g0]);
    if (!first) continue;
    if (seen == slot) bkt = s_hash[g0];
    ++seen;
  }
  if (bkt < 0) return;
  if (tid == 0) {
    int n = 0;
    for (int g = 0; g < G; ++g)
      if (s_hash[g] == bkt) q_rows[n++] = g;
    q_rows[FM_QTILE - 1] = n;
  }
  __syncthreads();
  const int n_q = q_rows[FM_QTILE - 1];
  attend_item<1>(qb, q_rows, n_q, Kb, Vb, idx_all + ds.idx_off + int64_t(bkt) * ds.bucket_size, ds.bucket_size,
                 ds.n_keys, scale2, out + int64_t(qrow) * G * kD, lse + int64_t(qrow) * G, red);
}

// Dense attention of one token per query head over L local keys (decode): one workgroup per KV
// head with its G <= 16 query heads; the four waves take the 32-key blocks in turn, as for a
// gathered bucket, so four blocks of loads are in flight per workgroup.  With one query per head a
// causal mask aligned bottom-right hides nothing.
__global__ __launch_bounds__(256) void local_attn_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    bf16_t* __restrict__ out, float* __restrict__ lse, int G, int L, float scale2) {
  extern __shared__ __attribute__((aligned(16))) float red[];
  __shared__ int q_rows[FM_QTILE];
  const int hk = blockIdx.x;
  if (threadIdx.x < FM_QTILE) q_rows[threadIdx.x] = threadIdx.x;
  __syncthreads();
  const int64_t qbase = int64_t(hk) * G;
  attend_item<1>(q + qbase * kD, q_rows, G, k + int64_t(hk) * L * kD, v + int64_t(hk) * L * kD, nullptr, L, L,
                 scale2, out + qbase * kD, lse + qbase, red);
}

int local_attn_decode(const void* q, const void* k, const void* v, void* out, float* lse, int H, int G, int L,
                      float sm_scale, hipStream_t st) {
  hipLaunchKernelGGL(local_attn_decode_kernel, dim3(unsigned(H)), dim3(256), red_floats(1) * sizeof(float), st,
                     (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (bf16_t*)out, lse, G, L,
                     sm_scale * kLog2e);
  return launch_status("fm_local_attn_fwd(decode)");
}

bool hash_attn_mfma_d_supported(int d, int N);  // attn_mfma_d.hip
int hash_attn_mfma_d(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                     const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                     int64_t max_items, void* out, float* lse, int Sq, int N, int d, int C, float sm_scale, bool f16,
                     hipStream_t st);

bool hash_attn_mfma_supported(int d, int dtype, int N) {
  return (d == kD || hash_attn_mfma_d_supported(d, N)) && (dtype == FM_BF16 || dtype == FM_F16);
}

int decode_hash_attn(const void* q, const void* A_all, const void* K_all, const void* V_all,
                     const int32_t* idx_all, const fm_rowdesc* desc, int rows, int G, float sm_scale,
                     void* out, float* lse, int32_t* hash_out, float* scores_out, hipStream_t st) {
  // the hash of every row first (one short workgroup each), then G workgroups per row that start on
  // their bucket at once
  hipLaunchKernelGGL(decode_hash_attn_kernel<1>, dim3(unsigned(rows)), dim3(256), 0, st, (const bf16_t*)q,
                     (const bf16_t*)A_all, (const bf16_t*)K_all, (const bf16_t*)V_all, idx_all, desc, G,
                     sm_scale * kLog2e, (bf16_t*)out, lse, hash_out, scores_out);
  hipLaunchKernelGGL(decode_hash_attn_kernel<2>, dim3(unsigned(rows) * unsigned(G)), dim3(256),
                     red_floats(1) * sizeof(float), st, (const bf16_t*)q, (const bf16_t*)A_all, (const bf16_t*)K_all,
                     (const bf16_t*)V_all, idx_all, desc, G, sm_scale * kLog2e, (bf16_t*)out, lse, hash_out,
                     scores_out);
  return launch_status("fm_decode_hash_attn");
}
bool local_attn_dense_supported(int d, int dtype);  // attn_local.hip
bool local_attn_mfma_supported(int d, int dtype) { return local_attn_dense_supported(d, dtype); }

int hash_attn_mfma_staged(const void* q, const void* k, const void* v, const int32_t* k_idx,
                          const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                          const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                          float* lse, int H, int Sq, int N, int C, float sm_scale, bool pairs, bool f16, bool per_row,
                          hipStream_t st);
int hash_attn_mfma_wave(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                        const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items,
                        const int32_t* n_items, int64_t max_items, void* out, float* lse, int Sq, int N, int C,
                        float sm_scale, bool f16, int H, bool per_row, hipStream_t st);
int hash_attn_mfma_ring(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                        const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items,
                        const int32_t* n_items, int64_t max_items, void* out, float* lse, int Sq, int N, int C,
                        float sm_scale, bool f16, int H, bool per_row, void* ws, size_t ws_bytes, hipStream_t st);
extern std::atomic<int> g_force_generic;

// Which grouped forward kernel a launch takes: 0 = rows gathered into registers (this file), 1 = rows
// staged in LDS through registers, one work item per workgroup, 2 = the same, two items per workgroup,
// 3 = rows loaded straight into LDS, three items per workgroup (attn_ring.hpp), 4 = the same loads, a wave
// per work item (attn_wave.hpp; its rule stands further down).  Measured rule: a kernel
// that shares a bucket's rows through LDS is at least as fast as the register-gather one wherever the launch
// has work items enough to fill the chip (at least 512, taking min(Sq, C) per row as their number) or buckets
// receive 24 queries or more on average; with few and small items the four waves of the gather kernel, which
// share one bucket's keys, finish an item sooner.  Of the LDS kernels form 3 wherever its 32-bit row offsets
// reach (2^24 keys), form 1 in its form with 64-bit row offsets beyond.  Form 3 against form 1: on keys
// that stay in the last-level cache (65536 keys, 1024 buckets of 3072, 16 / 32 / 64 / 128 queries per bucket)
// 1.51 / 1.57 / 1.69 / 2.51 ms against 1.54 / 1.67 / 2.30 / 3.05 ms; on large memories with few queries per
// bucket the two are level while the lists are in score order (a million keys, 16 queries per bucket: 17.9
// against 17.8 ms) and form 3 is ahead once they are in key order (figures below).  Forms 1 and 2 stay for
// the long memories and for tests to compare against.
//
// A launch per row, in row order, when K and V of all rows together are at least twice the last-level cache
// (512 MB), a row's are 32 MB or more, and a row fills the device twice over (the direct-load kernel runs 512 workgroups at a time, the
// staged one 768): with the lists in ascending key order the workgroups of a launch sweep the row's K and V
// at about the same pace, and a key row that several buckets list is fetched from HBM once and found in the
// last-level cache, or the L2, by the others; in a single launch over all rows the starts spread over the
// whole sweep after a few rounds of workgroups and two rows' sweeps overlap at every row boundary.  Measured
// (lists in key order; staged / direct loads in one launch, then per row): 8 rows of 2^20 keys, 2048 buckets
// of 16384, 16 queries per bucket 15.9 / 14.6 / 14.0 / 12.3 ms; 8 rows of 2^18 keys, 1024 buckets of 4096, 8
// queries per bucket 1.76 / 1.42 / 1.86 / 1.22 ms; 8 rows of 2^15 keys (134 MB in all), 256 buckets of 1024
// 0.134 / 0.112 / 0.241 / 0.191 ms.
// (Rows of 16 MB, 64 of them with 1024 buckets of 1024: 3.73 ms per row against 3.34 in one launch -- a launch of
// 60 us is mostly start and tail; rows of 32 MB, 32 of them with 1024 buckets of 3072: 4.58 against 5.23.)
static bool row_launches_pay(int choice, int H, int Sq, int N, int C) {
  return H > 1 && int64_t(H) * N * kD * 4 >= (int64_t(512) << 20) && int64_t(N) * kD * 4 >= (int64_t(32) << 20) &&
         (C < Sq ? C : Sq) >= (choice >= 3 ? 1024 : 1536);
}

// Form 4 (attn_wave.hpp: a wave per work item, eight buckets swept per compute unit instead of two, the sweeps
// of a launch paced against the device's clock) where the launches go per row, a row has 2048 buckets and
// queries or more (one item per wave: fewer do not fill the device) and a bucket receives 24 queries or fewer
// on average: there a launch is bound by the requests that miss the L2s, and waves that sweep the key range
// together find most of their rows in the L2.  Its tile is 16 keys and a wave's MFMA and softmax work grows
// with the queries of its item, so it loses from two tiles of queries per item on.  Measured against form 3,
// both per row, lists in key order, per step (ms), form 4 unpaced and paced (after its schedules have settled):
//   8 rows of 2^20 keys, 2048 buckets of 16384, the queries of the 1 M-key benchmark workload (16 per bucket on
//     average, as its hash deals them): 12.2 against 10.6 and 8.0
//   the same memory, queries assigned to buckets at random; 4 / 8 / 16 / 24 / 32 per bucket on average:
//     13.1 / 12.8 / 13.3 / 13.5 / 13.5 against 11.2 / 11.3 / 12.6 / 13.3 / 18.9 and 7.4 / 7.3 / 8.1 / 9.6 / 18.9
//   4 rows of 2^21 keys, 2048 buckets of 32768; 4 / 8 / 16 / 24 / 32: 14.0 / 14.0 / 14.4 / 14.4 / 14.5 against
//     13.1 / 13.1 / 14.0 / 14.5 / 18.9 and 7.3 / 7.4 / 8.0 / 9.4 / 18.0
//   8 rows of 2^20 keys, 4096 buckets of 4096; 4 / 8 / 16 / 24 / 32: 8.5 / 8.7 / 8.7 / 8.8 / 8.8 against
//     7.1 / 7.2 / 7.4 / 7.6 / 9.0 and the same paced (launches too short for a schedule to pay)
//   8 rows of 2^18 keys, 1024 buckets of 4096 (1024 items a row: four waves per compute unit), the queries of
//     the 256 K-key benchmark workload (8 per bucket on average): 1.22 against 1.46 (paced the same)
//   16 rows of 2^19 keys, 1024 buckets of 8192; 4 / 8 / 16: 5.84 / 5.83 / 5.89 against 5.12 / 5.56 / 6.20
static bool wave_per_item_pays(int H, int Sq, int N, int C) {
  return row_launches_pay(4, H, Sq, N, C) && (C < Sq ? C : Sq) >= 2048 && int64_t(Sq) <= int64_t(24) * C;
}

int hash_attn_mfma_choice(int H, int Sq, int N, int C) {
  const int force = g_force_generic;
  if (force == 3) return 0;
  if (force == 2 || force == 6) return 1;
  if (force == 4) return N <= (1 << 24) ? 2 : 1;
  if (force == 5 || force == 7) return N <= (1 << 24) ? 3 : 1;
  if (force >= 10 && force <= 13) return N <= (1 << 24) ? 4 : 1;
  const bool many_items = int64_t(H) * (Sq < C ? Sq : C) >= 512;
  const bool dense = Sq >= 24 * int64_t(C);
  if (!many_items && !dense) return 0;
  if (N > (1 << 24)) return 1;
  return wave_per_item_pays(H, Sq, N, C) ? 4 : 3;
}

// One launch per row (forms 1, 3 and 4 only).
bool hash_attn_mfma_per_row(int choice, int H, int Sq, int N, int C) {
  const int force = g_force_generic;
  if ((choice != 1 && choice != 3 && choice != 4) || force == 2 || force == 5 || force == 11) return false;
  if (force == 6 || force == 7 || force == 12 || force == 13) return true;
  return row_launches_pay(choice, H, Sq, N, C);
}

int hash_attn_mfma(const void* q, const void* k, const void* v, const int32_t* k_idx,
                   const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                   const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                   float* lse, int H, int Sq, int N, int d, int C, float sm_scale, int dtype, void* ws, size_t ws_bytes,
                   hipStream_t st) {
  // head dimensions 64 and 256, and 128 when a test asks for the kernel that takes every head dimension
  if (d != kD || (g_force_generic == 8 && int64_t(N) * 2 * d < (int64_t(1) << 32)))
    return hash_attn_mfma_d(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items, out, lse, Sq,
                            N, d, C, sm_scale, dtype == FM_F16, st);
  int choice = hash_attn_mfma_choice(H, Sq, N, C);
  if (dtype == FM_F16 && choice == 0) choice = 1;
  const bool per_row = hash_attn_mfma_per_row(choice, H, Sq, N, C);
  if (choice == 4)
    return hash_attn_mfma_wave(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items, out, lse, Sq,
                               N, C, sm_scale, dtype == FM_F16, H, per_row, st);
  if (choice == 3)
    return hash_attn_mfma_ring(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items, out, lse, Sq,
                               N, C, sm_scale, dtype == FM_F16, H, per_row, ws, ws_bytes, st);
  if (choice) {
    return hash_attn_mfma_staged(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items, out,
                                 lse, H, Sq, N, C, sm_scale, choice == 2, dtype == FM_F16, per_row, st);
  }
  FM_ALLOW_LDS(hash_attn_mfma_kernel, kRedFloats * sizeof(float), "fm_hash_attn_fwd: lds");
  hipLaunchKernelGGL(hash_attn_mfma_kernel, dim3(unsigned(max_items)), dim3(256),
                     kRedFloats * sizeof(float), st, (const bf16_t*)q, (const bf16_t*)k,
                     (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items,
                     (bf16_t*)out, lse, Sq, N, C, sm_scale * kLog2e);
  return launch_status("fm_hash_attn_fwd(mfma)");
}

int local_attn_dense(const void* q, const void* k, const void* v, void* out, float* lse, int H, int G, int S,
                     int L, int d, bool f16, float sm_scale, int causal, hipStream_t st);

int local_attn_mfma(const void* q, const void* k, const void* v, void* out, float* lse, int H, int G,
                    int S, int L, int d, int dtype, float sm_scale, int causal, hipStream_t st) {
  if (S == 1 && G <= 16 && L >= 1 && d == kD && dtype == FM_BF16)
    return local_attn_decode(q, k, v, out, lse, H, G, L, sm_scale, st);
  return local_attn_dense(q, k, v, out, lse, H, G, S, L, d, dtype == FM_F16, sm_scale, causal, st);
}

}  // namespace fm
