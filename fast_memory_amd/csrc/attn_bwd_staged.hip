// Backward of the bucket-gathered attention without atomics, for dense query
// sets (bf16, head dimension 128).
//
// A key belongs to many buckets (C Z / N of them on average), so its dK and dV
// rows collect contributions from many workgroups.  Memory-side fp32 atomics
// sustain a fraction of the HBM rate; here the contributions are staged:
//   1. hash_attn_bwd_staged_kernel (attn_bwd_mfma.hip): one workgroup per
//      (row, bucket) writes the bucket's own dK, dV partial rows, one bf16 row of
//      128 per listed key each, side by side at the key's flat list position --
//      plain coalesced stores, 512 B per (bucket, key) pair; dQ is complete after this step;
//   2. bwd_reduce_kernel: one wave per key sums the key's partial rows over the
//      list positions that name it, in ascending position order, and adds the
//      fp32 sums into dK, dV.
// Step 2 needs the inverse of the bucket lists: for every key the flat list
// positions holding it.  That index depends on the lists only (not on queries or
// gradients); fm_inverse_index builds it with a stable radix sort of
// (row * N + key, position) pairs and a binary search per key for the offsets.
// The partial rows of a pass must fit the caller's workspace: rows (KV heads) are
// processed in groups whose lists fit.
//
// Traffic per (bucket, key) pair: the forward's gather (2 x 256 B) + 512 B written
// + 512 B read, all as full lines, against 2 x 512 B of fp32 atomic read-modify-
// write per (16-query tile, key) pair on the atomic path.  A bucket nobody hashed
// to gets zero rows (its workgroup writes them), so step 2 reads every listed
// position without asking.  The summation order is fixed, so dK and dV do not
// depend on scheduling.
#include <cstring>

#include "common.hpp"
#include "radix_sort.hpp"

namespace fm {

int launch_unlisted_rows(const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                         const int32_t* bin_off, const int32_t* bin_count, int64_t n_bins, int64_t nq,
                         int row_bytes, void* rows, float* lse, hipStream_t st);  // group.hip
int launch_fill(int32_t* p, int64_t n, int32_t v, hipStream_t st);  // group.hip
int hash_attn_bwd_staged_partials(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                  const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                                  const int32_t* bin_off, const int32_t* bin_count, const void* out, const float* lse,
                                  const void* dout, const float* dlse, void* dq, void* dkp, void* dvp, void* dump, int64_t pos0,
                                  int row0, int rows, int Sq, int N, int C, float sm_scale, float* dk, float* dv,
                                  bool f16, hipStream_t st);  // attn_bwd_mfma.hip

// ---- inverse index ------------------------------------------------------------
// One workgroup per (row, bucket): sort keys row * N + key, values = flat positions.
__global__ __launch_bounds__(256) void inv_pairs_kernel(const int32_t* __restrict__ k_idx,
                                                        const int64_t* __restrict__ bucket_off,
                                                        const int32_t* __restrict__ bucket_cnt, int C, int N,
                                                        uint32_t* __restrict__ keys, uint32_t* __restrict__ vals) {
  const int64_t b = blockIdx.x;
  const int row = int(b / C);
  const int64_t off = bucket_off[b];
  const int cnt = bucket_cnt[b];
  for (int p = threadIdx.x; p < cnt; p += 256) {
    const int64_t f = off + p;
    const int key = min(max(k_idx[f], 0), N - 1);
    keys[f] = uint32_t(row) * uint32_t(N) + uint32_t(key);
    if (vals) vals[f] = uint32_t(f);
  }
}


// ---- inverse index of lists in ascending key order -----------------------------------
// When every list is in strictly ascending key order (as fm_lists_key_order leaves them: the order the
// attention and its backward read) the inverse is a transposition that needs no sort.  Keys are taken in
// ranges of kIrRange; inside a sorted list the entries of a range are one contiguous run.
//   inv_runs_kernel       per list: first the number of entries that break the order or lie outside [0, N);
//                         for a list in order, where each range's run starts (a table [row][bucket][range]);
//   inv_table_kernel      the table turned to [row][range][bucket], and the entries per (row, range), whose
//                         prefix sum is the range's first place in inv_pos;
//   inv_transpose_kernel  one workgroup per (row, range): the runs of all the row's buckets are counted per
//                         (group of consecutive buckets, key) in LDS, a prefix over the groups and over the
//                         keys gives every group its first place per key, and the groups then walk their
//                         buckets again in ascending order handing out places -- so a key's positions come out
//                         in ascending bucket order, which is ascending position order.  A group is 16 lanes
//                         (a run is 4 entries on average at the benchmark shapes, a longer one takes further
//                         rounds), its buckets go one after the other: a bucket lists a key once, so the
//                         entries of a step never share a counter, and the steps of one wave reach LDS in
//                         program order.  The bounds of 16 buckets are fetched by the group's lanes at once
//                         (the next 16 while these are worked on), then their entries at once.  The places
//                         are handed out into an LDS image of the range's part of inv_pos, written out in
//                         whole lines afterwards: 4-byte stores in arrival order over thousands of ranges at
//                         once leave the L2 as partial lines, which cost several times the index in traffic.
// The counters are 16 bits wide: a key is in at most C <= 65535 lists.
// Every index is clamped or checked, so lists that are not in order give no index but never an access
// outside the buffers; the count of inv_runs_kernel tells the caller which it has, and the later kernels
// end at once when it is not zero.
constexpr int kIrShift = 8, kIrRange = 1 << kIrShift;  // keys per range
constexpr int kIrGroups = 32;                          // groups of consecutive buckets per workgroup
constexpr int kIrThreads = kIrGroups * 16;
constexpr int kIrStage = 8320;  // entries of a range kept in LDS for the write-out (32.5 per key; more go direct)

// S[(list) * (n_ranges + 1) + r] = first position of the list with key >= r * kIrRange
__global__ __launch_bounds__(256) void inv_runs_kernel(const int32_t* __restrict__ k_idx,
                                                       const int64_t* __restrict__ bucket_off,
                                                       const int32_t* __restrict__ bucket_cnt, int N, int n_ranges,
                                                       int32_t* __restrict__ S, int32_t* __restrict__ n_bad) {
  const int64_t b = blockIdx.x;
  const int32_t* p = k_idx + bucket_off[b];
  const int cnt = bucket_cnt[b];
  int32_t* Sb = S + b * (n_ranges + 1);
  int bad = 0;
  for (int base = 0; base < cnt; base += 2048) {
    int here[8], prev[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {  // (the loads of a thread are in flight together)
      const int i = base + u * 256 + int(threadIdx.x);
      here[u] = i < cnt ? p[i] : N - 1;
      prev[u] = i > 0 && i < cnt ? p[i - 1] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) bad += (here[u] < 0 || here[u] >= N) || prev[u] >= here[u];
  }
  bad = __syncthreads_count(bad != 0);
  if (bad) {  // a list out of order: its table stays unwritten (no index comes out of this call)
    if (threadIdx.x == 0) atomicAdd(n_bad, bad);
    return;
  }
  for (int base = 0; base <= cnt; base += 1024) {
    int here[4], prev[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = base + u * 256 + int(threadIdx.x);
      here[u] = i < cnt ? p[i] : 0;
      prev[u] = i > 0 && i <= cnt ? p[i - 1] : 0;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = base + u * 256 + int(threadIdx.x);
      if (i > cnt) continue;
      // ranges whose run starts at position i: those above the range of entry i - 1, up to the range of entry i
      const int r_prev = i > 0 ? prev[u] >> kIrShift : -1;
      const int r_here = i < cnt ? here[u] >> kIrShift : n_ranges;
      for (int r = r_prev + 1; r <= r_here; ++r) Sb[r] = i;
    }
  }
}

// The table turned to [row][range][bucket] (what the workgroup of a range reads along the buckets), as flat
// positions in k_idx (the list's offset added, clamped into the list), and the entries per (row, range)
// added into totals (zero before).  One workgroup per (row, 64 ranges, 64 buckets), the tile through LDS.
__global__ __launch_bounds__(256) void inv_table_kernel(const int32_t* __restrict__ S,
                                                        const int64_t* __restrict__ bucket_off,
                                                        const int32_t* __restrict__ bucket_cnt, int C, int n_ranges,
                                                        const int32_t* __restrict__ n_bad, int32_t* __restrict__ St,
                                                        uint32_t* __restrict__ totals) {
  if (*n_bad) return;
  __shared__ int tile[64][66];
  const int row = blockIdx.z, r0 = blockIdx.x * 64, b0 = blockIdx.y * 64, w = threadIdx.x >> 6, l = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int bl = w + 4 * i, b = b0 + bl;
    if (b < C) {
      const int64_t list = int64_t(row) * C + b;
      const int cnt = bucket_cnt[list], off = int(bucket_off[list]);
      const int32_t* s = S + list * (n_ranges + 1);
      if (r0 + l <= n_ranges) tile[bl][l] = off + min(max(s[r0 + l], 0), cnt);
      if (l == 0 && r0 + 64 <= n_ranges) tile[bl][64] = off + min(max(s[r0 + 64], 0), cnt);
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int rr = w + 4 * i, r = r0 + rr, b = b0 + l;
    int t = 0;
    if (r <= n_ranges && b < C) {
      const int v = tile[l][rr];
      St[(int64_t(row) * (n_ranges + 1) + r) * C + b] = v;
      if (r < n_ranges) t = max(tile[l][rr + 1] - v, 0);
    }
    t = wave_sum_i(t);
    if (l == 0 && r < n_ranges && t) atomicAdd(&totals[int64_t(row) * n_ranges + r], uint32_t(t));
  }
}

__global__ __launch_bounds__(kIrThreads) void inv_transpose_kernel(
    const int32_t* __restrict__ k_idx, const int32_t* __restrict__ St, const uint32_t* __restrict__ range_first,
    const int32_t* __restrict__ n_bad, int n_rows, int C, int N, int n_ranges, int64_t T,
    int32_t* __restrict__ key_off, int32_t* __restrict__ inv_pos) {
  if (*n_bad) return;
  __shared__ uint32_t cnt2[kIrGroups][kIrRange / 2];  // 16-bit counters, two to a word: [group][key of the range]
  __shared__ uint32_t first[kIrRange];                // a key's first place within the range's part of inv_pos
  __shared__ int32_t stage[kIrStage];
  __shared__ __align__(16) int xst[kIrGroups][16];  // a group's 16 buckets in hand: first entry of the run ...
  __shared__ __align__(16) uint8_t xlen[kIrGroups][16];  // ... and its length (17 = longer than the group)
  __shared__ int tmp[17];
  // Workgroups go to the 8 XCDs in turn: every XCD gets a contiguous span of (row, range) pairs, so that
  // the ranges in flight on one L2 are neighbours (four consecutive ranges share a 64-byte line of a list).
  const int64_t n_work = int64_t(n_rows) * n_ranges, per_xcd = (n_work + 7) / 8;
  const int64_t work = int64_t(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((blockIdx.x >> 3) >= per_xcd || work >= n_work) return;
  const int row = int(work / n_ranges), r = int(work - int64_t(row) * n_ranges), tid = threadIdx.x;
  const int g = tid >> 4, gl = tid & 15;
  for (int i = tid; i < kIrGroups * kIrRange / 2; i += kIrThreads) (&cnt2[0][0])[i] = 0;
  __syncthreads();
  const int per_group = (C + kIrGroups - 1) / kIrGroups;
  const int b0 = min(C, g * per_group), b1 = min(C, b0 + per_group);
  const int key0 = r << kIrShift;
  const int32_t* s0 = St + (int64_t(row) * (n_ranges + 1) + r) * C;
  // the run of this range in bucket bb + (lane of the group): flat position of its first entry, its length
  auto bounds = [&](int bb, int& st, int& len) {
    const int b = bb + gl;
    st = 0, len = 0;
    if (b < b1) {
      st = s0[b];
      len = max(s0[C + b] - st, 0);
    }
  };
  // one pass over the group's buckets in ascending order: f(key index inside the range, flat list position)
  // for every entry of the range.  The 16 lanes of a group fetch the bounds of 16 buckets, hand them to
  // one another through LDS (the waves run on their own: a group's words are written and read by its own
  // wave, in program order) and then take the buckets one by one, lane i the i-th entry of the run.
  auto walk = [&](auto f) {
    int st_n, len_n;
    bounds(b0, st_n, len_n);
    for (int bb = b0; bb < b1; bb += 16) {
      const int st = st_n, len = len_n;
      bounds(bb + 16, st_n, len_n);
      __builtin_amdgcn_wave_barrier();
      xst[g][gl] = st;
      xlen[g][gl] = uint8_t(min(len, 17));
      __builtin_amdgcn_wave_barrier();
      const bool long_run = __any(len > 16);  // (the four groups of the wave step together)
      int k[16], pos[16];
      {
        int s_u[16];
        uint32_t l4[4];
        *reinterpret_cast<int4*>(&s_u[0]) = *reinterpret_cast<const int4*>(&xst[g][0]);
        *reinterpret_cast<int4*>(&s_u[4]) = *reinterpret_cast<const int4*>(&xst[g][4]);
        *reinterpret_cast<int4*>(&s_u[8]) = *reinterpret_cast<const int4*>(&xst[g][8]);
        *reinterpret_cast<int4*>(&s_u[12]) = *reinterpret_cast<const int4*>(&xst[g][12]);
        *reinterpret_cast<uint4*>(&l4[0]) = *reinterpret_cast<const uint4*>(&xlen[g][0]);
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int l_u = int((l4[u >> 2] >> (8 * (u & 3))) & 0xffu);
          pos[u] = s_u[u] + gl;
          k[u] = gl < l_u ? k_idx[pos[u]] : -1;
        }
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int j = k[u] - key0;
        if (k[u] >= 0 && j >= 0 && j < kIrRange) f(j, pos[u]);
        if (long_run) {
          const int l_u = __shfl(len, u, 16);
          for (int p = gl + 16; __any(p < l_u); p += 16) {
            if (p < l_u) {
              const int jj = k_idx[pos[u] - gl + p] - key0;
              if (jj >= 0 && jj < kIrRange) f(jj, pos[u] - gl + p);
            }
          }
        }
      }
    }
  };
  walk([&](int j, int) { atomicAdd(&cnt2[g][j >> 1], 1u << (16 * (j & 1))); });
  __syncthreads();
  // keys 2 tid and 2 tid + 1 (one word of counters): counts of the groups -> the groups' first places within
  // the key's entries; the keys' totals -> first
  uint32_t tot0 = 0, tot1 = 0;
  if (tid < kIrRange / 2)
    for (int gg = 0; gg < kIrGroups; ++gg) {
      const uint32_t w = cnt2[gg][tid];
      cnt2[gg][tid] = (tot0 & 0xffffu) | (tot1 << 16);
      tot0 += w & 0xffffu;
      tot1 += w >> 16;
    }
  int total;
  const int ex = block_excl_scan(int(tot0 + tot1), tmp, &total);
  const uint32_t base = range_first[int64_t(row) * n_ranges + r];
  if (tid < kIrRange / 2) {
    const int j = 2 * tid;
    first[j] = uint32_t(ex);
    first[j + 1] = uint32_t(ex) + tot0;
    if (key0 + j < N) key_off[int64_t(row) * N + key0 + j] = int32_t(base + uint32_t(ex));
    if (key0 + j + 1 < N) key_off[int64_t(row) * N + key0 + j + 1] = int32_t(base + uint32_t(ex) + tot0);
  }
  if (tid == 0 && row == n_rows - 1 && r == n_ranges - 1) key_off[int64_t(n_rows) * N] = int32_t(T);
  __syncthreads();
  walk([&](int j, int pos) {
    const uint32_t old = atomicAdd(&cnt2[g][j >> 1], 1u << (16 * (j & 1)));
    const uint32_t at = first[j] + ((old >> (16 * (j & 1))) & 0xffffu);
    if (at < uint32_t(kIrStage))
      stage[at] = pos;
    else if (uint64_t(base) + at < uint64_t(T))
      inv_pos[uint64_t(base) + at] = pos;
  });
  __syncthreads();
  const int n_stage = int(min<int64_t>(min(total, kIrStage), T - int64_t(base)));
  for (int i = tid; i < n_stage; i += kIrThreads) inv_pos[uint64_t(base) + i] = stage[i];
}

// ---- step 2 ---------------------------------------------------------------------
// One wave per key; its four 16-lane groups take the key's list positions j, j+1, j+2, j+3 (a
// partial row is 16 x 16 bytes), partial sums in ascending j per group, groups added in order.
__global__ __launch_bounds__(256) void bwd_reduce_kernel(const bf16_t* __restrict__ dkp, const bf16_t* __restrict__ dvp,
                                                         const int32_t* __restrict__ key_off,
                                                         const int32_t* __restrict__ inv_pos, float* __restrict__ dk,
                                                         float* __restrict__ dv, int64_t pos0, int64_t key0,
                                                         int64_t n_keys) {
  const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t kk = key0 + int64_t(blockIdx.x) * 4 + w;
  if (kk >= key0 + n_keys) return;
  const int g = l >> 4, c = l & 15;
  const int j0 = key_off[kk], j1 = key_off[kk + 1];
  float ak[8], av[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) ak[e] = av[e] = 0.f;
  auto add_row = [&](const uint4& xk, const uint4& xv) {
    const uint32_t kw[4] = {xk.x, xk.y, xk.z, xk.w}, vw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ak[2 * e] += __uint_as_float(kw[e] << 16);
      ak[2 * e + 1] += __uint_as_float(kw[e] & 0xffff0000u);
      av[2 * e] += __uint_as_float(vw[e] << 16);
      av[2 * e + 1] += __uint_as_float(vw[e] & 0xffff0000u);
    }
  };
  auto load_row = [&](int j, uint4& xk, uint4& xv) {
    xk = xv = make_uint4(0, 0, 0, 0);
    if (j < j1) {
      const int64_t f = uint32_t(inv_pos[j]);
      xk = *reinterpret_cast<const uint4*>(dkp + (f - pos0) * 256 + 8 * c);
      xv = *reinterpret_cast<const uint4*>(dvp + (f - pos0) * 256 + 8 * c);
    }
  };
  for (int j = j0 + g; j < j1; j += 16) {  // four rows per lane group in flight, added in ascending j
    uint4 xk[4], xv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) load_row(j + 4 * u, xk[u], xv[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u) add_row(xk[u], xv[u]);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {  // ((g0 + g1) + (g2 + g3)): a fixed order
    ak[e] += __shfl_xor(ak[e], 16);
    av[e] += __shfl_xor(av[e], 16);
    ak[e] += __shfl_xor(ak[e], 32);
    av[e] += __shfl_xor(av[e], 32);
  }
  if (g == 0 && j1 > j0) {
    float4* pk = reinterpret_cast<float4*>(dk + kk * 128 + 8 * c);
    float4* pv = reinterpret_cast<float4*>(dv + kk * 128 + 8 * c);
    float4 a = pk[0], b = pk[1];
    pk[0] = make_float4(a.x + ak[0], a.y + ak[1], a.z + ak[2], a.w + ak[3]);
    pk[1] = make_float4(b.x + ak[4], b.y + ak[5], b.z + ak[6], b.w + ak[7]);
    a = pv[0];
    b = pv[1];
    pv[0] = make_float4(a.x + av[0], a.y + av[1], a.z + av[2], a.w + av[3]);
    pv[1] = make_float4(b.x + av[4], b.y + av[5], b.z + av[6], b.w + av[7]);
  }
}

}  // namespace fm

extern "C" size_t fm_inverse_index_workspace(int64_t T, int H, int N) {
  if (T < 1 || H < 1 || N < 1) return 0;
  return fm::radix_plan(T, fm::key_bits(int64_t(H) * N)).total;
}

extern "C" int fm_inverse_index(const int32_t* k_idx, const int64_t* bucket_off, const int32_t* bucket_cnt, int H,
                                int C, int N, int64_t T, int32_t* key_off, int32_t* inv_pos, void* ws,
                                size_t ws_bytes, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && C >= 1 && N >= 1 && T >= 1, FM_ERR_ARG, "fm_inverse_index: H=%d C=%d N=%d T=%lld", H, C, N,
             (long long)T);
  FM_REQUIRE(k_idx && bucket_off && bucket_cnt && key_off && inv_pos && ws, FM_ERR_ARG,
             "fm_inverse_index: null pointer");
  FM_REQUIRE(T <= 0x7fffffffLL && int64_t(H) * N < 0xffffffffLL && int64_t(H) * C <= 0x7fffffffLL, FM_ERR_UNSUPPORTED,
             "fm_inverse_index: more than 2^31 list entries or 2^32 keys");
  FM_REQUIRE(ws_bytes >= fm_inverse_index_workspace(T, H, N), FM_ERR_WORKSPACE, "fm_inverse_index: workspace %zu < %zu",
             ws_bytes, fm_inverse_index_workspace(T, H, N));
  hipStream_t st = as_stream(stream);
  const int bits = key_bits(int64_t(H) * N);
  const RadixPlan p = radix_plan(T, bits);
  char* base = static_cast<char*>(ws);
  uint32_t* ka = reinterpret_cast<uint32_t*>(base);
  // the keys row * N + key of every list entry (the first pass takes a pair's position as its value)
  hipLaunchKernelGGL(inv_pairs_kernel, dim3(unsigned(int64_t(H) * C)), dim3(256), 0, st, k_idx, bucket_off, bucket_cnt,
                     C, N, ka, static_cast<uint32_t*>(nullptr));
  const uint32_t* kin = radix_sort_positions(ws, p, T, bits, reinterpret_cast<uint32_t*>(inv_pos), st);
  const int64_t n_keys = int64_t(H) * N;
  launch_sorted_offsets(kin, T, n_keys, key_off, st);
  return launch_status("fm_inverse_index");
}

namespace fm {
struct KeyOrderPlan {
  int n_ranges;
  size_t off_turned, off_totals, total;
};
static KeyOrderPlan key_order_plan(int H, int C, int N) {
  KeyOrderPlan p;
  p.n_ranges = int(ceil_div(N, kIrRange));
  p.off_turned = align_up(size_t(H) * (p.n_ranges + 1) * C * sizeof(int32_t), 256);
  p.off_totals = 2 * p.off_turned;
  p.total = p.off_totals + align_up(size_t(H) * p.n_ranges * sizeof(uint32_t), 256) + 256;
  return p;
}
}  // namespace fm

extern "C" size_t fm_inverse_index_key_order_workspace(int H, int C, int N) {
  if (H < 1 || C < 1 || N < 1) return 0;
  return fm::key_order_plan(H, C, N).total;
}

extern "C" int fm_inverse_index_key_order(const int32_t* k_idx, const int64_t* bucket_off, const int32_t* bucket_cnt,
                                          int H, int C, int N, int64_t T, int32_t* key_off, int32_t* inv_pos,
                                          int32_t* n_bad, void* ws, size_t ws_bytes, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && C >= 1 && N >= 1 && T >= 1, FM_ERR_ARG, "fm_inverse_index_key_order: H=%d C=%d N=%d T=%lld", H, C,
             N, (long long)T);
  FM_REQUIRE(k_idx && bucket_off && bucket_cnt && key_off && inv_pos && n_bad && ws, FM_ERR_ARG,
             "fm_inverse_index_key_order: null pointer");
  FM_REQUIRE(T <= 0x7fffffffLL && int64_t(H) * N < 0x7fffffffLL && H <= 65535 && C <= 65535,
             FM_ERR_UNSUPPORTED, "fm_inverse_index_key_order: more than 2^31 list entries or keys, H > 65535 or C > 65535");
  const KeyOrderPlan p = key_order_plan(H, C, N);
  FM_REQUIRE(ws_bytes >= p.total, FM_ERR_WORKSPACE, "fm_inverse_index_key_order: workspace %zu < %zu", ws_bytes, p.total);
  hipStream_t st = as_stream(stream);
  int32_t* S = static_cast<int32_t*>(ws);
  uint32_t* totals = reinterpret_cast<uint32_t*>(static_cast<char*>(ws) + p.off_totals);
  int rc = launch_fill(n_bad, 1, 0, st);
  if (rc) return rc;
  hipLaunchKernelGGL(inv_runs_kernel, dim3(unsigned(int64_t(H) * C)), dim3(256), 0, st, k_idx, bucket_off, bucket_cnt, N,
                     p.n_ranges, S, n_bad);
  int32_t* St = reinterpret_cast<int32_t*>(static_cast<char*>(ws) + p.off_turned);
  rc = launch_fill(reinterpret_cast<int32_t*>(totals), int64_t(H) * p.n_ranges, 0, st);
  if (rc) return rc;
  hipLaunchKernelGGL(inv_table_kernel, dim3(unsigned(ceil_div(p.n_ranges + 1, 64)), unsigned(ceil_div(C, 64)), unsigned(H)),
                     dim3(256), 0, st, S, bucket_off, bucket_cnt, C, p.n_ranges, n_bad, St, totals);
  launch_scan_u32(totals, int64_t(H) * p.n_ranges, st);
  const int64_t per_xcd = ceil_div(int64_t(H) * p.n_ranges, 8);
  hipLaunchKernelGGL(inv_transpose_kernel, dim3(unsigned(8 * per_xcd)), dim3(kIrThreads), 0, st, k_idx, St, totals, n_bad,
                     H, C, N, p.n_ranges, T, key_off, inv_pos);
  return launch_status("fm_inverse_index_key_order");
}

// behind the partial rows: 8 dump rows (stores past the end of a list land there) and alignment
static constexpr size_t kStagedSlack = 8 * 128 * sizeof(fm::bf16_t) + 512;

extern "C" size_t fm_hash_attn_bwd_staged_workspace(int64_t max_row_entries) {
  return max_row_entries < 1 ? 0 : size_t(max_row_entries) * 128 * sizeof(fm::bf16_t) * 2 + kStagedSlack;
}

extern "C" int fm_hash_attn_bwd_staged(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                       const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                                       const int32_t* bin_off, const int32_t* bin_count, const void* out,
                                       const float* lse, const void* dout, const float* dlse,
                                       const int32_t* key_off, const int32_t* inv_pos, void* dq, float* dk,
                                       float* dv, int H, int Sq, int N, int d, int C, const int64_t* row_pos_host,
                                       float sm_scale, int dtype, void* ws, size_t ws_bytes, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && Sq >= 1 && N >= 1 && C >= 1, FM_ERR_ARG, "fm_hash_attn_bwd_staged: H=%d Sq=%d N=%d C=%d", H, Sq,
             N, C);
  FM_REQUIRE((dtype == FM_BF16 || dtype == FM_F16) && d == 128, FM_ERR_UNSUPPORTED,
             "fm_hash_attn_bwd_staged: bf16 or fp16 with d=128 only");
  FM_REQUIRE(q && k && v && k_idx && bucket_off && bucket_cnt && q_perm && bin_off && bin_count && out && lse && dout &&
                 key_off && inv_pos && dq && dk && dv && row_pos_host && ws,
             FM_ERR_ARG, "fm_hash_attn_bwd_staged: null pointer");
  FM_REQUIRE(C <= 65535 * 1 && H <= 65535, FM_ERR_UNSUPPORTED, "fm_hash_attn_bwd_staged: C or H above 65535");
  for (int h = 0; h < H; ++h)
    FM_REQUIRE(row_pos_host[h + 1] >= row_pos_host[h], FM_ERR_ARG, "fm_hash_attn_bwd_staged: row_pos not ascending");
  hipStream_t st = as_stream(stream);
  {  // dq of the queries without a bucket (hash outside [0, C)): 0, as for an empty bucket
    int rc = launch_unlisted_rows(q_perm, nullptr, nullptr, bin_off, bin_count, int64_t(H) * C, int64_t(H) * Sq,
                                  128 * int(sizeof(bf16_t)), dq, nullptr, st);
    if (rc) return rc;
  }
  const size_t per_entry = 128 * sizeof(bf16_t) * 2;
  const int64_t cap = int64_t((ws_bytes - std::min<size_t>(ws_bytes, kStagedSlack)) / per_entry);
  int h0 = 0;
  while (h0 < H) {
    int h1 = h0 + 1;
    FM_REQUIRE(row_pos_host[h1] - row_pos_host[h0] <= cap, FM_ERR_WORKSPACE,
               "fm_hash_attn_bwd_staged: workspace %zu holds %lld list entries, row %d has %lld", ws_bytes,
               (long long)cap, h0, (long long)(row_pos_host[h1] - row_pos_host[h0]));
    while (h1 < H && row_pos_host[h1 + 1] - row_pos_host[h0] <= cap) ++h1;
    const int64_t pos0 = row_pos_host[h0], n_pos = row_pos_host[h1] - pos0;
    if (n_pos > 0) {
      bf16_t* dkp = static_cast<bf16_t*>(ws);
      bf16_t* dvp = dkp + 128;  // a position's rows side by side: [dK | dV]
      bf16_t* dump = dkp + size_t(n_pos) * 256;
      int rc = hash_attn_bwd_staged_partials(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, bin_off, bin_count, out,
                                             lse, dout, dlse, dq, dkp, dvp, dump, pos0, h0, h1 - h0, Sq, N, C, sm_scale, dk, dv, dtype == FM_F16, st);
      if (rc) return rc;
      const int64_t n_keys = int64_t(h1 - h0) * N;
      hipLaunchKernelGGL(bwd_reduce_kernel, dim3(unsigned(ceil_div(n_keys, int64_t(4)))), dim3(256), 0, st, dkp, dvp,
                         key_off, inv_pos, dk, dv, pos0, int64_t(h0) * N, n_keys);
    }
    h0 = h1;
  }
  return launch_status("fm_hash_attn_bwd_staged");
}
