// Backward of the bucket-gathered attention without atomics, for dense query
// sets (bf16, head dimension 128).
//
// A key belongs to many buckets (C Z / N of them on average), so its dK and dV
// rows collect contributions from many workgroups.  Memory-side fp32 atomics
// sustain a fraction of the HBM rate; here the contributions are staged:
//   1. hash_attn_bwd_staged_kernel (attn_bwd_mfma.hip): one workgroup per
//      (row, bucket) writes the bucket's own dK, dV partial rows, one bf16 row of
//      128 per listed key, at the key's flat list position -- plain coalesced
//      stores, 2 x 256 B per (bucket, key) pair; dQ is complete after this step;
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

#include <rocprim/device/device_radix_sort.hpp>

#include "common.hpp"

namespace fm {

int launch_unlisted_rows(const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                         const int32_t* bin_off, const int32_t* bin_count, int64_t n_bins, int64_t nq,
                         int row_bytes, void* rows, float* lse, hipStream_t st);  // group.hip
int hash_attn_bwd_staged_partials(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                  const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                                  const int32_t* bin_off, const int32_t* bin_count, const void* out, const float* lse,
                                  const void* dout, const float* dlse, void* dq, void* dkp, void* dvp, void* dump, int64_t pos0,
                                  int row0, int rows, int Sq, int N, int C, float sm_scale, float* dk, float* dv,
                                  hipStream_t st);  // attn_bwd_mfma.hip

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
    vals[f] = uint32_t(f);
  }
}

// key_off[kk] = first sorted position whose key is >= kk, for kk = 0 .. n_keys (n_keys + 1 outputs).
__global__ __launch_bounds__(256) void inv_offsets_kernel(const uint32_t* __restrict__ sorted_keys, int64_t T,
                                                          int64_t n_keys, int32_t* __restrict__ key_off) {
  const int64_t kk = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (kk > n_keys) return;
  int64_t lo = 0, hi = T;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (uint64_t(sorted_keys[mid]) < uint64_t(kk))
      lo = mid + 1;
    else
      hi = mid;
  }
  key_off[kk] = int32_t(lo);
}

static size_t sort_temp_bytes(int64_t T, int bits) {
  size_t bytes = 0;
  (void)rocprim::radix_sort_pairs(nullptr, bytes, static_cast<uint32_t*>(nullptr), static_cast<uint32_t*>(nullptr),
                                  static_cast<uint32_t*>(nullptr), static_cast<uint32_t*>(nullptr), size_t(T), 0,
                                  unsigned(bits), hipStream_t(nullptr));
  return bytes;
}

static int key_bits(int64_t n_keys) {
  int bits = 1;
  while ((int64_t(1) << bits) < n_keys) ++bits;
  return bits;
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
      xk = *reinterpret_cast<const uint4*>(dkp + (f - pos0) * 128 + 8 * c);
      xv = *reinterpret_cast<const uint4*>(dvp + (f - pos0) * 128 + 8 * c);
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
  const size_t arr = fm::align_up(size_t(T) * sizeof(uint32_t), 256);
  return 3 * arr + fm::align_up(fm::sort_temp_bytes(T, fm::key_bits(int64_t(H) * N)), 256) + 256;
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
  const size_t arr = align_up(size_t(T) * sizeof(uint32_t), 256);
  char* base = static_cast<char*>(ws);
  uint32_t* keys_in = reinterpret_cast<uint32_t*>(base);
  uint32_t* keys_out = reinterpret_cast<uint32_t*>(base + arr);
  uint32_t* vals_in = reinterpret_cast<uint32_t*>(base + 2 * arr);
  void* temp = base + 3 * arr;
  const int bits = key_bits(int64_t(H) * N);
  size_t temp_bytes = sort_temp_bytes(T, bits);
  hipLaunchKernelGGL(inv_pairs_kernel, dim3(unsigned(int64_t(H) * C)), dim3(256), 0, st, k_idx, bucket_off, bucket_cnt,
                     C, N, keys_in, vals_in);
  hipError_t e = rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, vals_in,
                                           reinterpret_cast<uint32_t*>(inv_pos), size_t(T), 0, unsigned(bits), st);
  FM_REQUIRE(e == hipSuccess, FM_ERR_LAUNCH, "fm_inverse_index: sort: %s", hipGetErrorString(e));
  const int64_t n_keys = int64_t(H) * N;
  hipLaunchKernelGGL(inv_offsets_kernel, dim3(unsigned(ceil_div(n_keys + 1, int64_t(256)))), dim3(256), 0, st, keys_out,
                     T, n_keys, key_off);
  return launch_status("fm_inverse_index");
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
  FM_REQUIRE(dtype == FM_BF16 && d == 128, FM_ERR_UNSUPPORTED, "fm_hash_attn_bwd_staged: bf16 with d=128 only");
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
      bf16_t* dvp = dkp + size_t(n_pos) * 128;
      bf16_t* dump = dvp + size_t(n_pos) * 128;
      int rc = hash_attn_bwd_staged_partials(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, bin_off, bin_count, out,
                                             lse, dout, dlse, dq, dkp, dvp, dump, pos0, h0, h1 - h0, Sq, N, C, sm_scale, dk, dv, st);
      if (rc) return rc;
      const int64_t n_keys = int64_t(h1 - h0) * N;
      hipLaunchKernelGGL(bwd_reduce_kernel, dim3(unsigned(ceil_div(n_keys, int64_t(4)))), dim3(256), 0, st, dkp, dvp,
                         key_off, inv_pos, dk, dv, pos0, int64_t(h0) * N, n_keys);
    }
    h0 = h1;
  }
  return launch_status("fm_hash_attn_bwd_staged");
}
