// Grouped launch of the staged bucket-gathered attention (attn_staged.hpp): one workgroup per work
// item, or per two consecutive items of a bucket.
#include "attn_staged.hpp"

namespace fm {

// NQW = 16-query tiles per wave.  1: a workgroup takes one work item (64 queries), three workgroups per
// CU.  2: a workgroup takes two consecutive items of a bucket (128 queries; the workgroup of the second
// item exits), each LDS operand read feeds two MFMAs, two workgroups per CU: half the LDS reads,
// staging and barriers per query -- the form for buckets that receive 64 queries or more on average.
template <int NQW, bool F16, bool BIGN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4 - NQW, 4 - NQW))) void hash_attn_staged_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2, int only_row) {
  extern __shared__ __attribute__((aligned(16))) bf16_t st_lds[];
  const int n_it = *n_items;
  int item_id = blockIdx.x;
  if (NQW == 1 && only_row >= 0) {
    // a launch per row: workgroup j takes the row's j-th item
    const int lo = first_item_of_row(items, n_it, only_row);
    item_id += lo;
    if (item_id >= n_it || items[item_id].row != only_row) return;
  }
  if (item_id >= n_it) return;
  const fm_item it = items[item_id];
  int n_q = it.n_q;
  if (NQW == 2) {
    // the items of a bucket are consecutive and their queries contiguous: this workgroup takes items
    // 2j and 2j+1 of the bucket, the one launched for item 2j+1 has nothing to do
    // (the bucket's first item by a galloping then a binary search over the item list: a bucket that holds most
    // of a row's queries has thousands of items, and a linear walk back would be that many dependent loads)
    const int me = blockIdx.x;
    auto same = [&](int i) { return items[i].row == it.row && items[i].bucket == it.bucket; };
    int lo = me, step = 1;                         // invariant: items lo..me belong to the bucket
    while (lo - step >= 0 && same(lo - step)) {
      lo -= step;
      step <<= 1;
    }
    int bad = max(lo - step, -1);                  // -1 or an item of another bucket, bad < lo
    while (lo - bad > 1) {
      const int mid = (lo + bad) >> 1;
      if (same(mid))
        lo = mid;
      else
        bad = mid;
    }
    if ((me - lo) & 1) return;
    if (int(blockIdx.x) + 1 < n_it) {
      const fm_item nx = items[blockIdx.x + 1];
      if (nx.row == it.row && nx.bucket == it.bucket) n_q += nx.n_q;
    }
  }
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int64_t qbase = int64_t(it.row) * Sq;
  attend_staged<NQW, F16, BIGN>(q + qbase * kSD, q_perm + it.q_start, n_q, k + int64_t(it.row) * N * kSD,
                     v + int64_t(it.row) * N * kSD, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                     out + qbase * kSD, lse + qbase, st_lds);
}

#define FM_STAGED_ROW_LAUNCH(F16, BIGN)                                                                              \
  do {                                                                                                              \
    FM_ALLOW_LDS((hash_attn_staged_kernel<1, F16, BIGN>), kStagedTileBytes, "fm_hash_attn_fwd: lds");               \
    hipLaunchKernelGGL((hash_attn_staged_kernel<1, F16, BIGN>), dim3(unsigned(row_items)), dim3(256),               \
                       kStagedTileBytes, st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx,           \
                       bucket_off, bucket_cnt, q_perm, items, n_items, (bf16_t*)out, lse, Sq, N, C,                 \
                       sm_scale * kLog2e, row);                                                                     \
  } while (0)

int hash_attn_mfma_staged(const void* q, const void* k, const void* v, const int32_t* k_idx,
                          const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                          const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                          float* lse, int H, int Sq, int N, int C, float sm_scale, bool pairs, bool f16, bool per_row,
                          hipStream_t st) {
  constexpr size_t kTileBytes = kStagedTileBytes;
  if (per_row && !pairs) {
    // One launch per row, in row order.  The workgroups of a launch start together and sweep the row's K
    // and V at about the same pace (lists in ascending key order), so a key row that several buckets list
    // is fetched from HBM once and found in the last-level cache, or the L2, by the others; in a single
    // launch over all rows the starts spread over the whole sweep after a few rounds of workgroups and two
    // rows' sweeps overlap at every row boundary.  Measured on 8 rows of 2^20 keys, 2048 buckets of 16384:
    // 14.0 ms against 15.9 ms.
    const int64_t row_items = std::min<int64_t>(max_items, int64_t(C < Sq ? C : Sq) + Sq / FM_QTILE + 1);
    for (int row = 0; row < H; ++row) {
      if (N > (1 << 24)) {
        if (f16)
          FM_STAGED_ROW_LAUNCH(true, true);
        else
          FM_STAGED_ROW_LAUNCH(false, true);
      } else if (f16) {
        FM_STAGED_ROW_LAUNCH(true, false);
      } else {
        FM_STAGED_ROW_LAUNCH(false, false);
      }
    }
    return launch_status("fm_hash_attn_fwd(mfma, staged, per row)");
  }
#define FM_STAGED_LAUNCH(NQW, F16) FM_STAGED_LAUNCH3(NQW, F16, false)
#define FM_STAGED_LAUNCH3(NQW, F16, BIGN)                                                                                   \
  do {                                                                                                               \
    FM_ALLOW_LDS((hash_attn_staged_kernel<NQW, F16, BIGN>), NQW * kTileBytes, "fm_hash_attn_fwd: lds");                     \
    hipLaunchKernelGGL((hash_attn_staged_kernel<NQW, F16, BIGN>), dim3(unsigned(max_items)), dim3(256), NQW * kTileBytes,  \
                       st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt,      \
                       q_perm, items, n_items, (bf16_t*)out, lse, Sq, N, C, sm_scale * kLog2e, -1);                  \
  } while (0)
  if (N > (1 << 24)) {  // 64-bit row offsets; one work item per workgroup only
    if (f16)
      FM_STAGED_LAUNCH3(1, true, true);
    else
      FM_STAGED_LAUNCH3(1, false, true);
  } else if (pairs && f16)
    FM_STAGED_LAUNCH(2, true);
  else if (pairs)
    FM_STAGED_LAUNCH(2, false);
  else if (f16)
    FM_STAGED_LAUNCH(1, true);
  else
    FM_STAGED_LAUNCH(1, false);
#undef FM_STAGED_LAUNCH
#undef FM_STAGED_ROW_LAUNCH
#undef FM_STAGED_LAUNCH3
  return launch_status("fm_hash_attn_fwd(mfma, staged)");
}

}  // namespace fm
