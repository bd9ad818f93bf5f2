// Grouped launch of the bucket-gathered attention whose rows go from global memory straight into LDS
// (attn_ring.hpp): one workgroup per three consecutive work items of a bucket (192 queries, 48 per wave),
// the form for buckets with many queries.  A bucket of up to 192 queries is swept once.
#include "attn_ring.hpp"

namespace fm {

template <bool F16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void hash_attn_ring_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2, int only_row) {
  extern __shared__ __attribute__((aligned(16))) bf16_t ring_lds[];
  int n_it = *n_items;
  int first = 0;
  if (only_row >= 0) {  // a launch per row: the row's items are [first, n_it)
    first = first_item_of_row(items, n_it, only_row);
    n_it = first_item_of_row(items, n_it, only_row + 1);
  }
  if (first + int(blockIdx.x) >= n_it) return;
  // Workgroups go to the eight XCDs in turn (workgroup b to XCD b % 8), each with an L2 of its own.  Within
  // every 64 items, XCD x takes the eight consecutive ones [8x, 8x + 8): the workgroups of one bucket, which
  // gather the same rows, then run at about the same time behind the same L2 and the second finds there what
  // the first has fetched (15 % fewer bytes fetched at the reference's harness shape), while the launch as a
  // whole still walks the items, and with them the rows of K and V, in order.
  int me = blockIdx.x;
  if (first + (me | 63) < n_it) me = (me & ~63) | ((me & 7) << 3) | ((me >> 3) & 7);
  me += first;
  const fm_item it = items[me];
  // The items of a bucket are consecutive and their queries contiguous: the workgroup of item lo + 3j takes
  // the items lo + 3j .. lo + 3j + 2 of the bucket, the ones launched for the other two have nothing to do.
  // (The bucket's first item by a galloping, then a binary search: a bucket may have thousands of items.)
  auto same = [&](int i) { return items[i].row == it.row && items[i].bucket == it.bucket; };
  int lo = me, step = 1;  // invariant: items lo..me belong to the bucket
  while (lo - step >= first && same(lo - step)) {
    lo -= step;
    step <<= 1;
  }
  int bad = max(lo - step, first - 1);  // first - 1 or an item of another bucket, bad < lo
  while (lo - bad > 1) {
    const int mid = (lo + bad) >> 1;
    if (same(mid))
      lo = mid;
    else
      bad = mid;
  }
  if ((me - lo) % 3) return;
  int n_q = it.n_q;
  if (me + 1 < n_it && same(me + 1)) {
    n_q += items[me + 1].n_q;
    if (me + 2 < n_it && same(me + 2)) n_q += items[me + 2].n_q;
  }
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int64_t qbase = int64_t(it.row) * Sq;
  attend_ring<3, F16>(q + qbase * kSD, q_perm + it.q_start, n_q, k + int64_t(it.row) * N * kSD,
                      v + int64_t(it.row) * N * kSD, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                      out + qbase * kSD, lse + qbase, ring_lds, it.bucket);
}

int hash_attn_mfma_ring(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                        const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items,
                        const int32_t* n_items, int64_t max_items, void* out, float* lse, int Sq, int N, int C,
                        float sm_scale, bool f16, int H, bool per_row, hipStream_t st) {
#define FM_RING_LAUNCH(F16, GRID, ROW)                                                                            \
  do {                                                                                                            \
    FM_ALLOW_LDS((hash_attn_ring_kernel<F16>), kRingLdsBytes, "fm_hash_attn_fwd: lds");                           \
    hipLaunchKernelGGL((hash_attn_ring_kernel<F16>), dim3(unsigned(GRID)), dim3(256), kRingLdsBytes, st,          \
                       (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm, \
                       items, n_items, (bf16_t*)out, lse, Sq, N, C, sm_scale * kLog2e, ROW);                      \
  } while (0)
  if (per_row) {
    // One launch per row, in row order: the workgroups of a launch start together and sweep the row's K and
    // V (lists in ascending key order) at about the same pace, so a key row that several buckets list is
    // fetched from HBM once and found in the last-level cache, or the L2, by the others.  In a single launch
    // over all rows the starts spread over the whole sweep after a few rounds of workgroups, and two rows'
    // sweeps overlap at every row boundary.
    const int64_t row_items = std::min<int64_t>(max_items, int64_t(C < Sq ? C : Sq) + Sq / FM_QTILE + 1);
    for (int row = 0; row < H; ++row) {
      if (f16)
        FM_RING_LAUNCH(true, row_items, row);
      else
        FM_RING_LAUNCH(false, row_items, row);
    }
  } else if (f16) {
    FM_RING_LAUNCH(true, max_items, -1);
  } else {
    FM_RING_LAUNCH(false, max_items, -1);
  }
#undef FM_RING_LAUNCH
  return launch_status("fm_hash_attn_fwd(mfma, ring)");
}

}  // namespace fm
