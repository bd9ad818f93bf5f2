// Grouped launch of the bucket-gathered attention whose rows go from global memory straight into LDS
// (attn_ring.hpp): one workgroup per three consecutive work items of a bucket (192 queries, 48 per wave),
// the form for buckets with many queries.  A bucket of up to 192 queries is swept once.
#include "attn_ring.hpp"

namespace fm {


// heads[j] = the first item of the j-th group of up to three consecutive items of one bucket, in item order;
// *n_heads = their number.  Two passes of one workgroup per 1024 items: the first counts the groups' first items
// of its 1024, the second adds the counts of the workgroups before it and packs them by a prefix sum.  An item's
// place in its bucket is its distance from the bucket's first item, found by a galloping, then a binary search
// to the left (a bucket may have thousands of items).
__device__ __forceinline__ bool ring_is_head(const fm_item* __restrict__ items, int i) {
  const fm_item it = items[i];
  auto same = [&](int j) { return items[j].row == it.row && items[j].bucket == it.bucket; };
  int lo = i, step = 1;  // invariant: items lo..i belong to the bucket
  while (lo - step >= 0 && same(lo - step)) {
    lo -= step;
    step <<= 1;
  }
  int bad = max(lo - step, -1);  // -1 or an item of another bucket, bad < lo
  while (lo - bad > 1) {
    const int mid = (lo + bad) >> 1;
    if (same(mid))
      lo = mid;
    else
      bad = mid;
  }
  return (i - lo) % 3 == 0;
}

__global__ __launch_bounds__(1024) void ring_heads_count_kernel(const fm_item* __restrict__ items,
                                                                const int32_t* __restrict__ n_items,
                                                                int32_t* __restrict__ counts) {
  __shared__ int scan_tmp[17];
  const int i = blockIdx.x * 1024 + threadIdx.x;
  const bool head = i < *n_items && ring_is_head(items, i);
  int total;
  block_excl_scan(head ? 1 : 0, scan_tmp, &total);
  if (threadIdx.x == 0) counts[blockIdx.x] = total;
}

__global__ __launch_bounds__(1024) void ring_heads_write_kernel(const fm_item* __restrict__ items,
                                                                const int32_t* __restrict__ n_items,
                                                                const int32_t* __restrict__ counts,
                                                                int32_t* __restrict__ heads,
                                                                int32_t* __restrict__ n_heads) {
  __shared__ int scan_tmp[17];
  int before = 0;
  for (int j = threadIdx.x; j < int(blockIdx.x); j += 1024) before += counts[j];
  int base;
  block_excl_scan(before, scan_tmp, &base);
  const int i = blockIdx.x * 1024 + threadIdx.x;
  const bool head = i < *n_items && ring_is_head(items, i);
  int total;
  const int pos = block_excl_scan(head ? 1 : 0, scan_tmp, &total);
  if (head) heads[base + pos] = i;
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) *n_heads = base + total;
}

template <bool F16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void hash_attn_ring_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2, int only_row,
    const int32_t* __restrict__ heads, const int32_t* __restrict__ n_heads) {
  extern __shared__ __attribute__((aligned(16))) bf16_t ring_lds[];
  int n_it = *n_items;
  if (heads) {  // the groups of items have been listed: every workgroup up to their number has one to work on
    const int n_h = *n_heads;
    if (int(blockIdx.x) >= n_h) return;
    int b = blockIdx.x;
    if ((b | 63) < n_h) b = (b & ~63) | ((b & 7) << 3) | ((b >> 3) & 7);  // (the XCD placement described below)
    const int head = heads[b];
    const fm_item it = items[head];
    int n_q = it.n_q;
    for (int j = 1; j < 3 && head + j < n_it && items[head + j].row == it.row && items[head + j].bucket == it.bucket; ++j)
      n_q += items[head + j].n_q;
    const int64_t bkt = int64_t(it.row) * C + it.bucket;
    const int64_t qbase = int64_t(it.row) * Sq;
    attend_ring<3, F16>(q + qbase * kSD, q_perm + it.q_start, n_q, k + int64_t(it.row) * N * kSD,
                        v + int64_t(it.row) * N * kSD, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                        out + qbase * kSD, lse + qbase, ring_lds, it.bucket);
    return;
  }
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
  // The items of a bucket are consecutive and their queries contiguous: the items lo + 3j .. lo + 3j + 2 of the
  // bucket are taken together by the workgroup launched for one of them, the ones launched for the other two
  // have nothing to do.  (The bucket's first item by a galloping, then a binary search: a bucket may have
  // thousands of items.)
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
  const int head = me - (me - lo) % 3;  // the first of the three
  int n_q = items[head].n_q, n_here = 1;
  if (head + 1 < n_it && same(head + 1)) {
    n_q += items[head + 1].n_q;
    n_here = 2;
    if (head + 2 < n_it && same(head + 2)) {
      n_q += items[head + 2].n_q;
      n_here = 3;
    }
  }
  // Which of them works changes with every 256 items, one round of the dispatcher over the device's compute
  // units: workgroups are handed to the compute units in turn and in order, one that has no room holds up all
  // that follow, and a workgroup that returns at once occupies nothing.  With the same member working in every
  // group, buckets of two items each (65 to 128 queries) gave every second compute unit all the work and the
  // others none (measured: compute units busy 49 % of the launch, 3.03 ms against 2.87 ms for half as much work
  // again in buckets of three items).
  if (me != head + ((head - first) >> 8) % n_here) return;
  const fm_item it0 = items[head];
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int64_t qbase = int64_t(it.row) * Sq;
  attend_ring<3, F16>(q + qbase * kSD, q_perm + it0.q_start, n_q, k + int64_t(it.row) * N * kSD,
                      v + int64_t(it.row) * N * kSD, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                      out + qbase * kSD, lse + qbase, ring_lds, it.bucket);
}

// n_heads (64 ints reserved), heads[max_items], counts[ceil(max_items / 1024)]
size_t hash_attn_ring_workspace(int64_t max_items) {
  return (size_t(max_items) + 64 + size_t(ceil_div(max_items, int64_t(1024)))) * sizeof(int32_t);
}

int hash_attn_mfma_ring(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                        const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items,
                        const int32_t* n_items, int64_t max_items, void* out, float* lse, int Sq, int N, int C,
                        float sm_scale, bool f16, int H, bool per_row, void* ws, size_t ws_bytes, hipStream_t st) {
  // With many queries per bucket most items are the second or third of a group of three, and a workgroup
  // launched for one of those returns at once.  Workgroups are handed to the compute units in turn and in
  // order, and one that finds its compute unit full holds up all that follow: a compute unit that keeps being
  // handed workgroups without work idles (measured at 128 queries per bucket on average, buckets of two and
  // three items mixed: the launch at 70 % of its rate with none of them).  Given memory for it, the groups are
  // listed first and only as many workgroups as there are groups do anything at all, the rest at the end of
  // the grid.
  int32_t* heads = nullptr;
  int32_t* n_heads = nullptr;
  if (!per_row && ws && ws_bytes >= hash_attn_ring_workspace(max_items) && int64_t(Sq) >= int64_t(FM_QTILE) * C) {
    n_heads = static_cast<int32_t*>(ws);
    heads = n_heads + 64;
    int32_t* counts = heads + max_items;
    const unsigned nblk = unsigned(ceil_div(max_items, int64_t(1024)));
    hipLaunchKernelGGL(ring_heads_count_kernel, dim3(nblk), dim3(1024), 0, st, items, n_items, counts);
    hipLaunchKernelGGL(ring_heads_write_kernel, dim3(nblk), dim3(1024), 0, st, items, n_items, counts, heads, n_heads);
  }
#define FM_RING_LAUNCH(F16, GRID, ROW)                                                                            \
  do {                                                                                                            \
    FM_ALLOW_LDS((hash_attn_ring_kernel<F16>), kRingLdsBytes, "fm_hash_attn_fwd: lds");                           \
    hipLaunchKernelGGL((hash_attn_ring_kernel<F16>), dim3(unsigned(GRID)), dim3(256), kRingLdsBytes, st,          \
                       (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm, \
                       items, n_items, (bf16_t*)out, lse, Sq, N, C, sm_scale * kLog2e, ROW, heads, n_heads);      \
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
