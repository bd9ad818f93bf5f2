// Device-side bookkeeping around the attention kernel: prefix sums of bucket
// sizes (triton_kernel.py:86-88), grouping of queries by (row, bucket)
// (triton_kernel.py:75-88) with the occupancy histogram (memory.py:285-286),
// and the window filter of bucket lists (memory.py:128-142).  All of it is
// integer work with data-independent launch shapes: nothing here reads a count
// back to the host.
#include "common.hpp"
#include "radix_sort.hpp"

namespace fm {

constexpr int kGrpBlock = 256;  // queries per ranking block

__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

// Single-workgroup exclusive scan int32 -> int64 over n elements.
__global__ __launch_bounds__(1024) void excl_scan_i32_i64_kernel(const int32_t* __restrict__ in,
                                                                 int64_t n,
                                                                 int64_t* __restrict__ out) {
  __shared__ long long tmp[17];
  long long carry = 0;
  for (int64_t base = 0; base < n; base += 1024) {
    int64_t i = base + threadIdx.x;
    long long v = i < n ? in[i] : 0;
    long long total;
    long long ex = block_excl_scan_ll(v, tmp, &total);
    if (i < n) out[i] = carry + ex;
    carry += total;
  }
}

// ---- grouping --------------------------------------------------------------
// Pass 1: per block of 256 consecutive queries of a row, rank every query among
// the earlier queries of the block with the same bucket; the first query of
// each bucket in the block records the block's count for that bucket.
// block_hist is [H][NB][C], zeroed beforehand.
__global__ __launch_bounds__(kGrpBlock) void group_rank_kernel(const int32_t* __restrict__ q_hash,
                                                               int C, int Sq, int NB,
                                                               int32_t* __restrict__ block_hist) {
  __shared__ int sh[kGrpBlock];
  const int h = blockIdx.y, blk = blockIdx.x, t = threadIdx.x;
  const int i = blk * kGrpBlock + t;
  int b = -1;
  if (i < Sq) {
    b = q_hash[int64_t(h) * Sq + i];
    if (b < 0 || b >= C) b = -1;  // belongs to no bucket: in no bin, no work item, no q_perm slot
  }
  sh[t] = b;
  __syncthreads();
  if (b < 0) return;
  int before = 0, total = 0;
  for (int j = 0; j < kGrpBlock; ++j) {
    int e = (sh[j] == b);
    total += e;
    before += (j < t) ? e : 0;
  }
  if (before == 0) block_hist[(int64_t(h) * NB + blk) * C + b] = total;
}

// Pass 2: per (row, bucket) turn the per-block counts into exclusive offsets
// over blocks; the total is the bucket's occupancy.
__global__ void group_colscan_kernel(int32_t* __restrict__ block_hist, int H, int C, int NB,
                                     int32_t* __restrict__ bin_count) {
  int64_t g = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (g >= int64_t(H) * C) return;
  int h = int(g / C), c = int(g - int64_t(h) * C);
  // sixteen independent loads in flight per thread; the prefix itself runs in registers
  int32_t* col = block_hist + int64_t(h) * NB * C + c;
  int run = 0;
  int blk = 0;
  for (; blk + 16 <= NB; blk += 16) {
    int v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = col[int64_t(blk + u) * C];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      col[int64_t(blk + u) * C] = run;
      run += v[u];
    }
  }
  for (; blk < NB; ++blk) {
    const int v = col[int64_t(blk) * C];
    col[int64_t(blk) * C] = run;
    run += v;
  }
  bin_count[g] = run;
}

// Pass 3: one workgroup scans the flattened [H*C] occupancies: bin_off = first
// sorted position of the bucket; item offsets = prefix sum of ceil(cnt/QTILE);
// items are written in (row, bucket, tile) order.
__global__ __launch_bounds__(1024) void group_items_kernel(const int32_t* __restrict__ bin_count,
                                                           int64_t n, int C,
                                                           int32_t* __restrict__ bin_off,
                                                           fm_item* __restrict__ items,
                                                           int32_t* __restrict__ n_items,
                                                           int64_t max_items,
                                                           int32_t* __restrict__ n_unlisted) {
  __shared__ int tmp[17];
  if (threadIdx.x == 0) *n_unlisted = 0;  // the scatter pass counts the queries without a bucket from zero
  int carry_q = 0, carry_i = 0;
  for (int64_t base = 0; base < n; base += 1024) {
    int64_t g = base + threadIdx.x;
    int cnt = g < n ? bin_count[g] : 0;
    int tiles = (cnt + FM_QTILE - 1) / FM_QTILE;
    int tq, ti;
    int exq = block_excl_scan(cnt, tmp, &tq);
    int exi = block_excl_scan(tiles, tmp, &ti);
    if (g < n) {
      int off = carry_q + exq;
      bin_off[g] = off;
      int row = int(g / C), bucket = int(g - int64_t(row) * C);
      for (int t = 0; t < tiles; ++t) {
        int64_t slot = int64_t(carry_i) + exi + t;
        if (slot < max_items) {
          fm_item it;
          it.row = row;
          it.bucket = bucket;
          it.q_start = off + t * FM_QTILE;
          it.n_q = min(FM_QTILE, cnt - t * FM_QTILE);
          items[slot] = it;
        }
      }
    }
    carry_q += tq;
    carry_i += ti;
  }
  if (threadIdx.x == 0) *n_items = int32_t(min(int64_t(carry_i), max_items));
}

// Pass 4: scatter.  position = bucket start + queries of the bucket in earlier
// blocks + rank inside the block  => stable ascending order.  A query without a bucket (hash outside
// [0, C)) goes behind the grouped ones: the grouped queries of all rows fill positions [0, T) of the
// flattened axis, T = bin_off + bin_count of the last bin, and exactly H*Sq - T queries have no bucket, so
// each takes one of the remaining slots (in no particular order) and leaves -(h*Sq + i) - 1 there, which
// is how the attention entry points find the rows no work item writes.
__global__ __launch_bounds__(kGrpBlock) void group_scatter_kernel(
    const int32_t* __restrict__ q_hash, int H, int C, int Sq, int NB,
    const int32_t* __restrict__ block_hist, const int32_t* __restrict__ bin_off,
    const int32_t* __restrict__ bin_count, int32_t* __restrict__ n_unlisted,
    int32_t* __restrict__ q_perm) {
  __shared__ int sh[kGrpBlock];
  const int h = blockIdx.y, blk = blockIdx.x, t = threadIdx.x;
  const int i = blk * kGrpBlock + t;
  int b = -1;
  if (i < Sq) {
    b = q_hash[int64_t(h) * Sq + i];
    if (b < 0 || b >= C) b = -1;
  }
  sh[t] = b;
  __syncthreads();
  if (b < 0) {
    if (i < Sq) {
      const int64_t last = int64_t(H) * C - 1;
      const int grouped = bin_off[last] + bin_count[last];
      q_perm[grouped + atomicAdd(n_unlisted, 1)] = -int32_t(int64_t(h) * Sq + i) - 1;
    }
    return;
  }
  int before = 0;
  for (int j = 0; j < t; ++j) before += (sh[j] == b);
  int pos = bin_off[int64_t(h) * C + b] + block_hist[(int64_t(h) * NB + blk) * C + b] + before;
  q_perm[pos] = i;  // pos runs over the flattened [H*Sq] sorted axis
}

// ---- grouping of long rows ----------------------------------------------------------
// The block table above is [H][Sq / 256][C] words: with a million entries a row (the keys of a K-means
// assignment, grouped by centroid) it is hundreds of megabytes that are zeroed, scanned and read again.
// From kGrpSortMinTable words of block table on the grouping is a stable radix sort of the keys row * C + bucket
// (H * C for an entry without a bucket, which therefore sorts behind all others): the sorted positions are
// q_perm, the bins' sizes come from the sorted keys.  Same q_perm, bin_off, bin_count and items as the block
// form.  (8 rows of 131072 queries over 1024 buckets, 4 M words of table: 0.11 ms by blocks, 0.13 by sort;
// 8 rows of 262144 keys over 1024 centroids, 8 M words: 0.19 against 0.15 ms; 8 rows of a million keys over
// 2048, 67 M words: 0.8 against 0.25 ms.)
constexpr int64_t kGrpSortMinTable = int64_t(1) << 23;

__global__ __launch_bounds__(256) void group_keys_kernel(const int32_t* __restrict__ q_hash, int64_t n, int C, int Sq,
                                                         uint32_t no_bucket, uint32_t* __restrict__ keys) {
  const int64_t f = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (f >= n) return;
  const int b = q_hash[f];
  keys[f] = b >= 0 && b < C ? uint32_t(f / Sq) * uint32_t(C) + uint32_t(b) : no_bucket;
}

__global__ __launch_bounds__(256) void group_bin_counts_kernel(const int32_t* __restrict__ off, int64_t n_bins,
                                                               int32_t* __restrict__ bin_count) {
  const int64_t g = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (g < n_bins) bin_count[g] = off[g + 1] - off[g];
}

// sorted flat positions -> q_perm: the entry's index inside its row, or -(flat position) - 1 without a bucket
__global__ __launch_bounds__(256) void group_perm_kernel(const uint32_t* __restrict__ sorted_keys,
                                                         const uint32_t* __restrict__ sorted_pos, int64_t n, int Sq,
                                                         uint32_t no_bucket, int32_t* __restrict__ q_perm) {
  const int64_t j = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (j >= n) return;
  const uint32_t f = sorted_pos[j];
  q_perm[j] = sorted_keys[j] == no_bucket ? -int32_t(f) - 1 : int32_t(f % uint32_t(Sq));
}

struct GroupSortPlan {
  RadixPlan radix;
  int bits;
  size_t off_pos, off_off, total;
};
static GroupSortPlan group_sort_plan(int H, int C, int Sq) {
  GroupSortPlan p;
  const int64_t n = int64_t(H) * Sq;
  p.bits = key_bits(int64_t(H) * C + 1);
  p.radix = radix_plan(n, p.bits);
  p.off_pos = p.radix.total;
  p.off_off = p.off_pos + align_up(size_t(n) * sizeof(uint32_t), 256);
  p.total = p.off_off + align_up((size_t(H) * C + 2) * sizeof(int32_t), 256);
  return p;
}
static bool group_by_sort(int H, int C, int Sq) {
  return int64_t(H) * ceil_div(Sq, kGrpBlock) * C >= kGrpSortMinTable;
}

// ---- window filter ----------------------------------------------------------
__global__ __launch_bounds__(256) void window_count_kernel(const int32_t* __restrict__ idx_in,
                                                           int64_t nb, int Z, int64_t lo,
                                                           int64_t hi, int32_t* __restrict__ cnt) {
  int64_t b = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (b >= nb) return;
  const int32_t* p = idx_in + b * Z;
  int c = 0;
  for (int j = lane_id(); j < Z; j += kWave) {
    int64_t v = p[j];
    c += (v >= lo && v < hi);
  }
  c = wave_sum_i(c);
  if (lane_id() == 0) cnt[b] = c;
}

__global__ __launch_bounds__(256) void window_compact_kernel(const int32_t* __restrict__ idx_in,
                                                             int64_t nb, int Z, int64_t lo,
                                                             int64_t hi,
                                                             const int64_t* __restrict__ off,
                                                             int32_t* __restrict__ idx_out) {
  int64_t b = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (b >= nb) return;
  const int32_t* p = idx_in + b * Z;
  int32_t* o = idx_out + off[b];
  int base = 0;
  const int l = lane_id();
  for (int j0 = 0; j0 < Z; j0 += kWave) {  // order inside the bucket is preserved
    int j = j0 + l;
    int64_t v = j < Z ? int64_t(p[j]) : -1;
    bool keep = (j < Z) && v >= lo && v < hi;
    unsigned long long m = __ballot(keep);
    int rank = __popcll(m & ((1ull << l) - 1ull));
    if (keep) o[base + rank] = int32_t(v - lo);
    base += __popcll(m);
  }
}

// Rows of the queries that are part of no work item (see group_scatter_kernel): `rows16` [nq, row_halves]
// two-byte units are zeroed and `lse` (if given) set to -FLT_MAX, the result of an empty bucket.  The number
// of grouped queries comes from the last work item, or from the last bin where there are no items at hand.
// A wave per row; usually there is none and every wave leaves after two loads.
__global__ __launch_bounds__(256) void unlisted_rows_kernel(
    const int32_t* __restrict__ q_perm, const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    const int32_t* __restrict__ bin_off, const int32_t* __restrict__ bin_count, int64_t n_bins, int64_t nq,
    int row_halves, uint16_t* __restrict__ rows16, float* __restrict__ lse) {
  int64_t grouped;
  if (items) {
    const int n = *n_items;
    grouped = n > 0 ? int64_t(items[n - 1].q_start) + items[n - 1].n_q : 0;
  } else {
    grouped = int64_t(bin_off[n_bins - 1]) + bin_count[n_bins - 1];
  }
  const int64_t wave = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6), n_waves = int64_t(gridDim.x) * 4;
  for (int64_t p = grouped + wave; p < nq; p += n_waves) {
    const int64_t g = -int64_t(q_perm[p]) - 1;
    if (g < 0 || g >= nq) continue;  // not a slot the grouping wrote: leave everything alone
    for (int w = lane_id(); w < row_halves; w += kWave) rows16[g * row_halves + w] = uint16_t(0);
    if (lse && lane_id() == 0) lse[g] = -FLT_MAX;
  }
}

int launch_unlisted_rows(const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                         const int32_t* bin_off, const int32_t* bin_count, int64_t n_bins, int64_t nq,
                         int row_bytes, void* rows, float* lse, hipStream_t st) {
  const unsigned blocks = unsigned(std::min<int64_t>(ceil_div(nq, 4), 256));
  hipLaunchKernelGGL(unlisted_rows_kernel, dim3(blocks), dim3(256), 0, st, q_perm, items, n_items, bin_off,
                     bin_count, n_bins, nq, row_bytes / 2, static_cast<uint16_t*>(rows), lse);
  return launch_status("unlisted rows");
}

int launch_fill(int32_t* p, int64_t n, int32_t v, hipStream_t st) {
  if (n <= 0) return FM_OK;
  unsigned blocks = unsigned(std::min<int64_t>(ceil_div(n, 256), 4096));
  hipLaunchKernelGGL(fill_i32_kernel, dim3(blocks), dim3(256), 0, st, p, n, v);
  return launch_status("fill");
}

}  // namespace fm

extern "C" int fm_bucket_offsets(const int32_t* cnt, int64_t n, int64_t* off_out, void* stream) {
  using namespace fm;
  FM_REQUIRE(n >= 0, FM_ERR_ARG, "fm_bucket_offsets: n=%lld", (long long)n);
  if (n == 0) return FM_OK;
  FM_REQUIRE(cnt && off_out, FM_ERR_ARG, "fm_bucket_offsets: null pointer");
  hipLaunchKernelGGL(excl_scan_i32_i64_kernel, dim3(1), dim3(1024), 0, as_stream(stream), cnt, n,
                     off_out);
  return launch_status("fm_bucket_offsets");
}

extern "C" int64_t fm_group_max_items(int H, int C, int Sq) {
  // sum over buckets of ceil(cnt/QTILE) <= #non-empty buckets + Sq/QTILE per row
  int64_t nonempty = C < Sq ? C : Sq;
  return int64_t(H) * (nonempty + Sq / FM_QTILE) + 1;
}

extern "C" size_t fm_group_queries_workspace(int H, int C, int Sq) {
  if (H >= 1 && C >= 1 && Sq >= 1 && fm::group_by_sort(H, C, Sq)) return fm::group_sort_plan(H, C, Sq).total + 256;
  int64_t NB = fm::ceil_div(Sq, fm::kGrpBlock);
  return fm::align_up(size_t(H) * size_t(NB) * size_t(C) * sizeof(int32_t), 256) + 256;
}

extern "C" int fm_group_queries(const int32_t* q_hash, int H, int C, int Sq, int32_t* q_perm,
                                int32_t* bin_count, int32_t* bin_off, fm_item* items,
                                int32_t* n_items, int64_t max_items, void* ws, size_t ws_bytes,
                                void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && C >= 1 && Sq >= 1, FM_ERR_ARG, "fm_group_queries: H=%d C=%d Sq=%d", H, C, Sq);
  FM_REQUIRE(q_hash && q_perm && bin_count && bin_off && items && n_items && ws, FM_ERR_ARG,
             "fm_group_queries: null pointer");
  FM_REQUIRE(int64_t(H) * Sq <= 0x7fffffffLL && int64_t(H) * C <= 0x7fffffffLL, FM_ERR_UNSUPPORTED,
             "fm_group_queries: H*Sq or H*C exceeds int32");
  FM_REQUIRE(H <= 65535, FM_ERR_UNSUPPORTED, "fm_group_queries: H=%d > 65535", H);
  FM_REQUIRE(max_items >= fm_group_max_items(H, C, Sq), FM_ERR_ARG,
             "fm_group_queries: max_items=%lld < %lld", (long long)max_items,
             (long long)fm_group_max_items(H, C, Sq));
  FM_REQUIRE(ws_bytes >= fm_group_queries_workspace(H, C, Sq), FM_ERR_WORKSPACE,
             "fm_group_queries: workspace %zu < %zu", ws_bytes, fm_group_queries_workspace(H, C, Sq));
  hipStream_t st = as_stream(stream);
  if (group_by_sort(H, C, Sq)) {
    const GroupSortPlan p = group_sort_plan(H, C, Sq);
    const int64_t n = int64_t(H) * Sq, n_bins = int64_t(H) * C;
    const uint32_t no_bucket = uint32_t(n_bins);
    char* base = static_cast<char*>(ws);
    uint32_t* pos = reinterpret_cast<uint32_t*>(base + p.off_pos);
    int32_t* off = reinterpret_cast<int32_t*>(base + p.off_off);
    int32_t* n_unlisted = reinterpret_cast<int32_t*>(base + p.total);  // (the items kernel zeroes it; unused here)
    const unsigned blocks = unsigned(ceil_div(n, int64_t(256)));
    hipLaunchKernelGGL(group_keys_kernel, dim3(blocks), dim3(256), 0, st, q_hash, n, C, Sq, no_bucket,
                       reinterpret_cast<uint32_t*>(base));
    const uint32_t* sorted = radix_sort_positions(ws, p.radix, n, p.bits, pos, st);
    launch_sorted_offsets(sorted, n, n_bins, off, st);
    hipLaunchKernelGGL(group_bin_counts_kernel, dim3(unsigned(ceil_div(n_bins, int64_t(256)))), dim3(256), 0, st, off,
                       n_bins, bin_count);
    hipLaunchKernelGGL(group_items_kernel, dim3(1), dim3(1024), 0, st, bin_count, n_bins, C, bin_off, items, n_items,
                       max_items, n_unlisted);
    hipLaunchKernelGGL(group_perm_kernel, dim3(blocks), dim3(256), 0, st, sorted, pos, n, Sq, no_bucket, q_perm);
    return launch_status("fm_group_queries");
  }
  const int NB = int(ceil_div(Sq, kGrpBlock));
  int32_t* block_hist = static_cast<int32_t*>(ws);
  // counter of the queries without a bucket: the spare 256 bytes behind the block table
  int32_t* n_unlisted = reinterpret_cast<int32_t*>(static_cast<char*>(ws) +
                                                   align_up(size_t(H) * size_t(NB) * size_t(C) * sizeof(int32_t), 256));
  int rc = launch_fill(block_hist, int64_t(H) * NB * C, 0, st);
  if (rc) return rc;
  hipLaunchKernelGGL(group_rank_kernel, dim3(NB, H), dim3(kGrpBlock), 0, st, q_hash, C, Sq, NB,
                     block_hist);
  hipLaunchKernelGGL(group_colscan_kernel, dim3(unsigned(ceil_div(int64_t(H) * C, 256))), dim3(256),
                     0, st, block_hist, H, C, NB, bin_count);
  hipLaunchKernelGGL(group_items_kernel, dim3(1), dim3(1024), 0, st, bin_count, int64_t(H) * C, C,
                     bin_off, items, n_items, max_items, n_unlisted);
  hipLaunchKernelGGL(group_scatter_kernel, dim3(NB, H), dim3(kGrpBlock), 0, st, q_hash, H, C, Sq, NB,
                     block_hist, bin_off, bin_count, n_unlisted, q_perm);
  return launch_status("fm_group_queries");
}

extern "C" size_t fm_window_filter_workspace(int64_t) { return 0; }

extern "C" int fm_window_filter(const int32_t* idx_in, int64_t nb, int Z, int64_t lo, int64_t hi,
                                int32_t* idx_out, int32_t* cnt_out, int64_t* off_out, void* ws,
                                size_t ws_bytes, void* stream) {
  using namespace fm;
  (void)ws;
  (void)ws_bytes;
  FM_REQUIRE(nb >= 0 && Z >= 1, FM_ERR_ARG, "fm_window_filter: nb=%lld Z=%d", (long long)nb, Z);
  if (nb == 0) return FM_OK;
  FM_REQUIRE(idx_in && idx_out && cnt_out && off_out, FM_ERR_ARG, "fm_window_filter: null pointer");
  hipStream_t st = as_stream(stream);
  unsigned blocks = unsigned(ceil_div(nb, 4));
  hipLaunchKernelGGL(window_count_kernel, dim3(blocks), dim3(256), 0, st, idx_in, nb, Z, lo, hi,
                     cnt_out);
  hipLaunchKernelGGL(excl_scan_i32_i64_kernel, dim3(1), dim3(1024), 0, st, cnt_out, nb, off_out);
  hipLaunchKernelGGL(window_compact_kernel, dim3(blocks), dim3(256), 0, st, idx_in, nb, Z, lo, hi,
                     off_out, idx_out);
  return launch_status("fm_window_filter");
}
