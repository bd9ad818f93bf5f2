#include <algorithm>

#include "radix_sort.hpp"

namespace fm {

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


// ---- stable radix sort of (key, position) pairs --------------------------------------
// Least significant digit first, digits of up to 8 bits, three kernels a pass:
//   radix_hist_kernel     a workgroup counts the digits of its tile of 4096 pairs; counts land digit-major
//                         ([digit][tile]), so that their exclusive prefix sum is every (digit, tile)'s first
//                         place in the output;
//   radix_scan_kernel /   that prefix sum in chunks of 16384 counts (a workgroup each) and, by one workgroup,
//   radix_scan_top_kernel over the chunks' totals;
//   radix_scatter_kernel  the tile again: wave w takes pairs 1024 w .. 1024 w + 1023 of the tile, 64 consecutive
//                         ones a step.  The lanes that hold the same digit find each other with one ballot per
//                         digit bit; a pair's rank among the wave's earlier pairs of its digit is the wave's
//                         counter of that digit plus the number of such lanes below it -- steps run in order and
//                         lanes are in pair order, so equal digits keep their order (the sort is stable: a key's
//                         positions come out ascending).  The waves' counters are then turned into their first
//                         places inside the tile, the tile is put in order in LDS, and it leaves as runs of
//                         consecutive places, one run per digit.
// HBM-bound: a pass reads 12 bytes and writes 8 per pair (the first pass forms its keys from the lists).
constexpr int kRsThreads = 256, kRsWaves = 4, kRsItems = 16;
constexpr int kRsTile = kRsThreads * kRsItems;  // 4096 pairs per workgroup
constexpr int kRsChunk = 16384;                 // counts per workgroup of the prefix sum

__global__ __launch_bounds__(kRsThreads) void radix_hist_kernel(const uint32_t* __restrict__ keys, int64_t T,
                                                                int shift, int nd, int64_t n_tiles,
                                                                uint32_t* __restrict__ hist) {
  __shared__ uint32_t h[256];
  const int tid = threadIdx.x;
  h[tid] = 0;
  __syncthreads();
  const int64_t base = int64_t(blockIdx.x) * kRsTile;
#pragma unroll
  for (int s = 0; s < kRsItems; ++s) {
    const int64_t i = base + int64_t(s) * kRsThreads + tid;
    if (i < T) atomicAdd(&h[(keys[i] >> shift) & uint32_t(nd - 1)], 1u);
  }
  __syncthreads();
  if (tid < nd) hist[int64_t(tid) * n_tiles + blockIdx.x] = h[tid];
}

// exclusive prefix sums inside chunks of kRsChunk counts (in place) and the chunks' totals
__global__ __launch_bounds__(1024) void radix_scan_kernel(uint32_t* __restrict__ hist, int64_t n,
                                                          uint32_t* __restrict__ chunk_total) {
  __shared__ int tmp[17];
  const int64_t base = int64_t(blockIdx.x) * kRsChunk + int64_t(threadIdx.x) * 16;
  uint32_t v[16];
  int local = 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    v[j] = base + j < n ? hist[base + j] : 0u;
    local += int(v[j]);
  }
  int total;
  int run = block_excl_scan(local, tmp, &total);
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    if (base + j < n) hist[base + j] = uint32_t(run);
    run += int(v[j]);
  }
  if (threadIdx.x == 0) chunk_total[blockIdx.x] = uint32_t(total);
}

// exclusive prefix sum over the chunks' totals, one workgroup
__global__ __launch_bounds__(1024) void radix_scan_top_kernel(uint32_t* __restrict__ chunk_total, int64_t n_chunks) {
  __shared__ int tmp[17];
  int carry = 0;
  for (int64_t base = 0; base < n_chunks; base += 1024) {
    const int64_t i = base + threadIdx.x;
    const int v = i < n_chunks ? int(chunk_total[i]) : 0;
    int total;
    const int ex = block_excl_scan(v, tmp, &total);
    if (i < n_chunks) chunk_total[i] = uint32_t(carry + ex);
    carry += total;
  }
}

// vals_in == nullptr: a pair's value is its index (the first pass).  The tile is put in order inside LDS first,
// so that what goes to memory are runs of consecutive places (a digit's pairs of the tile), not 64 scattered
// words per store.
__global__ __launch_bounds__(kRsThreads) void radix_scatter_kernel(
    const uint32_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, uint32_t* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, int64_t T, int shift, int nd, int n_bits, int64_t n_tiles,
    const uint32_t* __restrict__ hist, const uint32_t* __restrict__ chunk_off) {
  __shared__ uint32_t wcnt[kRsWaves][256];  // a wave's count of a digit, then its first place inside the tile
  __shared__ uint32_t dstart[256];          // first place of a digit inside the tile
  __shared__ uint32_t gfirst[256];          // ... in the output, minus dstart
  __shared__ uint32_t sk[kRsTile], sv[kRsTile];
  __shared__ int tmp[17];
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  for (int d = tid; d < kRsWaves * 256; d += kRsThreads) (&wcnt[0][0])[d] = 0;
  __syncthreads();
  constexpr int kWaveItems = kRsTile / kRsWaves;  // 1024 pairs per wave, kRsItems steps of 64
  const int64_t tile0 = int64_t(blockIdx.x) * kRsTile;
  const int64_t base = tile0 + int64_t(w) * kWaveItems + l;
  const uint64_t lt = (uint64_t(1) << l) - 1u;
  uint32_t key[kRsItems], rank[kRsItems];
#pragma unroll
  for (int s = 0; s < kRsItems; ++s) {
    const int64_t i = base + int64_t(s) * 64;
    const bool valid = i < T;
    key[s] = valid ? keys_in[i] : 0u;
    const uint32_t digit = (key[s] >> shift) & uint32_t(nd - 1);
    uint64_t peers = __ballot(valid);  // the lanes that hold this lane's digit
    for (int b = 0; b < n_bits; ++b) {
      const bool bit = (digit >> b) & 1u;
      const uint64_t m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    const uint32_t c0 = wcnt[w][digit];
    rank[s] = c0 + uint32_t(__popcll(peers & lt));
    if (valid && (peers & lt) == 0) wcnt[w][digit] = c0 + uint32_t(__popcll(peers));  // the group's first lane
  }
  __syncthreads();
  // digit d: the tile's count -> its first place inside the tile and in the output; the waves' counts -> their
  // first places inside the tile
  {
    uint32_t c[kRsWaves], tot = 0;
#pragma unroll
    for (int ww = 0; ww < kRsWaves; ++ww) {
      c[ww] = tid < nd ? wcnt[ww][tid] : 0u;
      tot += c[ww];
    }
    int total;
    const int first = block_excl_scan(int(tot), tmp, &total);
    if (tid < nd) {
      const int64_t e = int64_t(tid) * n_tiles + blockIdx.x;
      dstart[tid] = uint32_t(first);
      gfirst[tid] = hist[e] + chunk_off[e / kRsChunk] - uint32_t(first);
      uint32_t run = uint32_t(first);
#pragma unroll
      for (int ww = 0; ww < kRsWaves; ++ww) {
        wcnt[ww][tid] = run;
        run += c[ww];
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < kRsItems; ++s) {
    const int64_t i = base + int64_t(s) * 64;
    if (i < T) {
      const uint32_t at = wcnt[w][(key[s] >> shift) & uint32_t(nd - 1)] + rank[s];
      sk[at] = key[s];
      sv[at] = vals_in ? vals_in[i] : uint32_t(i);
    }
  }
  __syncthreads();
  const int n_here = int(min<int64_t>(kRsTile, T - tile0));
  for (int j = tid; j < n_here; j += kRsThreads) {
    const uint32_t k = sk[j];
    const uint32_t dest = gfirst[(k >> shift) & uint32_t(nd - 1)] + uint32_t(j);
    keys_out[dest] = k;
    vals_out[dest] = sv[j];
  }
}

RadixPlan radix_plan(int64_t T, int bits) {
  RadixPlan p;
  p.passes = std::max(1, (bits + 7) / 8);
  p.bits_per_pass = (bits + p.passes - 1) / p.passes;
  p.n_tiles = ceil_div(T, kRsTile);
  p.n_counts = p.n_tiles << p.bits_per_pass;
  p.n_chunks = ceil_div(p.n_counts, kRsChunk);
  p.arr = align_up(size_t(T) * sizeof(uint32_t), 256);
  p.off_hist = 4 * p.arr;
  p.off_chunks = p.off_hist + align_up(size_t(p.n_counts) * sizeof(uint32_t), 256);
  p.total = p.off_chunks + align_up(size_t(p.n_chunks) * sizeof(uint32_t), 256) + 256;
  return p;
}


int key_bits(int64_t n_keys) {
  int bits = 1;
  while ((int64_t(1) << bits) < n_keys) ++bits;
  return bits;
}

const uint32_t* radix_sort_positions(void* ws, const RadixPlan& p, int64_t T, int bits, uint32_t* vals_out,
                                     hipStream_t st) {
  char* base = static_cast<char*>(ws);
  uint32_t* ka = reinterpret_cast<uint32_t*>(base);
  uint32_t* va = reinterpret_cast<uint32_t*>(base + p.arr);
  uint32_t* kb = reinterpret_cast<uint32_t*>(base + 2 * p.arr);
  uint32_t* vb = reinterpret_cast<uint32_t*>(base + 3 * p.arr);
  uint32_t* hist = reinterpret_cast<uint32_t*>(base + p.off_hist);
  uint32_t* chunks = reinterpret_cast<uint32_t*>(base + p.off_chunks);
  const uint32_t* kin = ka;
  const uint32_t* vin = nullptr;  // the first pass takes a pair's position as its value
  uint32_t* kout = kb;
  for (int pass = 0; pass < p.passes; ++pass) {
    const int shift = pass * p.bits_per_pass;
    const int n_bits = std::min(p.bits_per_pass, std::max(bits - shift, 1));
    const int nd = 1 << n_bits;
    const bool last = pass + 1 == p.passes;
    uint32_t* vout = last ? vals_out : (kout == kb ? vb : va);
    const int64_t n_counts = p.n_tiles * nd;
    const int64_t n_chunks = ceil_div(n_counts, kRsChunk);
    hipLaunchKernelGGL(radix_hist_kernel, dim3(unsigned(p.n_tiles)), dim3(kRsThreads), 0, st, kin, T, shift, nd,
                       p.n_tiles, hist);
    hipLaunchKernelGGL(radix_scan_kernel, dim3(unsigned(n_chunks)), dim3(1024), 0, st, hist, n_counts, chunks);
    hipLaunchKernelGGL(radix_scan_top_kernel, dim3(1), dim3(1024), 0, st, chunks, n_chunks);
    hipLaunchKernelGGL(radix_scatter_kernel, dim3(unsigned(p.n_tiles)), dim3(kRsThreads), 0, st, kin, vin, kout, vout,
                       T, shift, nd, n_bits, p.n_tiles, hist, chunks);
    kin = kout;
    vin = vout;
    kout = kout == kb ? ka : kb;
  }
  return kin;
}

void launch_sorted_offsets(const uint32_t* sorted_keys, int64_t T, int64_t n_keys, int32_t* off, hipStream_t st) {
  hipLaunchKernelGGL(inv_offsets_kernel, dim3(unsigned(ceil_div(n_keys + 1, int64_t(256)))), dim3(256), 0, st,
                     sorted_keys, T, n_keys, off);
}

void launch_scan_u32(uint32_t* p, int64_t n, hipStream_t st) {
  hipLaunchKernelGGL(radix_scan_top_kernel, dim3(1), dim3(1024), 0, st, p, n);
}

}  // namespace fm
