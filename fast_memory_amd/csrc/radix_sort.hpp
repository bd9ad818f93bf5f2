// Stable least-significant-digit radix sort of (key, position) pairs on 32-bit keys, and the offsets of the
// keys in the sorted sequence.  Used where the library needs a sort: the inverse index of bucket lists in
// arbitrary order and the grouping of long query / key rows by bucket.
#pragma once
#include "common.hpp"

namespace fm {

struct RadixPlan {
  int passes, bits_per_pass;
  int64_t n_tiles, n_counts, n_chunks;
  size_t arr, off_hist, off_chunks, total;  // four arrays of T words, then the counts
};
RadixPlan radix_plan(int64_t T, int bits);

// bits needed for keys 0 .. n_keys - 1
int key_bits(int64_t n_keys);

// Sorts the T keys at the start of ws (T words, written by the caller; ws of radix_plan(T, bits).total
// bytes) by their low `bits` bits, stably; a key's value is its position 0 .. T-1 before the sort.
// The sorted values go to vals_out [T]; returns where the sorted keys are (inside ws).
const uint32_t* radix_sort_positions(void* ws, const RadixPlan& p, int64_t T, int bits, uint32_t* vals_out,
                                     hipStream_t st);

// off[kk] = first place of sorted_keys [T] whose key is >= kk, for kk = 0 .. n_keys (n_keys + 1 outputs)
void launch_sorted_offsets(const uint32_t* sorted_keys, int64_t T, int64_t n_keys, int32_t* off, hipStream_t st);

// exclusive prefix sum of n words in place, by one workgroup
void launch_scan_u32(uint32_t* p, int64_t n, hipStream_t st);

}  // namespace fm
