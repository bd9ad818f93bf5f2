// Launch of the bucket-gathered attention that gives every work item a wave of its own (attn_wave.hpp): four
// items per workgroup of 256 threads, two workgroups per compute unit, no barriers.  The form for long lists
// with few queries each on a memory whose key rows are listed in many buckets.
#include "attn_wave.hpp"

namespace fm {

template <bool F16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void hash_attn_wave_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2, int only_row) {
  extern __shared__ __attribute__((aligned(16))) bf16_t wave_lds[];
  int n_it = *n_items;
  int first = 0;
  if (only_row >= 0) {  // a launch per row: the row's items are [first, n_it)
    first = first_item_of_row(items, n_it, only_row);
    n_it = first_item_of_row(items, n_it, only_row + 1);
  }
  const int w = __builtin_amdgcn_readfirstlane(int(threadIdx.x) >> 6);
  const int me = first + 4 * int(blockIdx.x) + w;
  if (me >= n_it) return;  // (no barrier anywhere: a wave may leave alone)
  const fm_item it = items[me];
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int64_t qbase = int64_t(it.row) * Sq;
  // (an item has up to FM_QTILE = 64 queries, a sweep takes 48: the few items with more are swept twice)
  for (int q0 = 0; q0 < it.n_q; q0 += 48)
    attend_wave<3, F16>(q + qbase * kSD, q_perm + it.q_start + q0, min(it.n_q - q0, 48), k + int64_t(it.row) * N * kSD,
                        v + int64_t(it.row) * N * kSD, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                        out + qbase * kSD, lse + qbase, (lds_char_t*)wave_lds + w * kWWaveBytes);
}

int hash_attn_mfma_wave(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                        const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items,
                        const int32_t* n_items, int64_t max_items, void* out, float* lse, int Sq, int N, int C,
                        float sm_scale, bool f16, int H, bool per_row, hipStream_t st) {
#define FM_WAVE_LAUNCH(F16, ITEMS, ROW)                                                                           \
  do {                                                                                                            \
    FM_ALLOW_LDS((hash_attn_wave_kernel<F16>), kWaveLdsBytes, "fm_hash_attn_fwd: lds");                           \
    hipLaunchKernelGGL((hash_attn_wave_kernel<F16>), dim3(unsigned(ceil_div(int64_t(ITEMS), int64_t(4)))),        \
                       dim3(256), kWaveLdsBytes, st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, \
                       bucket_off, bucket_cnt, q_perm, items, n_items, (bf16_t*)out, lse, Sq, N, C,               \
                       sm_scale * kLog2e, ROW);                                                                   \
  } while (0)
  if (per_row) {
    // One launch per row, in row order, for the reason given in attn_mfma_ring.hip: the waves of a launch start
    // together and sweep the row's K and V at about the same pace.
    const int64_t row_items = std::min<int64_t>(max_items, int64_t(C < Sq ? C : Sq) + Sq / FM_QTILE + 1);
    for (int row = 0; row < H; ++row) {
      if (f16)
        FM_WAVE_LAUNCH(true, row_items, row);
      else
        FM_WAVE_LAUNCH(false, row_items, row);
    }
  } else if (f16) {
    FM_WAVE_LAUNCH(true, max_items, -1);
  } else {
    FM_WAVE_LAUNCH(false, max_items, -1);
  }
#undef FM_WAVE_LAUNCH
  return launch_status("fm_hash_attn_fwd(mfma, wave)");
}

}  // namespace fm
