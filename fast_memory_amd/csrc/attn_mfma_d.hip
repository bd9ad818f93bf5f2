// Grouped launch of the staged bucket-gathered attention for the head dimensions beside 128 that the MFMA
// path takes (attn_staged_d.hpp): one workgroup per work item.
#include "attn_staged_d.hpp"

namespace fm {

// (D = 256 is held to 256 registers, so that two workgroups share a compute unit)
template <int D, bool F16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 256 ? 2 : 1))) void hash_attn_staged_d_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2) {
  extern __shared__ __attribute__((aligned(16))) bf16_t std_lds[];
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int64_t qbase = int64_t(it.row) * Sq;
  attend_staged_d<D, F16>(q + qbase * D, q_perm + it.q_start, it.n_q, k + int64_t(it.row) * N * D,
                          v + int64_t(it.row) * N * D, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                          out + qbase * D, lse + qbase, std_lds);
}

bool hash_attn_mfma_d_supported(int d, int N) {
  return (d == 64 || d == 256) && int64_t(N) * 2 * d < (int64_t(1) << 32);
}

int hash_attn_mfma_d(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                     const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                     int64_t max_items, void* out, float* lse, int Sq, int N, int d, int C, float sm_scale, bool f16,
                     hipStream_t st) {
#define FM_STAGED_D(D, F16)                                                                                       \
  do {                                                                                                            \
    FM_ALLOW_LDS((hash_attn_staged_d_kernel<D, F16>), StagedD<D>::kLdsBytes, "fm_hash_attn_fwd: lds");            \
    hipLaunchKernelGGL((hash_attn_staged_d_kernel<D, F16>), dim3(unsigned(max_items)), dim3(256),                 \
                       StagedD<D>::kLdsBytes, st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx,    \
                       bucket_off, bucket_cnt, q_perm, items, n_items, (bf16_t*)out, lse, Sq, N, C,               \
                       sm_scale * kLog2e);                                                                        \
  } while (0)
  if (d == 64 && f16)
    FM_STAGED_D(64, true);
  else if (d == 64)
    FM_STAGED_D(64, false);
  else if (d == 256 && f16)
    FM_STAGED_D(256, true);
  else if (d == 256)
    FM_STAGED_D(256, false);
  else if (d == 128 && f16)  // the 128-wide instantiation: tests compare it with the kernels built for 128
    FM_STAGED_D(128, true);
  else
    FM_STAGED_D(128, false);
#undef FM_STAGED_D
  return launch_status("fm_hash_attn_fwd(mfma, any head dimension)");
}

}  // namespace fm
