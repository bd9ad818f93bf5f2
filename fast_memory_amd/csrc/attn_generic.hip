// Generic (any d <= 256, fp32 or bf16 storage) attention kernels: one wave per
// query, lane = key inside a 64-key chunk.  They define the numerics of the
// path for fp32 inputs and serve every shape the MFMA kernels do not take.
//
// Arithmetic follows the reference kernel (triton_kernel.py:230-272): scores
// are scaled by sm_scale*log2(e) and the softmax runs in base 2; the
// denominator is summed in fp32 from unrounded p while p is rounded to the
// storage type before P.V; o = acc / l; lse = (m + log2 l) * ln 2.
#include "common.hpp"

namespace fm {

template <typename T, bool GATHER>
__device__ __forceinline__ void attend_one_query(const T* __restrict__ qrow,
                                                 const T* __restrict__ Kb,
                                                 const T* __restrict__ Vb,
                                                 const int32_t* __restrict__ idx, int cnt, int N,
                                                 int d, float scale2, T* __restrict__ out_row,
                                                 float* __restrict__ lse_out) {
  const int l = lane_id();
  float m = -INFINITY, lsum = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int j0 = 0; j0 < cnt; j0 += kWave) {
    const int kk = j0 + l;
    const bool valid = kk < cnt;
    int row = 0;
    if (valid) {
      row = GATHER ? idx[kk] : kk;
      row = min(max(row, 0), N - 1);
    }
    float s = -INFINITY;
    if (valid) {
      const T* kr = Kb + int64_t(row) * d;
      float dot = 0.f;
      for (int k = 0; k < d; ++k) dot = fmaf(Elem<T>::load(qrow + k), Elem<T>::load(kr + k), dot);
      s = dot * scale2;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? exp2f(s - m_new) : 0.f;
    const float alpha = exp2f(m - m_new);
    lsum = lsum * alpha + wave_sum(p);
    const float pr = Elem<T>::round(p);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] *= alpha;
    const int nvalid = min(kWave, cnt - j0);
    for (int t = 0; t < nvalid; ++t) {
      const float pt = __shfl(pr, t);
      const int rt = __shfl(row, t);
      const T* vr = Vb + int64_t(rt) * d;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (l + 64 * r < d) acc[r] = fmaf(pt, Elem<T>::load(vr + l + 64 * r), acc[r]);
    }
    m = m_new;
  }
  if (cnt <= 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (l + 64 * r < d) Elem<T>::store(out_row + l + 64 * r, 0.f);
    if (l == 0) *lse_out = -FLT_MAX;
  } else {
    const float inv = 1.f / lsum;
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (l + 64 * r < d) Elem<T>::store(out_row + l + 64 * r, acc[r] * inv);
    if (l == 0) *lse_out = (m + log2f(lsum)) * kLn2;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void hash_attn_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items, T* __restrict__ out,
    float* __restrict__ lse, int Sq, int N, int d, int C, float scale2) {
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int64_t b = int64_t(it.row) * C + it.bucket;
  const int cnt = bucket_cnt[b];
  const int32_t* idx = k_idx + bucket_off[b];
  const T* Kb = k + int64_t(it.row) * N * d;
  const T* Vb = v + int64_t(it.row) * N * d;
  for (int j = threadIdx.x >> 6; j < it.n_q; j += 4) {
    const int qi = q_perm[it.q_start + j];
    const int64_t qrow = int64_t(it.row) * Sq + qi;
    attend_one_query<T, true>(q + qrow * d, Kb, Vb, idx, cnt, N, d, scale2, out + qrow * d,
                              lse + qrow);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void local_attn_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, T* __restrict__ out,
    float* __restrict__ lse, int G, int S, int L, int d, float scale2, int causal) {
  const int hq = blockIdx.y;
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= S) return;
  const int hk = hq / G;
  int cnt = L;
  if (causal) cnt = min(L, max(0, i + (L - S) + 1));
  const int64_t qrow = int64_t(hq) * S + i;
  attend_one_query<T, false>(q + qrow * d, k + int64_t(hk) * L * d, v + int64_t(hk) * L * d,
                             nullptr, cnt, L, d, scale2, out + qrow * d, lse + qrow);
}

int hash_attn_generic(const void* q, const void* k, const void* v, const int32_t* k_idx,
                      const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                      const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                      float* lse, int Sq, int N, int d, int C, float sm_scale, int dtype,
                      hipStream_t st) {
  const float scale2 = sm_scale * kLog2e;
  if (dtype == FM_F32)
    hipLaunchKernelGGL(hash_attn_generic_kernel<float>, dim3(unsigned(max_items)), dim3(256), 0, st,
                       (const float*)q, (const float*)k, (const float*)v, k_idx, bucket_off,
                       bucket_cnt, q_perm, items, n_items, (float*)out, lse, Sq, N, d, C, scale2);
  else
    hipLaunchKernelGGL(hash_attn_generic_kernel<bf16_t>, dim3(unsigned(max_items)), dim3(256), 0,
                       st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off,
                       bucket_cnt, q_perm, items, n_items, (bf16_t*)out, lse, Sq, N, d, C, scale2);
  return launch_status("fm_hash_attn_fwd(generic)");
}

int local_attn_generic(const void* q, const void* k, const void* v, void* out, float* lse, int H,
                       int G, int S, int L, int d, float sm_scale, int causal, int dtype,
                       hipStream_t st) {
  const float scale2 = sm_scale * kLog2e;
  dim3 grid = dim3(unsigned(ceil_div(S, 4)), unsigned(H * G));
  if (dtype == FM_F32)
    hipLaunchKernelGGL(local_attn_generic_kernel<float>, grid, dim3(256), 0, st, (const float*)q,
                       (const float*)k, (const float*)v, (float*)out, lse, G, S, L, d, scale2,
                       causal);
  else
    hipLaunchKernelGGL(local_attn_generic_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)q,
                       (const bf16_t*)k, (const bf16_t*)v, (bf16_t*)out, lse, G, S, L, d, scale2,
                       causal);
  return launch_status("fm_local_attn_fwd(generic)");
}

}  // namespace fm
