// Backward of the bucket-gathered attention (memory.py:166-206, which the
// reference evaluates densely over all keys; here only a query's bucket is
// visited).  With P = exp(scale*q.k - lse) on the gathered pairs:
//   dV_j += P_ij dO_i        dP_ij = dO_i . V_j        D_i = dO_i . O_i
//   dS_ij = P_ij (dP_ij - D_i)
//   dQ_i  = scale * sum_j dS_ij K_j        dK_j += scale * dS_ij Q_i
// `out` and `lse` may be those of a larger softmax (the result merged with the
// local attention): the gradients are then the gathered keys' share.
//
// Generic kernel: one wave per query, lane = key inside a 64-key chunk, any
// d <= 256, fp32 or bf16 storage, fp32 arithmetic.  dQ is owned by the wave; dK
// and dV rows collect contributions from every bucket a key belongs to and are
// accumulated in fp32 with atomic adds (their order, hence the last bits of dK
// and dV, depends on scheduling).
#include "common.hpp"

namespace fm {

template <typename T>
__device__ __forceinline__ void backward_one_query(const T* __restrict__ qrow, const T* __restrict__ orow,
                                                   const T* __restrict__ dorow, float lse, float dlse,
                                                   const T* __restrict__ Kb, const T* __restrict__ Vb,
                                                   const int32_t* __restrict__ idx, int cnt, int N, int d,
                                                   float sm_scale, T* __restrict__ dq_row,
                                                   float* __restrict__ dKb, float* __restrict__ dVb) {
  const int l = lane_id();
  // this lane's slice of the query-side rows: dimensions l, l+64, l+128, l+192
  float qv[4], dov[4], dq[4] = {0.f, 0.f, 0.f, 0.f};
  float dpart = 0.f;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int k = l + 64 * r;
    qv[r] = k < d ? Elem<T>::load(qrow + k) : 0.f;
    dov[r] = k < d ? Elem<T>::load(dorow + k) : 0.f;
    dpart += k < d ? dov[r] * Elem<T>::load(orow + k) : 0.f;
  }
  const float D = wave_sum(dpart) - dlse;  // dS = P (dP - D) + P dlse
  const float lse2 = lse * kLog2e;
  const float scale2 = sm_scale * kLog2e;
  for (int j0 = 0; j0 < cnt; j0 += kWave) {
    const int kk = j0 + l;
    const bool valid = kk < cnt;
    int row = 0;
    if (valid) row = min(max(idx[kk], 0), N - 1);
    float p = 0.f, ds = 0.f;
    if (valid) {
      const T* kr = Kb + int64_t(row) * d;
      const T* vr = Vb + int64_t(row) * d;
      float dot = 0.f, dp = 0.f;
      for (int k = 0; k < d; ++k) {
        dot = fmaf(Elem<T>::load(qrow + k), Elem<T>::load(kr + k), dot);
        dp = fmaf(Elem<T>::load(dorow + k), Elem<T>::load(vr + k), dp);
      }
      p = exp2f(dot * scale2 - lse2);
      ds = p * (dp - D);
    }
    const int nvalid = min(kWave, cnt - j0);
    for (int t = 0; t < nvalid; ++t) {
      const float pt = __shfl(p, t);
      const float dst = __shfl(ds, t) * sm_scale;
      const int rt = __shfl(row, t);
      const T* kr = Kb + int64_t(rt) * d;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int k = l + 64 * r;
        if (k < d) {
          dq[r] = fmaf(dst, Elem<T>::load(kr + k), dq[r]);
          unsafeAtomicAdd(dKb + int64_t(rt) * d + k, dst * qv[r]);
          unsafeAtomicAdd(dVb + int64_t(rt) * d + k, pt * dov[r]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (l + 64 * r < d) Elem<T>::store(dq_row + l + 64 * r, dq[r]);
}

template <typename T>
__global__ __launch_bounds__(256) void hash_attn_bwd_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const int32_t* __restrict__ k_idx,
    const int64_t* __restrict__ bucket_off, const int32_t* __restrict__ bucket_cnt,
    const int32_t* __restrict__ q_perm, const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    const T* __restrict__ out, const float* __restrict__ lse, const T* __restrict__ dout,
    const float* __restrict__ dlse, T* __restrict__ dq, float* __restrict__ dk, float* __restrict__ dv, int Sq, int N, int d, int C, float sm_scale) {
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int64_t b = int64_t(it.row) * C + it.bucket;
  const int cnt = bucket_cnt[b];
  const int32_t* idx = k_idx + bucket_off[b];
  const int64_t kv = int64_t(it.row) * N * d;
  for (int j = threadIdx.x >> 6; j < it.n_q; j += 4) {
    const int qi = q_perm[it.q_start + j];
    const int64_t qrow = int64_t(it.row) * Sq + qi;
    backward_one_query<T>(q + qrow * d, out + qrow * d, dout + qrow * d, lse[qrow], dlse ? dlse[qrow] : 0.f, k + kv, v + kv, idx, cnt, N, d,
                          sm_scale, dq + qrow * d, dk + kv, dv + kv);
  }
}

extern std::atomic<int> g_force_generic;
bool hash_attn_bwd_mfma_supported(int d, int dtype);
int hash_attn_bwd_mfma(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                       const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                       int64_t max_items, const void* out, const float* lse, const void* dout, const float* dlse, void* dq,
                       float* dk, float* dv, int Sq, int N, int C, float sm_scale, bool f16, hipStream_t st);

int launch_unlisted_rows(const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                         const int32_t* bin_off, const int32_t* bin_count, int64_t n_bins, int64_t nq,
                         int row_bytes, void* rows, float* lse, hipStream_t st);  // group.hip

}  // namespace fm

extern "C" int fm_hash_attn_bwd(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                                const fm_item* items, const int32_t* n_items, int64_t max_items, const void* out,
                                const float* lse, const void* dout, const float* dlse, void* dq, float* dk, float* dv,
                                int H, int Sq, int N, int d, int C, float sm_scale, int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && Sq >= 1 && N >= 1 && C >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG,
             "fm_hash_attn_bwd: H=%d Sq=%d N=%d C=%d d=%d", H, Sq, N, C, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_hash_attn_bwd: dtype=%d", dtype);
  FM_REQUIRE(q && k && v && k_idx && bucket_off && bucket_cnt && q_perm && items && n_items && out && lse && dout &&
                 dq && dk && dv,
             FM_ERR_ARG, "fm_hash_attn_bwd: null pointer");
  FM_REQUIRE(max_items >= 1 && max_items <= 0x7fffffffLL, FM_ERR_ARG, "fm_hash_attn_bwd: max_items=%lld",
             (long long)max_items);
  hipStream_t st = as_stream(stream);
  // dq of the queries that are part of no work item (hash outside [0, C)): 0, as for an empty bucket
  int rc = launch_unlisted_rows(q_perm, items, n_items, nullptr, nullptr, 0, int64_t(H) * Sq, d * dtype_bytes(dtype),
                                dq, nullptr, st);
  if (rc) return rc;
  if (g_force_generic != 1 && hash_attn_bwd_mfma_supported(d, dtype))
    return hash_attn_bwd_mfma(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items, out, lse,
                              dout, dlse, dq, dk, dv, Sq, N, C, sm_scale, dtype == FM_F16, st);
  if (dtype == FM_F32)
    hipLaunchKernelGGL(hash_attn_bwd_generic_kernel<float>, dim3(unsigned(max_items)), dim3(256), 0, st,
                       (const float*)q, (const float*)k, (const float*)v, k_idx, bucket_off, bucket_cnt, q_perm, items,
                       n_items, (const float*)out, lse, (const float*)dout, dlse, (float*)dq, dk, dv, Sq, N, d, C, sm_scale);
  else if (dtype == FM_BF16)
    hipLaunchKernelGGL(hash_attn_bwd_generic_kernel<bf16_t>, dim3(unsigned(max_items)), dim3(256), 0, st,
                       (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm,
                       items, n_items, (const bf16_t*)out, lse, (const bf16_t*)dout, dlse, (bf16_t*)dq, dk, dv, Sq, N, d, C,
                       sm_scale);
  else
    hipLaunchKernelGGL(hash_attn_bwd_generic_kernel<f16_t>, dim3(unsigned(max_items)), dim3(256), 0, st,
                       (const f16_t*)q, (const f16_t*)k, (const f16_t*)v, k_idx, bucket_off, bucket_cnt, q_perm,
                       items, n_items, (const f16_t*)out, lse, (const f16_t*)dout, dlse, (f16_t*)dq, dk, dv, Sq, N, d, C,
                       sm_scale);
  return launch_status("fm_hash_attn_bwd");
}
