// Generic (any d <= 256, fp32 or bf16 storage) attention kernels: lane = key
// inside a 64-key chunk; one wave per query for the local attention, the four
// waves of a workgroup sharing a query's chunks for the gathered attention
// (partial softmax states merged through LDS).  They define the numerics of the
// path for fp32 inputs and serve every shape the MFMA kernels do not take.
//
// Arithmetic follows the reference kernel (triton_kernel.py:230-272): scores
// are scaled by sm_scale*log2(e) and the softmax runs in base 2; the
// denominator is summed in fp32 from unrounded p while p is rounded to the
// storage type before P.V; o = acc / l; lse = (m + log2 l) * ln 2.
#include "common.hpp"

namespace fm {

// Online-softmax state of one wave for one query: running maximum (base-2 scores), denominator and
// this lane's slice of the unnormalised output (dimensions l, l+64, l+128, l+192).
struct SoftmaxState {
  float m, lsum, acc[4];
};

// Chunks chunk0, chunk0 + chunk_step, ... of the query's key list.
template <typename T, bool GATHER>
__device__ __forceinline__ SoftmaxState attend_chunks(const T* __restrict__ qrow, const T* __restrict__ Kb,
                                                      const T* __restrict__ Vb, const int32_t* __restrict__ idx,
                                                      int cnt, int N, int d, float scale2, int chunk0,
                                                      int chunk_step) {
  const int l = lane_id();
  float m = -INFINITY, lsum = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int j0 = chunk0 * kWave; j0 < cnt; j0 += chunk_step * kWave) {
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
      int k = 0;
      for (; k + 8 <= d; k += 8) {  // eight loads in flight, then the same ascending fma chain
        float kv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) kv[u] = Elem<T>::load(kr + k + u);
#pragma unroll
        for (int u = 0; u < 8; ++u) dot = fmaf(Elem<T>::load(qrow + k + u), kv[u], dot);
      }
      for (; k < d; ++k) dot = fmaf(Elem<T>::load(qrow + k), Elem<T>::load(kr + k), dot);
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
    int t = 0;
    for (; t + 8 <= nvalid; t += 8) {  // the V rows of eight keys in flight, accumulated in key order
      float vv[8][4];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const T* vr = Vb + int64_t(__shfl(row, t + u)) * d;
#pragma unroll
        for (int r = 0; r < 4; ++r) vv[u][r] = (l + 64 * r < d) ? Elem<T>::load(vr + l + 64 * r) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float pt = __shfl(pr, t + u);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = fmaf(pt, vv[u][r], acc[r]);
      }
    }
    for (; t < nvalid; ++t) {
      const float pt = __shfl(pr, t);
      const int rt = __shfl(row, t);
      const T* vr = Vb + int64_t(rt) * d;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (l + 64 * r < d) acc[r] = fmaf(pt, Elem<T>::load(vr + l + 64 * r), acc[r]);
    }
    m = m_new;
  }
  SoftmaxState st;
  st.m = m;
  st.lsum = lsum;
#pragma unroll
  for (int r = 0; r < 4; ++r) st.acc[r] = acc[r];
  return st;
}

// o = acc / l, lse = (m + log2 l) ln 2; an empty key list gives a zero row and the empty marker.
template <typename T>
__device__ __forceinline__ void write_query(const SoftmaxState& st, int cnt, int d, T* __restrict__ out_row,
                                            float* __restrict__ lse_out) {
  const int l = lane_id();
  const float inv = cnt > 0 ? 1.f / st.lsum : 0.f;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (l + 64 * r < d) Elem<T>::store(out_row + l + 64 * r, st.acc[r] * inv);
  if (l == 0) *lse_out = cnt > 0 ? (st.m + log2f(st.lsum)) * kLn2 : -FLT_MAX;
}

// grid (items, kGenQSplit): workgroup (i, y) takes queries y, y + kGenQSplit, ... of item i, one at a
// time; its four waves take the chunks of the bucket's key list in turn and wave 0 merges their states.
constexpr int kGenQSplit = 16;

template <typename T>
__global__ __launch_bounds__(256) void hash_attn_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items, T* __restrict__ out,
    float* __restrict__ lse, int Sq, int N, int d, int C, float scale2) {
  __shared__ float s_m[4], s_l[4], s_acc[4][FM_MAX_D];
  if (int(blockIdx.x) >= *n_items) return;
  const fm_item it = items[blockIdx.x];
  const int64_t b = int64_t(it.row) * C + it.bucket;
  const int cnt = bucket_cnt[b];
  const int32_t* idx = k_idx + bucket_off[b];
  const T* Kb = k + int64_t(it.row) * N * d;
  const T* Vb = v + int64_t(it.row) * N * d;
  const int w = threadIdx.x >> 6, l = lane_id();
  for (int j = blockIdx.y; j < it.n_q; j += kGenQSplit) {  // uniform over the workgroup
    const int qi = q_perm[it.q_start + j];
    const int64_t qrow = int64_t(it.row) * Sq + qi;
    SoftmaxState st = attend_chunks<T, true>(q + qrow * d, Kb, Vb, idx, cnt, N, d, scale2, w, 4);
    if (l == 0) {
      s_m[w] = st.m;
      s_l[w] = st.lsum;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (l + 64 * r < d) s_acc[w][l + 64 * r] = st.acc[r];
    __syncthreads();
    if (w == 0) {
      SoftmaxState tot;
      tot.m = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
      tot.lsum = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) tot.acc[r] = 0.f;
      for (int ww = 0; ww < 4; ++ww) {
        const float f = s_m[ww] == -INFINITY ? 0.f : exp2f(s_m[ww] - tot.m);  // a wave without chunks adds nothing
        tot.lsum = fmaf(s_l[ww], f, tot.lsum);
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (l + 64 * r < d) tot.acc[r] = fmaf(s_acc[ww][l + 64 * r], f, tot.acc[r]);
      }
      write_query<T>(tot, cnt, d, out + qrow * d, lse + qrow);
    }
    __syncthreads();
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
  const SoftmaxState st = attend_chunks<T, false>(q + qrow * d, k + int64_t(hk) * L * d, v + int64_t(hk) * L * d,
                                                  nullptr, cnt, L, d, scale2, 0, 1);
  write_query<T>(st, cnt, d, out + qrow * d, lse + qrow);
}

int hash_attn_generic(const void* q, const void* k, const void* v, const int32_t* k_idx,
                      const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                      const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                      float* lse, int Sq, int N, int d, int C, float sm_scale, int dtype,
                      hipStream_t st) {
  const float scale2 = sm_scale * kLog2e;
  if (dtype == FM_F32)
    hipLaunchKernelGGL(hash_attn_generic_kernel<float>, dim3(unsigned(max_items), kGenQSplit), dim3(256), 0, st,
                       (const float*)q, (const float*)k, (const float*)v, k_idx, bucket_off,
                       bucket_cnt, q_perm, items, n_items, (float*)out, lse, Sq, N, d, C, scale2);
  else if (dtype == FM_BF16)
    hipLaunchKernelGGL(hash_attn_generic_kernel<bf16_t>, dim3(unsigned(max_items), kGenQSplit), dim3(256), 0,
                       st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, bucket_off,
                       bucket_cnt, q_perm, items, n_items, (bf16_t*)out, lse, Sq, N, d, C, scale2);
  else
    hipLaunchKernelGGL(hash_attn_generic_kernel<f16_t>, dim3(unsigned(max_items), kGenQSplit), dim3(256), 0,
                       st, (const f16_t*)q, (const f16_t*)k, (const f16_t*)v, k_idx, bucket_off,
                       bucket_cnt, q_perm, items, n_items, (f16_t*)out, lse, Sq, N, d, C, scale2);
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
  else if (dtype == FM_BF16)
    hipLaunchKernelGGL(local_attn_generic_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)q,
                       (const bf16_t*)k, (const bf16_t*)v, (bf16_t*)out, lse, G, S, L, d, scale2,
                       causal);
  else
    hipLaunchKernelGGL(local_attn_generic_kernel<f16_t>, grid, dim3(256), 0, st, (const f16_t*)q,
                       (const f16_t*)k, (const f16_t*)v, (f16_t*)out, lse, G, S, L, d, scale2,
                       causal);
  return launch_status("fm_local_attn_fwd(generic)");
}

}  // namespace fm
