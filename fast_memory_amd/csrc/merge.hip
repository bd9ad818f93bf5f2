// LSE merge of two partial attentions, in place on the running pair
// (update_out_and_lse, memory.py:54-71).
//
// The reference writes  out -= sigmoid(D)*(out - b_out);  lse -= logsigmoid(-D)
// with D = b_lse - lse, which is  lse' = logaddexp(lse, b_lse)  and a convex
// combination with weights exp(lse - lse'), exp(b_lse - lse').  The kernel
// evaluates that closed form around max(lse, b_lse), which has the same value
// wherever the reference's form is accurate and stays accurate where one side
// is the empty-bucket marker -FLT_MAX.
#include "common.hpp"

namespace fm {

template <typename T>
__global__ __launch_bounds__(256) void lse_merge_kernel(float* __restrict__ out,
                                                        float* __restrict__ lse,
                                                        const T* __restrict__ b_out,
                                                        const float* __restrict__ b_lse, int64_t Q,
                                                        int d) {
  const int64_t qi = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (qi >= Q) return;
  const float la = lse[qi], lb = b_lse[qi];
  const float mx = fmaxf(la, lb);
  const float ea = expf(la - mx), eb = expf(lb - mx);  // one of them is 1
  const float den = ea + eb;
  const float wb = eb / den;
  float* o = out + qi * d;
  const T* bo = b_out + qi * d;
  for (int k = lane_id(); k < d; k += kWave) {
    float a = o[k];
    float b = Elem<T>::load(bo + k);
    o[k] = a - wb * (a - b);
  }
  if (lane_id() == 0) lse[qi] = mx + logf(den);
}

}  // namespace fm

extern "C" int fm_lse_merge(float* out, float* lse, const void* block_out, const float* block_lse,
                            int64_t Q, int d, int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(Q >= 0 && d >= 1, FM_ERR_ARG, "fm_lse_merge: Q=%lld d=%d", (long long)Q, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_lse_merge: dtype=%d", dtype);
  if (Q == 0) return FM_OK;
  FM_REQUIRE(out && lse && block_out && block_lse, FM_ERR_ARG, "fm_lse_merge: null pointer");
  FM_REQUIRE(ceil_div(Q, 4) <= 0x7fffffffLL, FM_ERR_UNSUPPORTED, "fm_lse_merge: Q too large");
  dim3 grid = dim3(unsigned(ceil_div(Q, 4)));
  if (dtype == FM_F32)
    hipLaunchKernelGGL(lse_merge_kernel<float>, grid, dim3(256), 0, as_stream(stream), out, lse,
                       (const float*)block_out, block_lse, Q, d);
  else if (dtype == FM_BF16)
    hipLaunchKernelGGL(lse_merge_kernel<bf16_t>, grid, dim3(256), 0, as_stream(stream), out, lse,
                       (const bf16_t*)block_out, block_lse, Q, d);
  else
    hipLaunchKernelGGL(lse_merge_kernel<f16_t>, grid, dim3(256), 0, as_stream(stream), out, lse,
                       (const f16_t*)block_out, block_lse, Q, d);
  return launch_status("fm_lse_merge");
}
