// Construction of the projection matrix A: row normalisation and the
// top-k-mean step of compute_centroids (memory.py:209-231, 256-258), and the
// centroid update of spherical K-means (README.md:37-45).  Sums run in a fixed
// order (member order of the index lists), so results do not depend on
// scheduling.
#include "common.hpp"

namespace fm {

__device__ __forceinline__ float block_sum_256(float v, float* sh) {
  v = wave_sum(v);
  if (lane_id() == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = sh[0] + sh[1] + sh[2] + sh[3];
  __syncthreads();
  return r;
}

// rows / max(||row||, eps); one wave per row
template <typename T>
__global__ __launch_bounds__(256) void l2_normalize_kernel(const T* __restrict__ X,
                                                           T* __restrict__ Xn, int64_t rows, int d,
                                                           float eps) {
  const int64_t r = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const T* x = X + r * d;
  float ss = 0.f;
  for (int k = lane_id(); k < d; k += kWave) {
    float v = Elem<T>::load(x + k);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.f / fmaxf(sqrtf(ss), eps);
  for (int k = lane_id(); k < d; k += kWave) Elem<T>::store(Xn + r * d + k, Elem<T>::load(x + k) * inv);
}

// bf16, d = 128: a row is 16 lanes x 16 bytes, four rows per wave and load instruction, four such
// loads in flight per thread.  HBM-bound: 2*d*2 bytes per row.
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 cbf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float cf32x2;
__device__ __forceinline__ uint32_t cent_pack_bf16(float lo, float hi) {
  cf32x2 x = {lo, hi};
  cbf16x2 y = __builtin_convertvector(x, cbf16x2);  // round to nearest even
  return *reinterpret_cast<uint32_t*>(&y);
}
__device__ __forceinline__ void cent_unpack8(uint4 u, float (&f)[8]) {
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

__global__ __launch_bounds__(256) void l2_normalize_bf16_d128_kernel(const bf16_t* __restrict__ X,
                                                                     bf16_t* __restrict__ Xn, int64_t rows,
                                                                     float eps) {
  constexpr int U = 4;
  const int c = threadIdx.x & 15;
  const int64_t stride = int64_t(gridDim.x) * 16;
  for (int64_t r0 = int64_t(blockIdx.x) * 16 + (threadIdx.x >> 4); r0 < rows; r0 += stride * U) {
    uint4 u[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t r = r0 + k * stride;
      u[k] = r < rows ? reinterpret_cast<const uint4*>(X + r * 128)[c] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t r = r0 + k * stride;
      float f[8];
      cent_unpack8(u[k], f);
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) ss += __shfl_xor(ss, o);
      const float inv = 1.f / fmaxf(sqrtf(ss), eps);
      if (r < rows)
        reinterpret_cast<uint4*>(Xn + r * 128)[c] =
            make_uint4(cent_pack_bf16(f[0] * inv, f[1] * inv), cent_pack_bf16(f[2] * inv, f[3] * inv),
                       cent_pack_bf16(f[4] * inv, f[5] * inv), cent_pack_bf16(f[6] * inv, f[7] * inv));
    }
  }
}

// A[c,h,:] = normalise( mean over g<G, j<k of Xn[h*G+g, top_idx[c,h*G+g,j], :] )
// one workgroup per (c,h); thread = dimension (d <= 256)
template <typename T>
__global__ __launch_bounds__(256) void topk_mean_kernel(const T* __restrict__ Xn,
                                                        const int32_t* __restrict__ top_idx,
                                                        T* __restrict__ A_out, int H, int G, int N,
                                                        int k, int d, int normalize) {
  __shared__ float sh[4];
  const int c = blockIdx.x, h = blockIdx.y, t = threadIdx.x;
  float acc = 0.f;
  for (int g = 0; g < G; ++g) {
    const int hg = h * G + g;
    const int32_t* ti = top_idx + (int64_t(c) * H * G + hg) * k;
    const T* xb = Xn + int64_t(hg) * N * d;
    for (int j = 0; j < k; ++j) {
      int row = min(max(ti[j], 0), N - 1);
      if (t < d) acc += Elem<T>::load(xb + int64_t(row) * d + t);
    }
  }
  acc /= float(G * k);
  if (normalize) {
    float ss = block_sum_256(t < d ? acc * acc : 0.f, sh);
    acc /= sqrtf(ss);
  }
  if (t < d) Elem<T>::store(A_out + (int64_t(c) * H + h) * d + t, acc);
}

// cent[h,c,:] = normalise( mean of X[h, perm[...], :] over the cluster's members )
// members = perm[seg_off[h,c] .. +seg_cnt[h,c]) (positions over the flattened
// [H*N] sorted axis, values are row indices inside head h); empty -> prev.
// NORM: the rows of X are taken as they are stored and every member contributes row / max(||row||, eps)
// (the mean of the members' directions; nothing normalised is kept in memory).
template <typename T, bool NORM>
__global__ __launch_bounds__(256) void segment_mean_kernel(
    const T* __restrict__ X, const int32_t* __restrict__ perm, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_cnt, const T* __restrict__ prev, T* __restrict__ out, int C,
    int N, int d, float eps) {
  __shared__ float sh[4];
  const int c = blockIdx.x, h = blockIdx.y, t = threadIdx.x;
  const int64_t hc = int64_t(h) * C + c;
  const int cnt = seg_cnt[hc];
  const int32_t* mem = perm + seg_off[hc];
  const T* xb = X + int64_t(h) * N * d;
  float acc = 0.f;
  for (int j = 0; j < cnt; ++j) {
    int row = min(max(mem[j], 0), N - 1);
    float x = t < d ? Elem<T>::load(xb + int64_t(row) * d + t) : 0.f;
    if constexpr (NORM) x *= 1.f / fmaxf(sqrtf(block_sum_256(x * x, sh)), eps);
    acc += x;
  }
  if (cnt > 0) acc /= float(cnt);
  float ss = block_sum_256(t < d ? acc * acc : 0.f, sh);
  float nrm = sqrtf(ss);
  if (t < d) {
    if (cnt == 0 || nrm < 1e-12f)
      out[hc * d + t] = prev[hc * d + t];
    else
      Elem<T>::store(out + hc * d + t, acc / nrm);
  }
}


// bf16, d = 128: sixteen groups of 16 lanes walk the member list in turn (member j goes to group
// j % 16), each lane adding its 8 dimensions of the gathered rows, four rows in flight per group;
// the sixteen partial sums are then added in group order, so the result does not depend on
// scheduling.  HBM-bound on the gathered rows (256 bytes per member).
// NORM as in segment_mean_kernel: a row's squared norm is summed inside its group of 16 lanes.
// F16: the rows are fp16 (else bf16); bf16_t and f16_t are both 16-bit words here.
template <bool NORM, bool F16 = false>
__global__ __launch_bounds__(256) void segment_mean_bf16_d128_kernel(
    const bf16_t* __restrict__ X, const int32_t* __restrict__ perm, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_cnt, const bf16_t* __restrict__ prev, bf16_t* __restrict__ out, int C,
    int N, float eps) {
  __shared__ float red[16][128];
  __shared__ float sh[4];
  const int c = blockIdx.x, h = blockIdx.y, t = threadIdx.x;
  const int g = t >> 4, ch = t & 15;
  const int64_t hc = int64_t(h) * C + c;
  const int cnt = seg_cnt[hc];
  const int32_t* mem = perm + seg_off[hc];
  const uint4* xb = reinterpret_cast<const uint4*>(X + int64_t(h) * N * 128);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  constexpr int U = 4;
  for (int j0 = g; j0 < cnt; j0 += 16 * U) {
    uint4 u[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int j = j0 + 16 * k;
      const int row = j < cnt ? min(max(mem[j], 0), N - 1) : 0;
      u[k] = j < cnt ? xb[int64_t(row) * 16 + ch] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      float f[8];
      if constexpr (F16) {
        const uint32_t w4[4] = {u[k].x, u[k].y, u[k].z, u[k].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          f[2 * i] = float(__builtin_bit_cast(_Float16, uint16_t(w4[i] & 0xffffu)));
          f[2 * i + 1] = float(__builtin_bit_cast(_Float16, uint16_t(w4[i] >> 16)));
        }
      } else {
        cent_unpack8(u[k], f);
      }
      if constexpr (NORM) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) ss += __shfl_xor(ss, o);
        const float inv = 1.f / fmaxf(sqrtf(ss), eps);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(f[i], inv, acc[i]);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += f[i];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) red[g][ch * 8 + i] = acc[i];
  __syncthreads();
  float v = 0.f;
  if (t < 128) {
#pragma unroll
    for (int gg = 0; gg < 16; ++gg) v += red[gg][t];
    if (cnt > 0) v /= float(cnt);
  }
  const float ss = block_sum_256(t < 128 ? v * v : 0.f, sh);
  const float nrm = sqrtf(ss);
  if (t < 128) {
    if (cnt == 0 || nrm < 1e-12f)
      out[hc * 128 + t] = prev[hc * 128 + t];
    else
      out[hc * 128 + t] = F16 ? bf16_t(__builtin_bit_cast(uint16_t, _Float16(v / nrm))) : f32_to_bf16(v / nrm);
  }
}


// out[h,c,:] = sum of X[h, perm[...], :] over the segment's members, fp32, member order; empty -> 0.
// One workgroup per (c, h); 16 groups of 16 lanes when a row is 16 chunks of 8 elements (bf16, d = 128),
// else thread = dimension.
template <typename T>
__global__ __launch_bounds__(256) void segment_sum_kernel(const T* __restrict__ X, const int32_t* __restrict__ perm,
                                                          const int32_t* __restrict__ seg_off,
                                                          const int32_t* __restrict__ seg_cnt,
                                                          float* __restrict__ out, int C, int N, int d) {
  const int c = blockIdx.x, h = blockIdx.y, t = threadIdx.x;
  const int64_t hc = int64_t(h) * C + c;
  const int cnt = seg_cnt[hc];
  const int32_t* mem = perm + seg_off[hc];
  const T* xb = X + int64_t(h) * N * d;
  float acc = 0.f;
  for (int j = 0; j < cnt; ++j) {
    const int row = min(max(mem[j], 0), N - 1);
    if (t < d) acc += Elem<T>::load(xb + int64_t(row) * d + t);
  }
  if (t < d) out[hc * d + t] = acc;
}

}  // namespace fm

extern "C" int fm_segment_sum(const void* X, const int32_t* perm, const int32_t* seg_off, const int32_t* seg_cnt,
                              float* sum_out, int H, int C, int N, int d, int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && C >= 1 && N >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG, "fm_segment_sum: H=%d C=%d N=%d d=%d",
             H, C, N, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_segment_sum: dtype=%d", dtype);
  FM_REQUIRE(X && perm && seg_off && seg_cnt && sum_out, FM_ERR_ARG, "fm_segment_sum: null pointer");
  FM_REQUIRE(H <= 65535, FM_ERR_UNSUPPORTED, "fm_segment_sum: H > 65535");
  dim3 grid = dim3(unsigned(C), unsigned(H));
  if (dtype == FM_F32)
    hipLaunchKernelGGL(segment_sum_kernel<float>, grid, dim3(256), 0, as_stream(stream), (const float*)X, perm,
                       seg_off, seg_cnt, sum_out, C, N, d);
  else if (dtype == FM_BF16)
    hipLaunchKernelGGL(segment_sum_kernel<bf16_t>, grid, dim3(256), 0, as_stream(stream), (const bf16_t*)X, perm,
                       seg_off, seg_cnt, sum_out, C, N, d);
  else
    hipLaunchKernelGGL(segment_sum_kernel<f16_t>, grid, dim3(256), 0, as_stream(stream), (const f16_t*)X, perm,
                       seg_off, seg_cnt, sum_out, C, N, d);
  return launch_status("fm_segment_sum");
}

extern "C" int fm_l2_normalize(const void* X, void* Xn, int64_t rows, int d, float eps, int dtype,
                               void* stream) {
  using namespace fm;
  FM_REQUIRE(rows >= 0 && d >= 1, FM_ERR_ARG, "fm_l2_normalize: rows=%lld d=%d", (long long)rows, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_l2_normalize: dtype=%d", dtype);
  if (rows == 0) return FM_OK;
  FM_REQUIRE(X && Xn, FM_ERR_ARG, "fm_l2_normalize: null pointer");
  FM_REQUIRE(ceil_div(rows, 4) <= 0x7fffffffLL, FM_ERR_UNSUPPORTED, "fm_l2_normalize: too many rows");
  dim3 grid = dim3(unsigned(ceil_div(rows, 4)));
  if (dtype == FM_BF16 && d == 128) {
    const unsigned wgs = unsigned(std::min<int64_t>(ceil_div(rows, 16 * 4), 256 * 64));
    hipLaunchKernelGGL(l2_normalize_bf16_d128_kernel, dim3(wgs), dim3(256), 0, as_stream(stream),
                       (const bf16_t*)X, (bf16_t*)Xn, rows, eps);
  } else if (dtype == FM_F32)
    hipLaunchKernelGGL(l2_normalize_kernel<float>, grid, dim3(256), 0, as_stream(stream),
                       (const float*)X, (float*)Xn, rows, d, eps);
  else if (dtype == FM_BF16)
    hipLaunchKernelGGL(l2_normalize_kernel<bf16_t>, grid, dim3(256), 0, as_stream(stream),
                       (const bf16_t*)X, (bf16_t*)Xn, rows, d, eps);
  else
    hipLaunchKernelGGL(l2_normalize_kernel<f16_t>, grid, dim3(256), 0, as_stream(stream),
                       (const f16_t*)X, (f16_t*)Xn, rows, d, eps);
  return launch_status("fm_l2_normalize");
}

extern "C" int fm_topk_mean(const void* Xn, const int32_t* top_idx, void* A_out, int C, int H, int G,
                            int N, int k, int d, int normalize, int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(C >= 1 && H >= 1 && G >= 1 && N >= 1 && k >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG,
             "fm_topk_mean: C=%d H=%d G=%d N=%d k=%d d=%d", C, H, G, N, k, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_topk_mean: dtype=%d", dtype);
  FM_REQUIRE(Xn && top_idx && A_out, FM_ERR_ARG, "fm_topk_mean: null pointer");
  FM_REQUIRE(H <= 65535, FM_ERR_UNSUPPORTED, "fm_topk_mean: H > 65535");
  dim3 grid = dim3(unsigned(C), unsigned(H));
  if (dtype == FM_F32)
    hipLaunchKernelGGL(topk_mean_kernel<float>, grid, dim3(256), 0, as_stream(stream),
                       (const float*)Xn, top_idx, (float*)A_out, H, G, N, k, d, normalize);
  else if (dtype == FM_BF16)
    hipLaunchKernelGGL(topk_mean_kernel<bf16_t>, grid, dim3(256), 0, as_stream(stream),
                       (const bf16_t*)Xn, top_idx, (bf16_t*)A_out, H, G, N, k, d, normalize);
  else
    hipLaunchKernelGGL(topk_mean_kernel<f16_t>, grid, dim3(256), 0, as_stream(stream),
                       (const f16_t*)Xn, top_idx, (f16_t*)A_out, H, G, N, k, d, normalize);
  return launch_status("fm_topk_mean");
}

namespace fm {
static int segment_mean_any(const char* name, bool norm, const void* X, const int32_t* perm, const int32_t* seg_off,
                            const int32_t* seg_cnt, const void* prev, void* cent_out, int H, int C, int N, int d,
                            float eps, int dtype, void* stream) {
  FM_REQUIRE(H >= 1 && C >= 1 && N >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG, "%s: H=%d C=%d N=%d d=%d", name, H, C,
             N, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "%s: dtype=%d", name, dtype);
  FM_REQUIRE(X && perm && seg_off && seg_cnt && prev && cent_out, FM_ERR_ARG, "%s: null pointer", name);
  FM_REQUIRE(H <= 65535, FM_ERR_UNSUPPORTED, "%s: H > 65535", name);
  dim3 grid = dim3(unsigned(C), unsigned(H));
  hipStream_t st = as_stream(stream);
#define FM_SEGMEAN(T, NORM)                                                                                    \
  hipLaunchKernelGGL((segment_mean_kernel<T, NORM>), grid, dim3(256), 0, st, (const T*)X, perm, seg_off, seg_cnt, \
                     (const T*)prev, (T*)cent_out, C, N, d, eps)
  if (dtype == FM_BF16 && d == 128) {
    if (norm)
      hipLaunchKernelGGL(segment_mean_bf16_d128_kernel<true>, grid, dim3(256), 0, st, (const bf16_t*)X, perm, seg_off,
                         seg_cnt, (const bf16_t*)prev, (bf16_t*)cent_out, C, N, eps);
    else
      hipLaunchKernelGGL(segment_mean_bf16_d128_kernel<false>, grid, dim3(256), 0, st, (const bf16_t*)X, perm, seg_off,
                         seg_cnt, (const bf16_t*)prev, (bf16_t*)cent_out, C, N, eps);
  } else if (dtype == FM_F16 && d == 128) {
    if (norm)
      hipLaunchKernelGGL((segment_mean_bf16_d128_kernel<true, true>), grid, dim3(256), 0, st, (const bf16_t*)X, perm,
                         seg_off, seg_cnt, (const bf16_t*)prev, (bf16_t*)cent_out, C, N, eps);
    else
      hipLaunchKernelGGL((segment_mean_bf16_d128_kernel<false, true>), grid, dim3(256), 0, st, (const bf16_t*)X, perm,
                         seg_off, seg_cnt, (const bf16_t*)prev, (bf16_t*)cent_out, C, N, eps);
  } else if (dtype == FM_F32) {
    if (norm) FM_SEGMEAN(float, true); else FM_SEGMEAN(float, false);
  } else if (dtype == FM_BF16) {
    if (norm) FM_SEGMEAN(bf16_t, true); else FM_SEGMEAN(bf16_t, false);
  } else {
    if (norm) FM_SEGMEAN(f16_t, true); else FM_SEGMEAN(f16_t, false);
  }
#undef FM_SEGMEAN
  return launch_status(name);
}
}  // namespace fm

extern "C" int fm_segment_mean(const void* X, const int32_t* perm, const int32_t* seg_off,
                               const int32_t* seg_cnt, const void* prev, void* cent_out, int H,
                               int C, int N, int d, int dtype, void* stream) {
  return fm::segment_mean_any("fm_segment_mean", false, X, perm, seg_off, seg_cnt, prev, cent_out, H, C, N, d, 0.f,
                              dtype, stream);
}

extern "C" int fm_segment_mean_directions(const void* X, const int32_t* perm, const int32_t* seg_off,
                                          const int32_t* seg_cnt, const void* prev, void* cent_out, int H,
                                          int C, int N, int d, float eps, int dtype, void* stream) {
  return fm::segment_mean_any("fm_segment_mean_directions", true, X, perm, seg_off, seg_cnt, prev, cent_out, H, C, N,
                              d, eps, dtype, stream);
}
