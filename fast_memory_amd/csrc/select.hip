// Arg-top-Z over the rows of an fp32 matrix (memory.py:273, triton_kernel.py:278).
//
// Contract: output row r lists the min(Z,N) indices of the largest entries of
// Y[r,:], ordered by (value descending, index ascending); -0 == +0, NaN is the
// largest value.
//
// One workgroup per row: radix select of the Zc-th largest composite (every
// pass re-reads the row and histograms one digit in LDS; the loop stops as soon
// as the bin that holds the cut is wanted whole), one more read collects the
// exactly Zc survivors into LDS, bitonic sort there, indices out.
// HBM traffic: (passes + 1) reads of the row, typically 4; LDS 8*pow2(Zc) + 16 KiB.
#include "select.hpp"

namespace fm {

// row_map / n_rows_dev are optional: when given, workgroup b works on input row
// b and writes output row row_map[b], and exits if b >= min(*n_rows_dev, grid).
__global__ __launch_bounds__(kSelThreads) void argtopz_kernel(
    const float* __restrict__ Y, int N, int64_t ldy, int Zc, int P, int32_t* __restrict__ idx_out,
    float* __restrict__ val_out, const int32_t* __restrict__ row_map, const int32_t* __restrict__ n_rows_dev) {
  extern __shared__ uint64_t buf[];  // P composites
  __shared__ SelectShared sh;
  if (n_rows_dev && int(blockIdx.x) >= *n_rows_dev) return;
  const int64_t out_row = row_map ? row_map[blockIdx.x] : int64_t(blockIdx.x);
  DenseRow src{Y + int64_t(blockIdx.x) * ldy, N};
  const uint64_t cut = radix_select_cut(src, Zc, 6, sh);
  collect_sort_write(src, cut, Zc, P, buf, sh, idx_out + out_row * Zc, val_out ? val_out + out_row * Zc : nullptr);
}

int launch_argtopz(const float* Y, int64_t rows, int N, int64_t ldy, int Zc, int32_t* idx_out, float* val_out,
                   const int32_t* row_map, const int32_t* n_rows_dev, hipStream_t st) {
  const int P = next_pow2(Zc);
  FM_ALLOW_LDS(argtopz_kernel, sort_lds_bytes(FM_MAX_Z), "argtopz: lds");
  hipLaunchKernelGGL(argtopz_kernel, dim3(unsigned(rows)), dim3(kSelThreads),
                     sort_lds_bytes(P), st, Y, N, ldy, Zc, P, idx_out, val_out, row_map, n_rows_dev);
  return launch_status("argtopz");
}

}  // namespace fm

extern "C" size_t fm_argtopz_workspace(int64_t, int, int) { return 0; }

extern "C" int fm_argtopz_f32(const float* Y, int64_t rows, int N, int64_t ldy, int Z,
                              int32_t* idx_out, float* val_out, void* ws, size_t ws_bytes, void* stream) {
  using namespace fm;
  (void)ws;
  (void)ws_bytes;
  FM_REQUIRE(rows >= 0 && N >= 1 && Z >= 1, FM_ERR_ARG, "fm_argtopz_f32: rows=%lld N=%d Z=%d",
             (long long)rows, N, Z);
  FM_REQUIRE(ldy >= N, FM_ERR_ARG, "fm_argtopz_f32: ldy=%lld < N=%d", (long long)ldy, N);
  if (rows == 0) return FM_OK;
  FM_REQUIRE(Y && idx_out, FM_ERR_ARG, "fm_argtopz_f32: null pointer");
  FM_REQUIRE(rows <= 0x7fffffffLL, FM_ERR_UNSUPPORTED, "fm_argtopz_f32: too many rows");
  const int Zc = Z < N ? Z : N;
  FM_REQUIRE(Zc <= FM_MAX_Z, FM_ERR_UNSUPPORTED, "fm_argtopz_f32: min(Z,N)=%d exceeds FM_MAX_Z=%d",
             Zc, FM_MAX_Z);
  return launch_argtopz(Y, rows, N, ldy, Zc, idx_out, val_out, nullptr, nullptr, as_stream(stream));
}
