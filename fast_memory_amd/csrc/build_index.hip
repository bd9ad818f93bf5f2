// Index build on one device (memory.py:260-278 without the collectives):
// projection rows are produced into the caller's workspace in passes of as
// many (head, bucket) rows as fit (whole heads when several fit) and handed to
// the selection kernel.
#include "common.hpp"

extern "C" size_t fm_build_index_workspace(int H, int C, int N, int d, int Z,
                                           int64_t rows_per_pass) {
  (void)d;
  if (H < 1 || C < 1 || N < 1) return 0;
  int64_t rows = rows_per_pass < 1 ? 1 : rows_per_pass;
  if (rows > int64_t(H) * C) rows = int64_t(H) * C;
  int64_t ldy = (int64_t(N) + 3) / 4 * 4;
  // lists longer than FM_MAX_Z are sorted in memory: that scratch sits in front of the projection rows
  return fm::align_up(fm_argtopz_workspace(int64_t(H) * C, N, Z), 256) + size_t(rows) * size_t(ldy) * sizeof(float);
}

extern "C" int fm_build_index(const void* A, const void* K, int32_t* idx_out, float* val_out, int H, int C,
                              int N, int d, int Z, int dtype, void* ws, size_t ws_bytes, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && C >= 1 && N >= 1 && d >= 1 && Z >= 1, FM_ERR_ARG,
             "fm_build_index: H=%d C=%d N=%d d=%d Z=%d", H, C, N, d, Z);
  FM_REQUIRE(A && K && idx_out && ws, FM_ERR_ARG, "fm_build_index: null pointer");
  const int64_t ldy = (int64_t(N) + 3) / 4 * 4;  // rows start 16-byte aligned
  const size_t sel_ws = align_up(fm_argtopz_workspace(int64_t(H) * C, N, Z), 256);
  FM_REQUIRE(ws_bytes > sel_ws, FM_ERR_WORKSPACE, "fm_build_index: workspace %zu does not hold the selection scratch %zu",
             ws_bytes, sel_ws);
  void* const sel = ws;
  ws = static_cast<char*>(ws) + sel_ws;
  ws_bytes -= sel_ws;
  const int64_t fit = int64_t(ws_bytes / (size_t(ldy) * sizeof(float)));
  FM_REQUIRE(fit >= 1, FM_ERR_WORKSPACE, "fm_build_index: workspace %zu holds no row of %lld floats",
             ws_bytes, (long long)ldy);
  const int Zc = Z < N ? Z : N;
  const size_t esz = size_t(dtype_bytes(dtype));
  float* Y = static_cast<float*>(ws);
  // a pass takes as many whole heads as fit, or a bucket range [c0, c0+nc) of one head
  for (int h = 0; h < H;) {
    if (fit >= C) {
      const int hb = int(std::min<int64_t>(fit / C, H - h));
      const char* Ah = static_cast<const char*>(A) + int64_t(h) * C * d * esz;
      const char* Kh = static_cast<const char*>(K) + int64_t(h) * N * d * esz;
      int rc = fm_project(Ah, Kh, Y, hb, C, N, d, ldy, dtype, stream);
      if (rc) return rc;
      rc = fm_argtopz_f32(Y, int64_t(hb) * C, N, ldy, Z, idx_out + int64_t(h) * C * Zc,
                          val_out ? val_out + int64_t(h) * C * Zc : nullptr, sel, sel_ws, stream);
      if (rc) return rc;
      h += hb;
      continue;
    }
    for (int c0 = 0; c0 < C;) {
      int nc = int(std::min<int64_t>(fit, C - c0));
      const char* Ah = static_cast<const char*>(A) + (int64_t(h) * C + c0) * d * esz;
      const char* Kh = static_cast<const char*>(K) + int64_t(h) * N * d * esz;
      int rc = fm_project(Ah, Kh, Y, 1, nc, N, d, ldy, dtype, stream);
      if (rc) return rc;
      rc = fm_argtopz_f32(Y, nc, N, ldy, Z, idx_out + (int64_t(h) * C + c0) * Zc,
                          val_out ? val_out + (int64_t(h) * C + c0) * Zc : nullptr, sel, sel_ws, stream);
      if (rc) return rc;
      c0 += nc;
    }
    ++h;
  }
  return FM_OK;
}
