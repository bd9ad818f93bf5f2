// placeholder until the MFMA attention kernels land
#include "common.hpp"
namespace fm {
bool hash_attn_mfma_supported(int, int) { return false; }
int hash_attn_mfma(const void*, const void*, const void*, const int32_t*, const int64_t*,
                   const int32_t*, const int32_t*, const fm_item*, const int32_t*, int64_t, void*,
                   float*, int, int, int, int, float, hipStream_t) {
  set_error("hash_attn_mfma: not built");
  return FM_ERR_UNSUPPORTED;
}
bool local_attn_mfma_supported(int, int) { return false; }
int local_attn_mfma(const void*, const void*, const void*, void*, float*, int, int, int, int, int,
                    float, int, hipStream_t) {
  set_error("local_attn_mfma: not built");
  return FM_ERR_UNSUPPORTED;
}
}  // namespace fm
