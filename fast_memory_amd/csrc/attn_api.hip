// C entry points of the attention operators; picks the MFMA kernels for the
// shapes they are built for and the generic kernels otherwise.
#include "common.hpp"

#include <mutex>

namespace fm {
int hash_attn_generic(const void* q, const void* k, const void* v, const int32_t* k_idx,
                      const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                      const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                      float* lse, int Sq, int N, int d, int C, float sm_scale, int dtype,
                      hipStream_t st);
int local_attn_generic(const void* q, const void* k, const void* v, void* out, float* lse, int H,
                       int G, int S, int L, int d, float sm_scale, int causal, int dtype,
                       hipStream_t st);
bool hash_attn_mfma_supported(int d, int dtype, int N);
int hash_attn_mfma(const void* q, const void* k, const void* v, const int32_t* k_idx,
                   const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                   const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                   float* lse, int H, int Sq, int N, int d, int C, float sm_scale, int dtype, void* ws, size_t ws_bytes,
                   hipStream_t st);
size_t hash_attn_ring_workspace(int64_t max_items);
int hash_attn_mfma_choice(int H, int Sq, int N, int C);
bool hash_attn_mfma_per_row(int choice, int H, int Sq, int N, int C);
bool local_attn_mfma_supported(int d, int dtype);
int local_attn_mfma(const void* q, const void* k, const void* v, void* out, float* lse, int H, int G,
                    int S, int L, int d, int dtype, float sm_scale, int causal, hipStream_t st);

int launch_unlisted_rows(const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                         const int32_t* bin_off, const int32_t* bin_count, int64_t n_bins, int64_t nq,
                         int row_bytes, void* rows, float* lse, hipStream_t st);  // group.hip

int decode_hash_attn(const void* q, const void* A_all, const void* K_all, const void* V_all,
                     const int32_t* idx_all, const fm_rowdesc* desc, int rows, int G, float sm_scale,
                     void* out, float* lse, int32_t* hash_out, float* scores_out, hipStream_t st);

// 0 = automatic, 1 = force the generic kernels (used by tests to compare paths); for the grouped
// forward on MFMA, 2 = always the form that stages a bucket's rows in LDS (4: two work items per
// workgroup), 5 = always the form that loads them straight into LDS, 3 = always the form that gathers them
// into registers
std::atomic<int> g_force_generic{0};
}  // namespace fm

extern "C" void fm_debug_force_generic(int on) {
  if (fm::debug_hooks_enabled()) fm::g_force_generic.store(on, std::memory_order_relaxed);
}

extern "C" const char* fm_hash_attn_fwd_kernel(int H, int Sq, int N, int d, int C, int dtype) {
  using namespace fm;
  if (g_force_generic == 1 || !hash_attn_mfma_supported(d, dtype, N)) return "hash_attn_generic_kernel";
  if (d == 64) return dtype == FM_F16 ? "hash_attn_staged_d_kernel<64, f16>" : "hash_attn_staged_d_kernel<64>";
  if (d == 256) return dtype == FM_F16 ? "hash_attn_staged_d_kernel<256, f16>" : "hash_attn_staged_d_kernel<256>";
  if (g_force_generic == 8) return dtype == FM_F16 ? "hash_attn_staged_d_kernel<128, f16>" : "hash_attn_staged_d_kernel<128>";
  const int choice = hash_attn_mfma_choice(H, Sq, N, C);
  if (choice && N > (1 << 24))
    return dtype == FM_F16 ? "hash_attn_staged_kernel<1, f16, 64-bit rows>" : "hash_attn_staged_kernel<1, 64-bit rows>";
  if (choice == 4) return dtype == FM_F16 ? "hash_attn_wave_kernel<f16>" : "hash_attn_wave_kernel";
  if (dtype == FM_F16)
    return choice == 3 ? "hash_attn_ring_kernel<f16>"
                       : choice == 2 ? "hash_attn_staged_kernel<2, f16>" : "hash_attn_staged_kernel<1, f16>";
  switch (choice) {
    case 1: return "hash_attn_staged_kernel<1>";
    case 2: return "hash_attn_staged_kernel<2>";
    case 3: return "hash_attn_ring_kernel";
    default: return "hash_attn_mfma_kernel";
  }
}

extern "C" const char* fm_local_attn_fwd_kernel(int G, int S, int L, int d, int dtype) {
  using namespace fm;
  if (g_force_generic == 1 || !local_attn_mfma_supported(d, dtype)) return "local_attn_generic_kernel";
  if (S == 1 && G <= 16 && L >= 1 && d == 128 && dtype == FM_BF16) return "local_attn_decode_kernel";
  if (d == 64) return dtype == FM_F16 ? "local_attn_dense_kernel<f16, 64>" : "local_attn_dense_kernel<bf16, 64>";
  if (d == 128) return dtype == FM_F16 ? "local_attn_dense_kernel<f16, 128>" : "local_attn_dense_kernel<bf16, 128>";
  return dtype == FM_F16 ? "local_attn_dense_kernel<f16, 256>" : "local_attn_dense_kernel<bf16, 256>";
}

namespace fm {
int wave_pace_state(int N, int C, int Sq, const void* lists, int row, float* out);
}
extern "C" int fm_debug_wave_pace_state(int N, int C, int Sq, const void* k_idx, int row, float* out8) {
  if (!out8) return FM_ERR_ARG;
  return fm::wave_pace_state(N, C, Sq, k_idx, row, out8);
}

extern "C" int fm_hash_attn_fwd_launches(int H, int Sq, int N, int d, int C, int dtype) {
  using namespace fm;
  if (g_force_generic == 1 || !hash_attn_mfma_supported(d, dtype, N) || d != 128 || g_force_generic == 8) return 1;
  int choice = hash_attn_mfma_choice(H, Sq, N, C);
  if (dtype == FM_F16 && choice == 0) choice = 1;
  return hash_attn_mfma_per_row(choice, H, Sq, N, C) ? H : 1;
}

extern "C" size_t fm_hash_attn_fwd_workspace(int64_t max_items) {
  return max_items >= 1 ? fm::hash_attn_ring_workspace(max_items) : 0;
}

extern "C" int fm_hash_attn_fwd_ws(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                   const int64_t* bucket_off, const int32_t* bucket_cnt,
                                   const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                                   int64_t max_items, void* out, float* lse, int H, int Sq, int N,
                                   int d, int C, float sm_scale, int dtype, void* ws, size_t ws_bytes,
                                   void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && Sq >= 1 && N >= 1 && C >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG,
             "fm_hash_attn_fwd: H=%d Sq=%d N=%d C=%d d=%d", H, Sq, N, C, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_hash_attn_fwd: dtype=%d", dtype);
  FM_REQUIRE(q && k && v && k_idx && bucket_off && bucket_cnt && q_perm && items && n_items && out &&
                 lse,
             FM_ERR_ARG, "fm_hash_attn_fwd: null pointer");
  FM_REQUIRE(max_items >= 1 && max_items <= 0x7fffffffLL, FM_ERR_ARG,
             "fm_hash_attn_fwd: max_items=%lld", (long long)max_items);
  FM_REQUIRE(!ws || ws_bytes >= hash_attn_ring_workspace(max_items), FM_ERR_WORKSPACE,
             "fm_hash_attn_fwd_ws: workspace %zu < %zu", ws_bytes, hash_attn_ring_workspace(max_items));
  hipStream_t st = as_stream(stream);
  int rc;
  if (g_force_generic != 1 && hash_attn_mfma_supported(d, dtype, N))
    rc = hash_attn_mfma(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items,
                        out, lse, H, Sq, N, d, C, sm_scale, dtype, ws, ws ? ws_bytes : 0, st);
  else
    rc = hash_attn_generic(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items,
                           max_items, out, lse, Sq, N, d, C, sm_scale, dtype, st);
  if (rc) return rc;
  // queries that are part of no work item (hash outside [0, C)): the result of an empty bucket
  return launch_unlisted_rows(q_perm, items, n_items, nullptr, nullptr, 0, int64_t(H) * Sq,
                              d * dtype_bytes(dtype), out, lse, st);
}

extern "C" int fm_hash_attn_fwd(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                const int64_t* bucket_off, const int32_t* bucket_cnt,
                                const int32_t* q_perm, const fm_item* items, const int32_t* n_items,
                                int64_t max_items, void* out, float* lse, int H, int Sq, int N,
                                int d, int C, float sm_scale, int dtype, void* stream) {
  return fm_hash_attn_fwd_ws(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items, out, lse,
                             H, Sq, N, d, C, sm_scale, dtype, nullptr, 0, stream);
}

// workspace layout of the one-call operator
namespace fm {
struct VarlenWs {
  size_t off_bucket_off, off_q_perm, off_bin_count, off_bin_off, off_items, off_n_items, off_group,
      off_attn, total;
  int64_t max_items;
};
static VarlenWs varlen_layout(int H, int C, int Sq) {
  VarlenWs w;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    size_t r = o;
    o = align_up(o + bytes, 256);
    return r;
  };
  w.max_items = fm_group_max_items(H, C, Sq);
  w.off_bucket_off = take(size_t(H) * C * sizeof(int64_t));
  w.off_q_perm = take(size_t(H) * Sq * sizeof(int32_t));
  w.off_bin_count = take(size_t(H) * C * sizeof(int32_t));
  w.off_bin_off = take(size_t(H) * C * sizeof(int32_t));
  w.off_items = take(size_t(w.max_items) * sizeof(fm_item));
  w.off_n_items = take(sizeof(int32_t));
  w.off_group = take(fm_group_queries_workspace(H, C, Sq));
  w.off_attn = take(fm_hash_attn_fwd_workspace(w.max_items));
  w.total = o;
  return w;
}
}  // namespace fm

extern "C" size_t fm_attention_hash_varlen_workspace(int H, int C, int Sq) {
  if (H < 1 || C < 1 || Sq < 1) return 0;
  return fm::varlen_layout(H, C, Sq).total;
}

namespace fm {
// bucket offsets + grouping + attention with every intermediate in the buffer at `base`
static int varlen_run(const void* q, const void* k, const void* v, const int32_t* k_idx,
                      const int32_t* bucket_cnt, const int32_t* q_hash, void* out, float* lse, int H,
                      int Sq, int N, int d, int C, float sm_scale, int dtype, char* base,
                      const VarlenWs& w, void* stream) {
  int64_t* bucket_off = reinterpret_cast<int64_t*>(base + w.off_bucket_off);
  int32_t* q_perm = reinterpret_cast<int32_t*>(base + w.off_q_perm);
  int32_t* bin_count = reinterpret_cast<int32_t*>(base + w.off_bin_count);
  int32_t* bin_off = reinterpret_cast<int32_t*>(base + w.off_bin_off);
  fm_item* items = reinterpret_cast<fm_item*>(base + w.off_items);
  int32_t* n_items = reinterpret_cast<int32_t*>(base + w.off_n_items);
  int rc = fm_bucket_offsets(bucket_cnt, int64_t(H) * C, bucket_off, stream);
  if (rc) return rc;
  rc = fm_group_queries(q_hash, H, C, Sq, q_perm, bin_count, bin_off, items, n_items, w.max_items,
                        base + w.off_group, fm_group_queries_workspace(H, C, Sq), stream);
  if (rc) return rc;
  rc = fm_hash_attn_fwd_ws(q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, w.max_items, out,
                           lse, H, Sq, N, d, C, sm_scale, dtype, base + w.off_attn,
                           fm_hash_attn_fwd_workspace(w.max_items), stream);
  return rc;
}

// every argument check of the one-call operators, ahead of their first launch (a caller that records
// the call into a graph must not be left with half a sequence)
static int varlen_check(const char* name, const void* q, const void* k, const void* v, const int32_t* k_idx,
                        const int32_t* bucket_cnt, const int32_t* q_hash, const void* out, const float* lse,
                        int H, int Sq, int N, int d, int C, int dtype) {
  FM_REQUIRE(H >= 1 && Sq >= 1 && N >= 1 && C >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG,
             "%s: H=%d Sq=%d N=%d C=%d d=%d", name, H, Sq, N, C, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "%s: dtype=%d", name, dtype);
  FM_REQUIRE(q && k && v && k_idx && bucket_cnt && q_hash && out && lse, FM_ERR_ARG, "%s: null pointer", name);
  FM_REQUIRE(int64_t(H) * Sq <= 0x7fffffffLL && int64_t(H) * C <= 0x7fffffffLL && H <= 65535, FM_ERR_UNSUPPORTED,
             "%s: H*Sq or H*C exceeds int32, or H > 65535", name);
  return FM_OK;
}
}  // namespace fm

extern "C" int fm_attention_hash_varlen(const void* q, const void* k, const void* v,
                                        const int32_t* k_idx, const int32_t* bucket_cnt,
                                        const int32_t* q_hash, void* out, float* lse, int H, int Sq,
                                        int N, int d, int C, float sm_scale, int dtype, void* ws,
                                        size_t ws_bytes, void* stream) {
  using namespace fm;
  int rc = varlen_check("fm_attention_hash_varlen", q, k, v, k_idx, bucket_cnt, q_hash, out, lse, H, Sq, N, d, C, dtype);
  if (rc) return rc;
  FM_REQUIRE(ws, FM_ERR_ARG, "fm_attention_hash_varlen: null pointer");
  VarlenWs w = varlen_layout(H, C, Sq);
  FM_REQUIRE(ws_bytes >= w.total, FM_ERR_WORKSPACE, "fm_attention_hash_varlen: workspace %zu < %zu",
             ws_bytes, w.total);
  return varlen_run(q, k, v, k_idx, bucket_cnt, q_hash, out, lse, H, Sq, N, d, C, sm_scale, dtype,
                    static_cast<char*>(ws), w, stream);
}

// ---- the same operator for callers that cannot allocate ------------------------------------
// The grouping tables, the permutation and the work items live in a device array of the library
// itself, one copy per GPU.  In host code the array's name only stands for the symbol: the device
// address comes from hipGetSymbolAddress, once per device, and only that pointer is used below.
namespace fm {
static __device__ __align__(256) unsigned char scratch[FM_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, 0 = not asked yet

static int scratch_of_current_device(char** ptr_out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    set_error("fm_attention_hash_varlen_static: no current device (hipGetDevice gave %d)", dev);
    return FM_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      set_error("fm_attention_hash_varlen_static: hipGetSymbolAddress on device %d: %s", dev,
                hipGetErrorString(e));
      return FM_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = p;
  }
  *ptr_out = static_cast<char*>(g_scratch_ptr[dev]);
  return FM_OK;
}
}  // namespace fm

extern "C" int fm_attention_hash_varlen_static(const void* q, const void* k, const void* v,
                                               const int32_t* k_idx, const int32_t* bucket_cnt,
                                               const int32_t* q_hash, void* out, float* lse, int H,
                                               int Sq, int N, int d, int C, float sm_scale, int dtype,
                                               void* stream) {
  using namespace fm;
  int rc = varlen_check("fm_attention_hash_varlen_static", q, k, v, k_idx, bucket_cnt, q_hash, out, lse, H, Sq, N, d,
                        C, dtype);
  if (rc) return rc;
  VarlenWs w = varlen_layout(H, C, Sq);
  FM_REQUIRE(w.total <= size_t(FM_STATIC_SCRATCH_BYTES), FM_ERR_WORKSPACE,
             "fm_attention_hash_varlen_static: H=%d C=%d Sq=%d needs %zu bytes of scratch, the static "
             "array holds %zu; use fm_attention_hash_varlen with a workspace",
             H, C, Sq, w.total, size_t(FM_STATIC_SCRATCH_BYTES));
  char* base = nullptr;
  rc = scratch_of_current_device(&base);
  if (rc) return rc;
  // nothing in the array has to survive from an earlier call: the grouping clears its block table
  // with a fill kernel and every other region is written before it is read
  return varlen_run(q, k, v, k_idx, bucket_cnt, q_hash, out, lse, H, Sq, N, d, C, sm_scale, dtype,
                    base, w, stream);
}

extern "C" int fm_local_attn_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                                 int H, int G, int S, int L, int d, float sm_scale, int causal,
                                 int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && G >= 1 && S >= 1 && L >= 1 && d >= 1 && d <= FM_MAX_D, FM_ERR_ARG,
             "fm_local_attn_fwd: H=%d G=%d S=%d L=%d d=%d", H, G, S, L, d);
  FM_REQUIRE(dtype_ok(dtype), FM_ERR_ARG, "fm_local_attn_fwd: dtype=%d", dtype);
  FM_REQUIRE(q && k && v && out && lse, FM_ERR_ARG, "fm_local_attn_fwd: null pointer");
  FM_REQUIRE(int64_t(H) * G <= 65535, FM_ERR_UNSUPPORTED, "fm_local_attn_fwd: H*G > 65535");
  FM_REQUIRE(S <= 65535 * 128, FM_ERR_UNSUPPORTED, "fm_local_attn_fwd: S=%d > 65535 * 128", S);
  hipStream_t st = as_stream(stream);
  if (g_force_generic != 1 && local_attn_mfma_supported(d, dtype))
    return local_attn_mfma(q, k, v, out, lse, H, G, S, L, d, dtype, sm_scale, causal, st);
  return local_attn_generic(q, k, v, out, lse, H, G, S, L, d, sm_scale, causal, dtype, st);
}

extern "C" int fm_decode_hash_attn(const void* q, const void* A_all, const void* K_all,
                                   const void* V_all, const int32_t* idx_all, const fm_rowdesc* desc,
                                   int rows, int G, int d, float sm_scale, void* out, float* lse,
                                   int32_t* hash_out, float* scores_out, int dtype, void* stream) {
  using namespace fm;
  FM_REQUIRE(rows >= 0 && G >= 1 && G <= 16, FM_ERR_ARG, "fm_decode_hash_attn: rows=%d G=%d", rows, G);
  FM_REQUIRE(int64_t(rows) * G <= 0x7fffffffLL, FM_ERR_UNSUPPORTED, "fm_decode_hash_attn: rows * G = %lld workgroups",
             (long long)(int64_t(rows) * G));
  FM_REQUIRE(dtype == FM_BF16 && d == 128, FM_ERR_UNSUPPORTED,
             "fm_decode_hash_attn: built for bf16, d=128 (got dtype=%d d=%d)", dtype, d);
  if (rows == 0) return FM_OK;
  FM_REQUIRE(q && A_all && K_all && V_all && idx_all && desc && out && lse && hash_out, FM_ERR_ARG,
             "fm_decode_hash_attn: null pointer");
  return decode_hash_attn(q, A_all, K_all, V_all, idx_all, desc, rows, G, sm_scale, out, lse, hash_out,
                          scores_out, as_stream(stream));
}
