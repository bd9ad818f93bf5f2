// Extending an index by new keys without rebuilding it (the reference rebuilds
// the bucket lists from all keys on every forward, memory.py:252-278).
//
// A bucket's list is the top-Z of its row of Y = A.K^T by (value descending, key
// index ascending).  Given the list with its values and M new keys (indices
// N_old .. N_old+M-1), the new list is the top-Z of the union.  Per (head, bucket)
// row, one workgroup:
//   1. projections of the new keys are read from the workspace (fm_project wrote
//      them: the same MFMA sums a rebuild would see) and those that beat the
//      list's last entry are collected into LDS as 64-bit composites (a new key
//      never wins a tie: its index is larger than every old one);
//   2. the m survivors are sorted (the bitonic network of the selection kernels);
//   3. merge by ranks: an old entry at position p moves to p + (new entries ahead
//      of it), found by binary search among the survivors in LDS; a new entry of
//      rank r moves to r + (old entries ahead of it), which the old entries'
//      searches give as a by-product (the survivors between old entries p-1 and
//      p have p old entries ahead); positions >= the new length fall off the end.
// Work is O(Z + M) memory operations per row instead of a projection over all
// N keys.  HBM-bound: out of place the lists are read and written once (8 B per
// entry each way) plus 4 B per new (bucket, key) pair.  In place (full lists
// only) a row without survivors reads its last entry and nothing else, and a row
// with survivors is staged in LDS and rewritten from its first insertion on: a
// few new keys against long lists touch almost nothing.
#include "select.hpp"

namespace fm {

int launch_fill(int32_t* p, int64_t n, int32_t v, hipStream_t st);  // group.hip

constexpr int kAppendMaxNew = 8192;                    // survivors per row the LDS sort buffer takes at most
constexpr int kAppendPer = FM_MAX_Z / kSelThreads;     // old entries a thread holds in registers, at most
constexpr int kAppendWaves = kSelThreads / 64;
static_assert(kAppendPer * kSelThreads == FM_MAX_Z, "a workgroup's registers hold one full list");

// INPLACE: idx_out/val_out are idx_in/val_in (L_out == L_in); no __restrict__ on the lists for that reason.
// Every thread reads its share of the old list into registers before the barrier that precedes the
// first write, so one code path serves both modes.
template <bool INPLACE, int PER>
__device__ __forceinline__ void append_row(
    int64_t row, uint64_t* nb, int& s_cnt, int (&s_wlast)[PER][kAppendWaves],
    const float* __restrict__ Ynew, int64_t ldm, int M, int n_old, const int32_t* idx_in, const float* val_in, int L_in,
    int32_t* idx_out, float* val_out, int L_out, int Z, int max_new, int32_t* __restrict__ status) {
  int* ahead = reinterpret_cast<int*>(nb + sort_lds_bytes(max_new) / sizeof(uint64_t));  // old entries ahead of survivor r
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* y = Ynew + row * ldm;
  const int32_t* ii = idx_in + row * L_in;
  const float* vi = val_in + row * L_in;
  int32_t* io = idx_out + row * L_out;
  float* vo = val_out + row * L_out;
  if (tid == 0) s_cnt = 0;
  __syncthreads();
  // the list's last entry is the bar while the list is full; a shorter list takes every new key
  const bool full = L_in >= Z;
  const uint64_t bar = full ? composite(vi[L_in - 1], uint32_t(ii[L_in - 1])) : 0ull;
  for (int j = tid; j < M; j += kSelThreads) {
    const uint64_t c = composite(y[j], uint32_t(n_old + j));
    if (!full || c > bar) {
      const int pos = atomicAdd(&s_cnt, 1);
      if (pos < max_new) nb[sort_phys(pos)] = c;
    }
  }
  __syncthreads();
  const int m = s_cnt;
  if (m > max_new) {  // more survivors than the buffer takes: the caller rebuilds
    if (tid == 0) atomicAdd(status, 1);
    return;
  }
  if (INPLACE && m == 0) return;  // nothing beats the bar: the row stands
  int P = 64;
  while (P < m) P <<= 1;
  for (int i = m + tid; i < P; i += kSelThreads) nb[sort_phys(i)] = 0ull;
  for (int j = tid; j < m; j += kSelThreads) ahead[j] = L_in;  // survivors behind every old entry
  __syncthreads();
  if (m > 1) bitonic_sort_desc(nb, 31 - __clz(P));
  __syncthreads();
  // the old list, entry p = tid + k*kSelThreads in register k
  int32_t ix[PER];
  float v[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int p = tid + k * kSelThreads;
    ix[k] = p < L_in ? ii[p] : 0;
    v[k] = p < L_in ? vi[p] : 0.f;
  }
  // old entry p moves back by lo = the number of survivors ahead of it (composites are unique)
  int lo[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int p = tid + k * kSelThreads;
    int a = 0, b = p < L_in ? m : 0;  // first survivor position whose composite is < c
    const uint64_t c = composite(v[k], uint32_t(ix[k]));
    while (a < b) {
      const int mid = (a + b) >> 1;
      if (nb[sort_phys(mid)] > c)
        a = mid + 1;
      else
        b = mid;
    }
    lo[k] = a;
    if (lane == 63) s_wlast[k][wave] = a;
  }
  __syncthreads();  // the old list is in registers everywhere: writes may start
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int p = tid + k * kSelThreads;
    if (k * kSelThreads >= L_in) break;
    const bool valid = p < L_in;
    // survivors lo(p-1) .. lo(p)-1 sit between old entries p-1 and p: exactly p old entries are ahead of them
    int lo_prev = __shfl_up(lo[k], 1);
    if (lane == 0) lo_prev = wave > 0 ? s_wlast[k][wave - 1] : (k > 0 ? s_wlast[k - 1][kAppendWaves - 1] : 0);
    uint64_t runs = __ballot(valid && lo[k] > lo_prev);
    while (runs) {  // rare; the whole wavefront fills one run at a time
      const int l = __builtin_ctzll(runs);
      runs &= runs - 1;
      const int ja = __shfl(lo_prev, l), jb = __shfl(lo[k], l), pp = __shfl(p, l);
      for (int j = ja + lane; j < jb; j += 64) ahead[j] = pp;
    }
    const int pos = p + lo[k];
    if (valid && pos < L_out && !(INPLACE && lo[k] == 0)) {  // in place, entries ahead of the first insertion stay
      io[pos] = ix[k];
      vo[pos] = v[k];
    }
  }
  __syncthreads();
  // survivors: new position = rank + number of old entries ahead
  for (int r = tid; r < m; r += kSelThreads) {
    const uint64_t c = nb[sort_phys(r)];
    const int pos = r + ahead[r];
    if (pos < L_out) {
      io[pos] = int32_t(0xffffffffu - uint32_t(c));
      vo[pos] = key_to_float(uint32_t(c >> 32));
    }
  }
}

// one workgroup per row
template <bool INPLACE, int PER>
__global__ __launch_bounds__(kSelThreads) void index_append_kernel(
    const float* __restrict__ Ynew, int64_t ldm, int M, int n_old, const int32_t* idx_in, const float* val_in, int L_in,
    int32_t* idx_out, float* val_out, int L_out, int Z, int max_new, int32_t* __restrict__ status) {
  extern __shared__ uint64_t nb[];  // sorted survivors (sort_phys layout), then ahead[max_new]
  __shared__ int s_cnt;
  __shared__ int s_wlast[PER][kAppendWaves];
  append_row<INPLACE, PER>(blockIdx.x, nb, s_cnt, s_wlast, Ynew, ldm, M, n_old, idx_in, val_in, L_in, idx_out, val_out,
                           L_out, Z, max_new, status);
}

// In place with few new keys, most rows stand as they are (a new key enters a list with probability
// about Z/N): one thread per row finds the rows some new key enters ...
__global__ __launch_bounds__(256) void append_precheck_kernel(const float* __restrict__ Ynew, int64_t ldm, int M,
                                                              int n_old, const int32_t* __restrict__ idx_in,
                                                              const float* __restrict__ val_in, int L, int64_t rows,
                                                              int32_t* __restrict__ list, int32_t* __restrict__ n_list) {
  const int64_t row = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (row >= rows) return;
  const uint64_t bar = composite(val_in[row * L + L - 1], uint32_t(idx_in[row * L + L - 1]));
  bool any = false;
  for (int j = 0; j < M; ++j) any = any || composite(Ynew[row * ldm + j], uint32_t(n_old + j)) > bar;
  if (any) list[atomicAdd(n_list, 1)] = int32_t(row);
}

// ... and a fixed number of workgroups walks that list (the order of the list does not matter: rows
// are independent).
template <int PER>
__global__ __launch_bounds__(kSelThreads) void index_append_listed_kernel(
    const int32_t* __restrict__ list, const int32_t* __restrict__ n_list, const float* __restrict__ Ynew, int64_t ldm,
    int M, int n_old, int32_t* idx, float* val, int L, int Z, int max_new, int32_t* __restrict__ status) {
  extern __shared__ uint64_t nb[];
  __shared__ int s_cnt;
  __shared__ int s_wlast[PER][kAppendWaves];
  const int n = *n_list;
  for (int i = blockIdx.x; i < n; i += gridDim.x) {
    if (i != int(blockIdx.x)) __syncthreads();  // the row before is done with the shared buffers
    append_row<true, PER>(list[i], nb, s_cnt, s_wlast, Ynew, ldm, M, n_old, idx, val, L, idx, val, L, Z, max_new, status);
  }
}

}  // namespace fm

extern "C" size_t fm_index_append_workspace(int H, int C, int M) {
  if (H < 1 || C < 1 || M < 1) return 0;
  const int64_t ldm = (int64_t(M) + 3) / 4 * 4;
  // projections of the new keys, then the list of rows they enter and its length
  return fm::align_up(size_t(H) * C * ldm * sizeof(float), 256) + fm::align_up(size_t(H) * C * sizeof(int32_t), 256) + 256;
}

extern "C" int fm_index_append(const void* A, const void* K_new, int n_old, int M, const int32_t* idx_in,
                               const float* val_in, int32_t* idx_out, float* val_out, int H, int C, int Z, int d,
                               int dtype, void* ws, size_t ws_bytes, int32_t* status_dev, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && C >= 1 && Z >= 1 && d >= 1 && n_old >= 1 && M >= 1, FM_ERR_ARG,
             "fm_index_append: H=%d C=%d Z=%d d=%d n_old=%d M=%d", H, C, Z, d, n_old, M);
  FM_REQUIRE(A && K_new && idx_in && val_in && idx_out && val_out && ws && status_dev, FM_ERR_ARG,
             "fm_index_append: null pointer");
  const bool inplace = idx_in == idx_out;
  FM_REQUIRE(inplace == (val_in == val_out), FM_ERR_ARG, "fm_index_append: idx and val must both be in place or neither");
  FM_REQUIRE(int64_t(n_old) + M <= 0x7fffffffLL && int64_t(H) * C <= 0x7fffffffLL, FM_ERR_UNSUPPORTED,
             "fm_index_append: index space exhausted");
  FM_REQUIRE(ws_bytes >= fm_index_append_workspace(H, C, M), FM_ERR_WORKSPACE, "fm_index_append: workspace %zu < %zu",
             ws_bytes, fm_index_append_workspace(H, C, M));
  const int64_t ldm = (int64_t(M) + 3) / 4 * 4;
  const int L_in = Z < n_old ? Z : n_old;
  const int L_out = int(std::min<int64_t>(Z, int64_t(n_old) + M));
  FM_REQUIRE(L_out <= FM_MAX_Z, FM_ERR_UNSUPPORTED, "fm_index_append: list length %d exceeds FM_MAX_Z", L_out);
  float* Y = static_cast<float*>(ws);
  hipStream_t st = as_stream(stream);
  int rc = launch_fill(status_dev, 1, 0, st);
  if (rc) return rc;
  rc = fm_project(A, K_new, Y, H, C, M, d, ldm, dtype, stream);
  if (rc) return rc;
  const dim3 grid(unsigned(int64_t(H) * C));
  int max_new = 64;  // a row accepts at most M new keys: small appends take little LDS
  while (max_new < M && max_new < kAppendMaxNew) max_new <<= 1;
  const size_t lds = sort_lds_bytes(max_new) + size_t(max_new) * sizeof(int);
  const size_t lds_max = sort_lds_bytes(kAppendMaxNew) + size_t(kAppendMaxNew) * sizeof(int);
  FM_REQUIRE(!inplace || L_in == L_out, FM_ERR_ARG, "fm_index_append: in place needs full lists (n_old=%d < Z=%d)",
             n_old, Z);
#define FM_APPEND_LAUNCH(INPL, PER)                                                                               \
  do {                                                                                                            \
    FM_ALLOW_LDS((index_append_kernel<INPL, PER>), lds_max, "fm_index_append: lds");                              \
    hipLaunchKernelGGL((index_append_kernel<INPL, PER>), grid, dim3(kSelThreads), lds, st, Y, ldm, M, n_old,      \
                       idx_in, val_in, L_in, idx_out, val_out, L_out, Z, max_new, status_dev);                    \
  } while (0)
  const bool small = L_in <= 8 * kSelThreads;  // 8 list entries per thread instead of 16
  if (inplace && M <= 64) {
    // few new keys, lists stay where they are: only the rows a new key enters are touched
    const int64_t rows = int64_t(H) * C;
    char* base = static_cast<char*>(ws) + align_up(size_t(rows) * ldm * sizeof(float), 256);
    int32_t* list = reinterpret_cast<int32_t*>(base);
    int32_t* n_list = reinterpret_cast<int32_t*>(base + align_up(size_t(rows) * sizeof(int32_t), 256));
    rc = launch_fill(n_list, 1, 0, st);
    if (rc) return rc;
    hipLaunchKernelGGL(append_precheck_kernel, dim3(unsigned(ceil_div(rows, 256))), dim3(256), 0, st, Y, ldm, M, n_old,
                       idx_in, val_in, L_in, rows, list, n_list);
    const dim3 lgrid(unsigned(std::min<int64_t>(rows, 1024)));
    if (small) {
      FM_ALLOW_LDS((index_append_listed_kernel<8>), lds_max, "fm_index_append: lds");
      hipLaunchKernelGGL((index_append_listed_kernel<8>), lgrid, dim3(kSelThreads), lds, st, list, n_list, Y, ldm, M,
                         n_old, idx_out, val_out, L_in, Z, max_new, status_dev);
    } else {
      FM_ALLOW_LDS((index_append_listed_kernel<kAppendPer>), lds_max, "fm_index_append: lds");
      hipLaunchKernelGGL((index_append_listed_kernel<kAppendPer>), lgrid, dim3(kSelThreads), lds, st, list, n_list, Y,
                         ldm, M, n_old, idx_out, val_out, L_in, Z, max_new, status_dev);
    }
  } else if (inplace) {
    if (small) FM_APPEND_LAUNCH(true, 8); else FM_APPEND_LAUNCH(true, kAppendPer);
  } else {
    if (small) FM_APPEND_LAUNCH(false, 8); else FM_APPEND_LAUNCH(false, kAppendPer);
  }
#undef FM_APPEND_LAUNCH
  return launch_status("fm_index_append");
}
