// Bucket lists rewritten in ascending key order.
//
// The gathered attention (triton_kernel.py:230-272) walks a bucket's list in stored order and its result
// does not depend on that order beyond the rounding of the fp32 sums.  torch.topk (memory.py:273) leaves
// the lists in descending score order, i.e. in random key order: every 64-key tile then touches 64
// unrelated pages of K and of V.  In ascending key order a tile's rows lie within a few pages and a
// workgroup moves through K and V front to back, which the address translation and the memory side
// reward (measured: 10 % on the 1M-key workload, 20 % on the prefill chunk; nothing for single-query
// decode).
//
// Per list, a counting sort over a bitmap of the key range in LDS: set the bit of every listed key, then
// walk the bitmap in order.  A wave owns an equal share of a pass's words (2048 of a full range) and takes
// them 64 at a time, a lane a word: the wave's scan of the lanes' bit counts gives every lane its output position, and the keys
// of 64 neighbouring words land in one or two lines per store.  Ranges of NT * 1024 keys per pass, as many
// passes as N needs; cost per list ~ N / 32 word visits + its length, independent of the order it arrives
// in, and no limit on the length of a list (the list itself never sits in LDS).  A list that names a key
// twice, or a key outside [0, N), marks fewer bits than it has entries: it is copied unchanged and
// counted.
#include "common.hpp"

namespace fm {

template <int NT>
__global__ __launch_bounds__(NT) void lists_key_order_kernel(const int32_t* __restrict__ in,
                                                             const int64_t* __restrict__ off,
                                                             const int32_t* __restrict__ cnt, int N,
                                                             int32_t* __restrict__ out,
                                                             int32_t* __restrict__ n_unsorted) {
  extern __shared__ uint32_t lo_bm[];  // 32 * NT words
  __shared__ int scan_tmp[17];
  constexpr int64_t kRange = int64_t(NT) * 1024;  // keys per pass
  constexpr int kHeld = 16;                       // entries per thread kept in registers between passes
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = cnt[blockIdx.x];
  if (n <= 0) return;
  const int32_t* src = in + off[blockIdx.x];
  int32_t* dst = out + off[blockIdx.x];
  const bool held = n <= kHeld * NT;
  int mine[kHeld];
  if (held) {
#pragma unroll
    for (int r = 0; r < kHeld; ++r) mine[r] = tid + r * NT < n ? src[tid + r * NT] : -1;
  }
  int written = 0;  // entries the earlier passes wrote (the same in every thread)
  for (int64_t r0 = 0; r0 < N; r0 += kRange) {
    const int n_keys = int(min(kRange, int64_t(N) - r0));
    const int n_words = (n_keys + 31) >> 5;
    for (int s = tid; s < n_words; s += NT) lo_bm[s] = 0;
    __syncthreads();
    auto mark = [&](int k) {
      const int64_t rel = int64_t(k) - r0;
      if (rel >= 0 && rel < n_keys) atomicOr(&lo_bm[uint32_t(rel) >> 5], 1u << (uint32_t(rel) & 31u));
    };
    if (held) {
#pragma unroll
      for (int r = 0; r < kHeld; ++r) mark(mine[r]);
    } else {
      for (int i = tid; i < n; i += NT) mark(src[i]);
    }
    __syncthreads();
    // the pass's words in equal shares of whole 64-word steps (2048 words a wave when the range is full)
    const int wave_words = ((n_words + NT - 1) / NT) * 64;
    const int w0 = wave * wave_words;
    int c = 0;
    for (int s = w0 + lane; s < min(n_words, w0 + wave_words); s += 64) c += __popc(lo_bm[s]);
    c = __builtin_amdgcn_readlane(wave_incl_scan_dpp(c), 63);
    int total;
    int base = block_excl_scan(lane == 0 ? c : 0, scan_tmp, &total);
    base = written + __builtin_amdgcn_readfirstlane(base);
    if (c > 0) {
      for (int s0 = w0; s0 < min(n_words, w0 + wave_words); s0 += 64) {
        const int s = s0 + lane;
        uint32_t w = s < n_words ? lo_bm[s] : 0u;
        const int pc = __popc(w);
        const int incl = wave_incl_scan_dpp(pc);
        int pos = base + incl - pc;
        const int key0 = int(r0) + (s << 5);
        while (w) {
          const int b = __ffs(int(w)) - 1;
          w &= w - 1u;
          dst[pos++] = key0 + b;
        }
        base += __builtin_amdgcn_readlane(incl, 63);
      }
    }
    written += total;
    __syncthreads();  // the bitmap is cleared again by the next pass
  }
  if (written != n) {  // some entry marked no bit of its own
    for (int i = tid; i < n; i += NT) dst[i] = src[i];
    if (tid == 0 && n_unsorted) atomicAdd(n_unsorted, 1);
  }
}

__global__ void lists_zero_count_kernel(int32_t* p) { *p = 0; }

}  // namespace fm

extern "C" int fm_lists_key_order(const int32_t* k_idx, const int64_t* bucket_off, const int32_t* bucket_cnt,
                                  int64_t n_lists, int N, int32_t* k_idx_out, int32_t* n_unsorted,
                                  void* stream) {
  using namespace fm;
  FM_REQUIRE(n_lists >= 0 && N >= 1, FM_ERR_ARG, "fm_lists_key_order: n_lists=%lld N=%d", (long long)n_lists, N);
  FM_REQUIRE(n_lists <= 0x7fffffffLL, FM_ERR_UNSUPPORTED, "fm_lists_key_order: too many lists");
  FM_REQUIRE(n_lists == 0 || (k_idx && bucket_off && bucket_cnt && k_idx_out), FM_ERR_ARG,
             "fm_lists_key_order: null pointer");
  FM_REQUIRE(n_lists == 0 || k_idx != k_idx_out, FM_ERR_ARG,
             "fm_lists_key_order: the lists cannot be reordered in place");
  hipStream_t st = as_stream(stream);
  if (n_unsorted) hipLaunchKernelGGL(lists_zero_count_kernel, dim3(1), dim3(1), 0, st, n_unsorted);
  if (n_lists == 0) return n_unsorted ? launch_status("fm_lists_key_order") : FM_OK;
  // narrow workgroups (several per CU) while one pass of theirs covers the key range: every pass walks
  // the whole list again, so beyond that the widest form, with the fewest passes, is the fastest
  const int nt = N <= 256 * 1024 ? 256 : N <= 512 * 1024 ? 512 : 1024;
  if (nt == 256) {
    constexpr size_t lds = 256 * 32 * sizeof(uint32_t);
    hipLaunchKernelGGL(lists_key_order_kernel<256>, dim3(unsigned(n_lists)), dim3(256), lds, st, k_idx, bucket_off,
                       bucket_cnt, N, k_idx_out, n_unsorted);
  } else if (nt == 512) {
    constexpr size_t lds = 512 * 32 * sizeof(uint32_t);
    hipLaunchKernelGGL(lists_key_order_kernel<512>, dim3(unsigned(n_lists)), dim3(512), lds, st, k_idx, bucket_off,
                       bucket_cnt, N, k_idx_out, n_unsorted);
  } else {
    constexpr size_t lds = 1024 * 32 * sizeof(uint32_t);
    FM_ALLOW_LDS(lists_key_order_kernel<1024>, lds, "fm_lists_key_order: lds");
    hipLaunchKernelGGL(lists_key_order_kernel<1024>, dim3(unsigned(n_lists)), dim3(1024), lds, st, k_idx, bucket_off,
                       bucket_cnt, N, k_idx_out, n_unsorted);
  }
  return launch_status("fm_lists_key_order");
}
