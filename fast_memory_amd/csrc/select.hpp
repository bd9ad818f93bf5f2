// Exact top-Z selection shared by the dense arg-top-Z kernel and the fused
// index build: radix select over unique 64-bit composites, collection of the
// survivors into LDS and a register-blocked in-LDS bitonic sort.
//
// composite(y, i) = (float_key(y) << 32) | (2^32-1 - i): descending composite
// order is "value descending, index ascending", and composites are unique, so
// ties never need a special case.
//
// A `Source` is any callable  src(f)  that calls  f(float value, uint32 index)
// once for every candidate element, from all threads of the workgroup
// together (each element exactly once).
#pragma once
#include "common.hpp"


namespace fm {

constexpr int kSelThreads = 1024;
constexpr int kSelMaxBins = 4096;

__device__ __forceinline__ uint64_t composite(float y, uint32_t i) {
  return (uint64_t(float_key(y)) << 32) | uint64_t(0xffffffffu - i);
}

// inverse of float_key (any 32-bit pattern maps back to some float bit pattern)
__device__ __forceinline__ float key_to_float(uint32_t key) {
  uint32_t u = (key & 0x80000000u) ? (key ^ 0x80000000u) : ~key;
  return __uint_as_float(u);
}

struct SelectShared {
  uint32_t hist[kSelMaxBins];
  int scan_tmp[17];
  uint64_t prefix;
  int need, hit, cnt;
};

// Finds a cut such that exactly `need0` composites of the source are >= cut,
// looking at no more than `max_passes` digits (12,10,10 value bits, then
// 11,11,10 index bits).  With all 6 passes the cut is exact; with fewer it is a
// lower bound of the need0-th largest composite (at least need0 are >= cut).
// Every thread of the workgroup (NT threads, a power of two between 64 and 1024) must call
// this; returns the same cut to all.
template <int NT = kSelThreads, typename Source>
__device__ __forceinline__ uint64_t radix_select_cut(Source& src, int need0, int max_passes,
                                                     SelectShared& sh) {
  const int tid = threadIdx.x;
  if (tid == 0) {
    sh.prefix = 0;
    sh.need = need0;
    sh.hit = 0;
  }
  const int kBits[6] = {12, 10, 10, 11, 11, 10};
  int top = 64;  // bits [top,64) of the cut are known and equal sh.prefix
  for (int pass = 0; pass < max_passes; ++pass) {
    const int bits = kBits[pass];
    const int shift = top - bits;
    const int nb = 1 << bits;
    for (int i = tid; i < nb; i += NT) sh.hist[i] = 0;
    __syncthreads();
    const uint64_t prefix = sh.prefix;
    const int need = sh.need;
    const bool first = (top == 64);
    src([&](float y, uint32_t i) {
      uint64_t c = composite(y, i);
      if (first || (c >> top) == prefix) atomicAdd(&sh.hist[(c >> shift) & uint64_t(nb - 1)], 1u);
    });
    __syncthreads();
    // thread t owns `per` bins, walking digits from the largest down
    const int per = nb / NT;
    int local = 0;
    for (int j = 0; j < per; ++j) local += int(sh.hist[nb - 1 - (tid * per + j)]);
    int total;
    int running = block_excl_scan(local, sh.scan_tmp, &total);
    for (int j = 0; j < per; ++j) {
      int b = nb - 1 - (tid * per + j);
      int h = int(sh.hist[b]);
      if (running < need && need <= running + h) {
        sh.prefix = (prefix << bits) | uint64_t(b);
        sh.need = need - running;
        sh.hit = (h == need - running);
      }
      running += h;
    }
    __syncthreads();
    top = shift;
    if (sh.hit || top == 0) break;
  }
  const uint64_t cut = sh.prefix << top;
  __syncthreads();
  return cut;
}

// ---- in-LDS bitonic sort, descending, register-blocked -------------------------
// The P = 2^logP keys live in LDS at phys(e) = e + e/16 (one pad slot per 16 keeps
// every access pattern below spread over the banks; an XOR swizzle of the low index bits that
// looks conflict-free on paper measured slower).  A thread owns 16 keys whose
// indices differ in four consecutive bits [p, p+4); all compare-exchange stages
// whose distance bit falls in that window run in registers, so a pass over LDS
// (load 16, up to four stages, store 16) replaces up to four passes of the plain
// network: 29 passes instead of 105 at P = 16384.
__device__ __forceinline__ int sort_phys(int e) { return e + (e >> 4); }
static inline size_t sort_lds_bytes(int P) { return size_t(P + (P >> 4) + 1) * sizeof(uint64_t); }

// One compare-exchange stage at register distance 2^D.  Key i of a thread sorts descending when
// bit L of its index is 0; that bit is either a thread bit (tdesc, the same for all 16 keys) or,
// when ib >= 0, bit ib of the register number i (uniform per unrolled i).  Keys are unique (or equal
// padding), so "a > b" is "!(a < b)".
template <int D>
__device__ __forceinline__ void sort_stage_regs(uint64_t (&r)[16], bool tdesc, int ib) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (i & (1 << D)) continue;
    const int j = i | (1 << D);
    const bool flip = ib >= 0 && ((i >> ib) & 1);
    const uint64_t a = r[i], b = r[j];
    const bool sw = (a < b) == (tdesc != flip);
    r[i] = sw ? b : a;
    r[j] = sw ? a : b;
  }
}

__device__ __forceinline__ void bitonic_sort_desc(uint64_t* buf, int logP) {
  const int tid = threadIdx.x;
  if (logP < 6) {  // tiny: plain network, one key pair per thread step
    const int P = 1 << logP;
    for (int k = 2; k <= P; k <<= 1)
      for (int j = k >> 1; j > 0; j >>= 1) {
        for (int t = tid; t < (P >> 1); t += kSelThreads) {
          const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
          const int q = i | j;
          const uint64_t a = buf[sort_phys(i)], b = buf[sort_phys(q)];
          const bool desc = (i & k) == 0;
          if (desc ? (a < b) : (a > b)) {
            buf[sort_phys(i)] = b;
            buf[sort_phys(q)] = a;
          }
        }
        __syncthreads();
      }
    return;
  }
  const bool active = tid < (1 << (logP - 4));
  uint64_t r[16];
  // A pass whose window lies below bit 10 only moves keys inside aligned groups of 1024, and a
  // group of 1024 is exactly what one wave owns in such a pass (64 threads x 16 keys).  Between
  // two such passes the waves need no workgroup barrier, only program order inside the wave (the
  // LDS serves one wave's requests in order); they drift apart and one wave's LDS traffic overlaps
  // another's compare-exchanges.  A barrier stands only around the passes with a window above bit 6.
  int prev_p = 31;
  auto pass = [&](int p, int L, int s_hi, int s_lo, int L_first, int L_last) {
    // one LDS round trip; either the stages s_hi..s_lo of level L, or (L_first > 0) all stages of
    // the levels L_first..L_last, which must all lie in the window [p, p+4)
    if (p > 6 || prev_p > 6)
      __syncthreads();
    else
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    prev_p = p;
    if (active) {
      const int base = (tid & ((1 << p) - 1)) | ((tid >> p) << (p + 4));
#pragma unroll
      for (int i = 0; i < 16; ++i) r[i] = buf[sort_phys(base | (i << p))];
      auto run = [&](int lev, int hi, int lo) {
        const int ib = (lev >= p && lev < p + 4) ? lev - p : -1;  // level bit inside the register window?
        const bool tdesc = ib >= 0 ? true : (((base >> lev) & 1) == 0);
        for (int s = hi; s >= lo; --s) {
          switch (s - p) {
            case 0: sort_stage_regs<0>(r, tdesc, ib); break;
            case 1: sort_stage_regs<1>(r, tdesc, ib); break;
            case 2: sort_stage_regs<2>(r, tdesc, ib); break;
            default: sort_stage_regs<3>(r, tdesc, ib); break;
          }
        }
      };
      if (L_first > 0)
        for (int lev = L_first; lev <= L_last; ++lev) run(lev, lev - 1, 0);
      else
        run(L, s_hi, s_lo);
#pragma unroll
      for (int i = 0; i < 16; ++i) buf[sort_phys(base | (i << p))] = r[i];
    }
  };
  pass(0, 0, 0, 0, 1, 4);  // levels 1..4 entirely in registers
  for (int L = 5; L <= logP; ++L) {
    int s = L - 1;
    while (s >= 0) {
      const int lo = s - 3 > 0 ? s - 3 : 0;
      const int p = lo < logP - 4 ? lo : logP - 4;
      pass(p, L, s, lo, 0, 0);
      s = lo - 1;
    }
  }
  __syncthreads();
}

// Collects the composites >= cut (at most P) into buf, pads to P with zeros,
// sorts descending and writes the first Zc indices to out.  buf holds
// sort_lds_bytes(P) bytes.
template <typename Source>
__device__ __forceinline__ void collect_sort_write(Source& src, uint64_t cut, int Zc, int P,
                                                   uint64_t* buf, SelectShared& sh,
                                                   int32_t* __restrict__ out) {
  const int tid = threadIdx.x;
  if (tid == 0) sh.cnt = 0;
  __syncthreads();
  src([&](float y, uint32_t i) {
    uint64_t c = composite(y, i);
    if (c >= cut) {
      int pos = atomicAdd(&sh.cnt, 1);
      if (pos < P) buf[sort_phys(pos)] = c;
    }
  });
  for (int i = Zc + tid; i < P; i += kSelThreads) buf[sort_phys(i)] = 0;
  __syncthreads();
  bitonic_sort_desc(buf, 31 - __clz(P));
  for (int i = tid; i < Zc; i += kSelThreads) out[i] = int32_t(0xffffffffu - uint32_t(buf[sort_phys(i)]));
}

// Dense fp32 row as a source; 128-bit loads on the aligned body, kUnroll of
// them in flight per thread.
struct DenseRow {
  const float* row;
  int N;
  static constexpr int kUnroll = 8;
  template <typename F>
  __device__ __forceinline__ void operator()(F f) const {
    const int tid = threadIdx.x;
    int head = int((4 - ((reinterpret_cast<uintptr_t>(row) >> 2) & 3)) & 3);
    if (head > N) head = N;
    if (tid < head) f(row[tid], uint32_t(tid));
    const int nvec = (N - head) >> 2;
    const float4* v = reinterpret_cast<const float4*>(row + head);
    for (int i0 = tid; i0 < nvec; i0 += kSelThreads * kUnroll) {
      float4 x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int i = i0 + u * kSelThreads;
        if (i < nvec) x[u] = v[i];
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int i = i0 + u * kSelThreads;
        if (i < nvec) {
          uint32_t b = uint32_t(head + 4 * i);
          f(x[u].x, b);
          f(x[u].y, b + 1);
          f(x[u].z, b + 2);
          f(x[u].w, b + 3);
        }
      }
    }
    const int tail0 = head + 4 * nvec;
    if (tail0 + tid < N) f(row[tail0 + tid], uint32_t(tail0 + tid));
  }
};

static inline int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

}  // namespace fm
