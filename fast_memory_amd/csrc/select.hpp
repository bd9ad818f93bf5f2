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
constexpr int kSelMaxBins = 2048;

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
// looking at no more than `max_passes` digits (11,11,10 value bits, then
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
  const int kBits[6] = {11, 11, 10, 11, 11, 10};
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
__host__ __device__ static inline size_t sort_lds_bytes(int P) { return size_t(P + (P >> 4) + 1) * sizeof(uint64_t); }

// The 16 keys of a thread as separate low and high words: the compare-exchange below works on
// 32-bit registers.
struct SortKeys {
  uint32_t lo[16], hi[16];
};

// Compare-exchange, larger key to slot i.  A 64-bit subtract (two full-rate instructions) leaves
// "key i < key j" in the carry, which selects the four output words; the quarter-rate 64-bit
// compare is avoided.
__device__ __forceinline__ void sort_ce(SortKeys& k, int i, int j) {
  uint32_t t, nil, nih, njl, njh;
  asm("v_sub_co_u32 %0, vcc, %5, %7\n\t"
      "v_subb_co_u32 %0, vcc, %6, %8, vcc\n\t"
      "v_cndmask_b32 %1, %5, %7, vcc\n\t"
      "v_cndmask_b32 %2, %6, %8, vcc\n\t"
      "v_cndmask_b32 %3, %7, %5, vcc\n\t"
      "v_cndmask_b32 %4, %8, %6, vcc"
      : "=&v"(t), "=&v"(nil), "=&v"(nih), "=&v"(njl), "=&v"(njh)
      : "v"(k.lo[i]), "v"(k.hi[i]), "v"(k.lo[j]), "v"(k.hi[j])
      : "vcc");
  k.lo[i] = nil;
  k.hi[i] = nih;
  k.lo[j] = njl;
  k.hi[j] = njh;
}

// One stage at register distance 2^D, descending, except that pairs whose register number has
// bit FLIP set (FLIP >= 0) sort ascending.  A direction that depends on the thread is not a case
// here: such keys are held bit-inverted (see bitonic_sort_desc), which turns it into descending.
template <int D, int FLIP>
__device__ __forceinline__ void sort_stage_regs(SortKeys& k) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (i & (1 << D)) continue;
    const int j = i | (1 << D);
    if (FLIP >= 0 && ((i >> (FLIP >= 0 ? FLIP : 0)) & 1))
      sort_ce(k, j, i);
    else
      sort_ce(k, i, j);
  }
}

__device__ __forceinline__ void sort_xor_keys(SortKeys& k, uint32_t m_low_half, uint32_t m_high_half) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t m = i < 8 ? m_low_half : m_high_half;
    k.lo[i] ^= m;
    k.hi[i] ^= m;
  }
}

__device__ __forceinline__ void bitonic_sort_desc(uint64_t* buf, int logP) {
  const int tid = threadIdx.x;
  if (logP < 6) {  // tiny: plain network, one key pair per thread step
    const int P = 1 << logP;
    for (int k = 2; k <= P; k <<= 1)
      for (int j = k >> 1; j > 0; j >>= 1) {
        for (int t = tid; t < (P >> 1); t += int(blockDim.x)) {
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
  SortKeys k;
  // Direction.  In level L a key sorts ascending if bit L of its index is set.  Instead of a
  // per-thread direction in every compare-exchange, keys of ascending positions are held
  // bit-inverted while level L runs (in registers and in LDS), so that every compare-exchange is
  // "descending".  The pattern moves from bit L-1 to bit L in the first pass of level L, where
  // bit L-1 is bit 3 of the register number and bit L a bit of the thread; in the last level bit L
  // is zero for every index and the keys come out plain.
  //
  // Barriers.  A pass whose window lies below bit 10 only moves keys inside aligned groups of 1024,
  // and a group of 1024 is exactly what one wave owns in such a pass (64 threads x 16 keys).
  // Between two such passes the waves need no workgroup barrier, only program order inside the
  // wave (the LDS serves one wave's requests in order); they drift apart and one wave's LDS traffic
  // overlaps another's compare-exchanges.  A barrier stands only around passes with a window above
  // bit 6.
  int prev_p = 31;
  auto pass = [&](int p, int L, int n_stages, bool first_of_level) {
    if (p > 6 || prev_p > 6)
      __syncthreads();
    else
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    prev_p = p;
    if (active) {
      const int base = (tid & ((1 << p) - 1)) | ((tid >> p) << (p + 4));
      // base and i << p share no bit, so phys(base | i << p) = phys(base) + phys(i << p); the second
      // term is the same for all threads and stays in scalar registers
      uint64_t* pb = buf + sort_phys(base);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint64_t v = pb[sort_phys(i << p)];
        k.lo[i] = uint32_t(v);
        k.hi[i] = uint32_t(v >> 32);
      }
      // Stage sequences are spelled out at compile time: a loop over stages makes the compiler
      // copy the 16 keys back to fixed registers after every stage.
      if (L == 0) {
        // levels 1..4 in the window [0,4): for levels 1..3 the level bit is a bit of the register
        // number; level 4 takes its direction from bit 4 of the index, a thread bit
        sort_stage_regs<0, 1>(k);
        sort_stage_regs<1, 2>(k);
        sort_stage_regs<0, 2>(k);
        sort_stage_regs<2, 3>(k);
        sort_stage_regs<1, 3>(k);
        sort_stage_regs<0, 3>(k);
        const uint32_t m = 0u - uint32_t((base >> 4) & 1);
        sort_xor_keys(k, m, m);
        sort_stage_regs<3, -1>(k);
        sort_stage_regs<2, -1>(k);
        sort_stage_regs<1, -1>(k);
        sort_stage_regs<0, -1>(k);
      } else {
        if (first_of_level) {  // window [L-4, L): pattern from bit L-1 (bit 3 of i) to bit L (thread)
          const uint32_t m = 0u - uint32_t((base >> L) & 1);
          sort_xor_keys(k, m, ~m);
        }
        switch (n_stages) {
          case 4:
            sort_stage_regs<3, -1>(k);
            sort_stage_regs<2, -1>(k);
            sort_stage_regs<1, -1>(k);
            sort_stage_regs<0, -1>(k);
            break;
          case 3:
            sort_stage_regs<2, -1>(k);
            sort_stage_regs<1, -1>(k);
            sort_stage_regs<0, -1>(k);
            break;
          case 2:
            sort_stage_regs<1, -1>(k);
            sort_stage_regs<0, -1>(k);
            break;
          default:
            sort_stage_regs<0, -1>(k);
            break;
        }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) pb[sort_phys(i << p)] = (uint64_t(k.hi[i]) << 32) | k.lo[i];
    }
  };
  pass(0, 0, 4, true);  // levels 1..4 entirely in registers
  for (int L = 5; L <= logP; ++L) {
    int s = L - 1;
    while (s >= 0) {
      const int lo = s - 3 > 0 ? s - 3 : 0;  // lo <= logP - 4: the window [lo, lo+4) fits
      pass(lo, L, s - lo + 1, s == L - 1);
      s = lo - 1;
    }
  }
  __syncthreads();
}

// Collects the composites >= cut (at most P) into buf, pads to P with zeros,
// sorts descending and writes the first Zc indices to out (and, if val_out is
// given, their values: -0 reads back as +0).  buf holds sort_lds_bytes(P) bytes.
template <typename Source>
__device__ __forceinline__ void collect_sort_write(Source& src, uint64_t cut, int Zc, int P,
                                                   uint64_t* buf, SelectShared& sh,
                                                   int32_t* __restrict__ out,
                                                   float* __restrict__ val_out = nullptr) {
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
  for (int i = Zc + tid; i < P; i += int(blockDim.x)) buf[sort_phys(i)] = 0;
  __syncthreads();
  bitonic_sort_desc(buf, 31 - __clz(P));
  for (int i = tid; i < Zc; i += int(blockDim.x)) {
    const uint64_t c = buf[sort_phys(i)];
    out[i] = int32_t(0xffffffffu - uint32_t(c));
    if (val_out) val_out[i] = key_to_float(uint32_t(c >> 32));
  }
}

// ---- selection by value bins: no radix passes, no sorting network --------------------------
// For candidate sets that are a modest superset of the answer (the fused build's ~1.2 Zc candidates per
// row).  The value keys are cut into up to kSelBins equal-width bins over [min, max] of the row (a shift,
// so between kSelBins / 2 and kSelBins bins are in use), descending; one histogram (16-bit counters packed
// two to a word) and a scan give every bin's first output position and the bin that holds the Zc-th
// element; the candidates of the bins up to that one are scattered into their bins' slots (any order), and
// every element's final position is its bin's start plus the number of larger composites in its bin,
// counted by brute force: a bin holds a few elements, a dozen next to the cut where the values are densest.
// Composites are unique, so the positions are a permutation and the result is exactly "value descending,
// index ascending".
// Returns false, with nothing written, when a bin is longer than kSelMaxBin (many equal or nearly equal
// values): the caller then takes the radix select and the sorting network.
// (Measured at 16384-entry lists, 16384 rows: 8192 bins instead of 4096 and four bin members fetched per
// round of the counting loop take the selection from 2.55 to 2.32 ms; rounds that read past the end of their
// bin without clamping or masking -- what lies there compares as smaller -- to 1.88 ms, of which the counting
// loop is 0.55 ms, the read of the candidates 0.63 ms.  A second level of bins that splits the dense ones
// into sub-bins of about 8 members costs more in its extra passes, 0.4 ms, than it saves.)
constexpr int kSelBinBits = 13;
constexpr int kSelBins = 1 << kSelBinBits;
constexpr int kSelMaxBin = 256;
// LDS of the selection for lists of Zc entries: the composites, then the packed counters
constexpr size_t binned_lds_bytes(int Zc) { return size_t(Zc + kSelMaxBin) * sizeof(uint64_t) + size_t(kSelBins) * 2; }

struct BinShared {
  uint32_t red_min[16], red_max[16];
  int scan_tmp[17];
  int cut_bin, n_keep, max_bin;
};

// buf holds Zc + kSelMaxBin composites, hist kSelBins / 2 words.
template <int NT, typename Source>
__device__ __forceinline__ bool binned_select_write(Source& src, int Zc, uint64_t* buf, uint32_t* hist,
                                                    BinShared& bs, int32_t* __restrict__ out,
                                                    float* __restrict__ val_out) {
  static_assert(NT >= 256 && NT <= 1024 && kSelBins % (2 * NT) == 0, "threads per row");
  const int tid = threadIdx.x, w = tid >> 6;
  constexpr int nw = NT / 64;
  uint32_t mn = 0xffffffffu, mx = 0u;
  src([&](float y, uint32_t) {
    const uint32_t k = float_key(y);
    mn = min(mn, k);
    mx = max(mx, k);
  });
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = min(mn, uint32_t(__shfl_xor(int(mn), o)));
    mx = max(mx, uint32_t(__shfl_xor(int(mx), o)));
  }
  if (lane_id() == 0) {
    bs.red_min[w] = mn;
    bs.red_max[w] = mx;
  }
  for (int i = tid; i < kSelBins / 2; i += NT) hist[i] = 0;
  if (tid == 0) {
    bs.max_bin = 0;
    bs.cut_bin = -1;
    bs.n_keep = 0;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < nw; ++i) {
    mn = min(mn, bs.red_min[i]);
    mx = max(mx, bs.red_max[i]);
  }
  if (mx < mn) return false;  // no candidate at all
  const uint32_t range1 = mx - mn;
  const int hb = range1 ? 32 - __clz(int(range1)) : 0;
  const int shift = hb > kSelBinBits ? hb - kSelBinBits : 0;
  const uint32_t top = range1 >> shift;  // < kSelBins
  auto dbin = [&](uint32_t k) { return int(top - ((k - mn) >> shift)); };  // 0 = the largest values
  // the 16-bit counter of bin d is half d % 2 of word d / 2 (a row has at most 32 candidates per thread, so
  // neither a count nor an offset reaches 65536 and no half carries into its neighbour)
  auto half_of = [&](int d) { return int((hist[d >> 1] >> (16 * (d & 1))) & 0xffffu); };
  src([&](float y, uint32_t) {
    const int d = dbin(float_key(y));
    atomicAdd(&hist[d >> 1], 1u << (16 * (d & 1)));
  });
  __syncthreads();
  {
    constexpr int per = kSelBins / NT;  // even
    int h[per], local = 0;
#pragma unroll
    for (int j = 0; j < per; j += 2) {
      const uint32_t x = hist[(tid * per + j) >> 1];
      h[j] = int(x & 0xffffu);
      h[j + 1] = int(x >> 16);
      local += h[j] + h[j + 1];
    }
    int total;
    int running = block_excl_scan(local, bs.scan_tmp, &total);
    int longest = 0;
    uint32_t pack = 0;
#pragma unroll
    for (int j = 0; j < per; ++j) {
      if (running < Zc) {
        longest = max(longest, h[j]);
        if (Zc <= running + h[j]) {
          bs.cut_bin = tid * per + j;
          bs.n_keep = running + h[j];
        }
      }
      if (j & 1)
        hist[(tid * per + j) >> 1] = pack | (uint32_t(running) << 16);
      else
        pack = uint32_t(running);
      running += h[j];
    }
    if (longest > kSelMaxBin - 4) atomicMax(&bs.max_bin, longest);  // (four places stay free behind the kept ones)
  }
  __syncthreads();
  const int cut_bin = bs.cut_bin, n_keep = bs.n_keep;
  if (cut_bin < 0 || bs.max_bin > kSelMaxBin - 4) return false;  // fewer than Zc candidates, or a long bin
  if (tid < 4) buf[n_keep + tid] = 0;  // smaller than any composite: what a rank round reads past the last bin
  src([&](float y, uint32_t i) {
    const int d = dbin(float_key(y));
    if (d <= cut_bin) {
      const uint32_t old = atomicAdd(&hist[d >> 1], 1u << (16 * (d & 1)));
      buf[(old >> (16 * (d & 1))) & 0xffffu] = composite(y, i);
    }
  });
  __syncthreads();
  // the counter of bin d is now the end of bin d (for d <= cut_bin), i.e. the start of bin d + 1
  for (int p = tid; p < n_keep; p += NT) {
    const uint64_t c = buf[p];
    const uint32_t clo = uint32_t(c), chi = uint32_t(c >> 32);
    const int d = dbin(chi);
    const int s0 = d ? half_of(d - 1) : 0, e0 = half_of(d);
    int rank = s0;
    // rank += (c < o) for the bin's members o: the borrow of the 64-bit subtraction c - o, two full-rate
    // instructions.  Four members per round, fetched before the first is used.  A round's reads past the
    // bin's end need no mask: what follows in the buffer are the members of the bins after it, all smaller
    // than c, and behind the last bin four zeros.
    for (int q = s0; q < e0; q += 4) {
      uint64_t o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = buf[q + i];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t t;
        asm("v_sub_co_u32 %0, vcc, %2, %4\n\t"
            "v_subb_co_u32 %0, vcc, %3, %5, vcc\n\t"
            "v_addc_co_u32 %1, vcc, 0, %1, vcc"
            : "=&v"(t), "+v"(rank)
            : "v"(clo), "v"(chi), "v"(uint32_t(o[i])), "v"(uint32_t(o[i] >> 32))
            : "vcc");
      }
    }
    if (rank < Zc) {
      out[rank] = int32_t(0xffffffffu - clo);
      if (val_out) val_out[rank] = key_to_float(chi);
    }
  }
  return true;
}

// Dense fp32 row as a source; 128-bit loads on the aligned body, kUnroll of
// them in flight per thread.
template <int NT = kSelThreads>
struct DenseRowT {
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
    for (int i0 = tid; i0 < nvec; i0 += NT * kUnroll) {
      float4 x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int i = i0 + u * NT;
        if (i < nvec) x[u] = v[i];
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int i = i0 + u * NT;
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
  // Half h (0 or 1) of the row: every other round of the loop above (rounds of NT * kUnroll * 4 elements,
  // interleaved so that a trend along the row lands in both halves alike); the unaligned head and tail
  // belong to half 0.
  template <typename F>
  __device__ __forceinline__ void half(int h, F f) const {
    const int tid = threadIdx.x;
    int head = int((4 - ((reinterpret_cast<uintptr_t>(row) >> 2) & 3)) & 3);
    if (head > N) head = N;
    if (h == 0 && tid < head) f(row[tid], uint32_t(tid));
    const int nvec = (N - head) >> 2;
    const float4* v = reinterpret_cast<const float4*>(row + head);
    for (int i0 = tid + h * NT * kUnroll; i0 < nvec; i0 += 2 * NT * kUnroll) {
      float4 x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int i = i0 + u * NT;
        if (i < nvec) x[u] = v[i];
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        int i = i0 + u * NT;
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
    if (h == 0 && tail0 + tid < N) f(row[tail0 + tid], uint32_t(tail0 + tid));
  }
};

using DenseRow = DenseRowT<>;

static inline int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

}  // namespace fm
