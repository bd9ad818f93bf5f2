// Arg-top-Z over the rows of an fp32 matrix (memory.py:273, triton_kernel.py:278).
//
// Contract: output row r lists the min(Z,N) indices of the largest entries of
// Y[r,:], ordered by (value descending, index ascending); -0 == +0, NaN is the
// largest value.
//
// One workgroup per row.  Two ways to the same result:
//  * sampled (long rows): 1/16 of the row is read as whole 128-byte
//    lines spread over the row and kept in registers; the sample's value of rank
//    mu + 4 sqrt(mu) + 3 (mu = Z n_sample / N) is a threshold that at least Z
//    elements of the row reach in all but about one row in 30 000.  ONE read of
//    the row then collects the elements that reach it into LDS (about 1.3-1.6 Z),
//    and the exact cut, the sort and the output run on those.  HBM traffic: 1.06
//    reads of the row.
//  * exact passes (every other shape, and any row whose sample misled: fewer than
//    Z or more than the buffer's capacity collected, e.g. rows of mostly equal
//    values): radix select of the Zc-th largest composite, each pass re-reading
//    the row and histogramming one digit in LDS, stopping as soon as the bin that
//    holds the cut is wanted whole; one more read collects the exactly Zc
//    survivors.  HBM traffic: (passes + 1) reads of the row, typically 4.
// Then the bitonic sort in LDS, indices (and values) out.  The result does not
// depend on which way a row took.  LDS: max(8 pow2(Zc) * 17/16, 8 cap) + 16 KiB.
#include "select.hpp"

namespace fm {

std::atomic<bool> g_argtopz_exact_only{false};  // test hook: fm_debug_argtopz_exact_only

constexpr int kSampleRegs = 32;  // sampled elements per thread: samples of up to 32768 elements
constexpr int kCollectRegs = 16; // collected candidates per thread: capacity up to 16384
constexpr int kCollectRegsWide = 24;  // ... of the form for lists longer than 8192: up to 24576

struct SamplePlan {
  int n_lines;      // sampled 128-byte lines (32 floats each); 0 = exact passes only
  int line_stride;  // in lines
  int rank;
  int cap;          // candidates the LDS buffer takes
};

// `wide`: the form that buffers candidate indices only (lists longer than 8 * nt).
static SamplePlan sample_plan(int N, int Zc, int P, int nt, bool wide = false) {
  SamplePlan p{0, 0, 0, 0};
  if (N < 65536 || int64_t(Zc) * 8 > N || (P > 8 * nt) != wide) return p;
  const int lines = N / 32;                         // whole lines only; a ragged tail is never sampled
  int stride = 16;
  while (lines / stride > kSampleRegs * nt / 32) stride *= 2;
  const int n_lines = lines / stride;
  const double ns = 32.0 * n_lines;
  const double mu = double(Zc) * ns / N;
  const int rank = int(mu + 4.0 * sqrt(mu) + 3.0);
  const double m_exp = double(rank) * N / ns, m_sd = double(N) / ns * sqrt(double(rank));
  int cap;
  if (wide) {
    cap = kCollectRegsWide * nt;                    // what the registers take; LDS holds half of them at a time
  } else {
    cap = 2 * P;
    while (cap < m_exp + 5.0 * m_sd && cap < kCollectRegs * nt) cap *= 2;
  }
  if (cap < m_exp + 5.0 * m_sd || rank * 4 > ns) return p;
  p.n_lines = n_lines;
  p.line_stride = stride;
  p.rank = rank;
  p.cap = cap;
  return p;
}

// The sampled lines of a row, in registers.
template <int NT>
struct SampleRegs {
  float v[kSampleRegs];
  int n;
  template <typename F>
  __device__ __forceinline__ void operator()(F f) const {
#pragma unroll
    for (int r = 0; r < kSampleRegs; ++r)
      if (r < n) f(v[r], uint32_t(threadIdx.x + r * NT));
  }
};

// Candidates collected in LDS, dealt to the threads' registers as composites.
template <int CR>
struct CollectedRegs {
  uint64_t c[CR];
  int n;
  template <typename F>
  __device__ __forceinline__ void operator()(F f) const {
#pragma unroll
    for (int r = 0; r < CR; ++r)
      if (r < n) f(key_to_float(uint32_t(c[r] >> 32)), 0xffffffffu - uint32_t(c[r]));
  }
};

// The same for candidates collected in two rounds (the two halves of a row): registers 0 .. CR/2 - 1 hold a
// thread's share of the first round, the others its share of the second.
template <int CR>
struct CollectedHalves {
  uint64_t c[CR];
  int n0, n1;
  template <typename F>
  __device__ __forceinline__ void operator()(F f) const {
#pragma unroll
    for (int r = 0; r < CR; ++r)
      if (r < CR / 2 ? r < n0 : r - CR / 2 < n1) f(key_to_float(uint32_t(c[r] >> 32)), 0xffffffffu - uint32_t(c[r]));
  }
};

// row_map / n_rows_dev are optional: when given, workgroup b works on input row
// b and writes output row row_map[b], and exits if b >= min(*n_rows_dev, grid).
template <int NT, bool WIDE = false>
__global__ __launch_bounds__(NT) void argtopz_kernel(
    const float* __restrict__ Y, int N, int64_t ldy, int Zc, int P, int32_t* __restrict__ idx_out,
    float* __restrict__ val_out, const int32_t* __restrict__ row_map, const int32_t* __restrict__ n_rows_dev,
    SamplePlan sp, int sh_off) {
  // dynamic LDS: [P composites in the sort's layout, or before that up to sp.cap candidates | SelectShared];
  // the binned selection of the sampled path reuses all of it as [Zc + kSelMaxBin composites | histogram]
  extern __shared__ uint64_t buf[];
  __shared__ BinShared bs;
  SelectShared& sh = *reinterpret_cast<SelectShared*>(reinterpret_cast<char*>(buf) + sh_off);
  if (n_rows_dev && int(blockIdx.x) >= *n_rows_dev) return;
  const int64_t out_row = row_map ? row_map[blockIdx.x] : int64_t(blockIdx.x);
  const float* row = Y + int64_t(blockIdx.x) * ldy;
  int32_t* out = idx_out + out_row * Zc;
  float* vout = val_out ? val_out + out_row * Zc : nullptr;
  DenseRowT<NT> src{row, N};
  if (sp.n_lines > 0) {
    const int tid = threadIdx.x;
    SampleRegs<NT> smp;
    const int n_s = sp.n_lines * 32;
    smp.n = tid < n_s ? (n_s - tid + NT - 1) / NT : 0;
#pragma unroll
    for (int r = 0; r < kSampleRegs; ++r) {
      const int j = tid + r * NT;  // sample element j = element (j % 32) of sampled line j / 32
      if (r < smp.n) smp.v[r] = row[(int64_t(j >> 5) * sp.line_stride << 5) + (j & 31)];
    }
    const uint64_t tau = radix_select_cut<NT>(smp, sp.rank, 3, sh) & 0xffffffff00000000ull;  // value bits only
    // tau has value bits only, so "composite >= tau" is a comparison of values: one float compare per
    // element of the row (NaN, the largest key, passes: it is not below anything)
    const float tau_f = key_to_float(uint32_t(tau >> 32));
    if constexpr (WIDE) {
      // Lists longer than 8 * NT: the candidates (about 1.2 Zc) do not fit LDS as composites all at once, so the
      // row is taken in two interleaved halves; each half's candidates go to LDS as composites (sp.cap / 2
      // slots) and from there to the threads' registers, which hold them all.  (Buffering indices only and fetching the
      // candidates' values again afterwards moved a 128-byte line per candidate: 0.47 x the row once more.)
      constexpr int CR = kCollectRegsWide;
      CollectedHalves<CR> cr;
      const int cap_h = sp.cap / 2;  // = CR / 2 * NT
      int m_all = 0;
      bool fits = true;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if (tid == 0) sh.cnt = 0;
        __syncthreads();
        src.half(h, [&](float y, uint32_t i) {
          if (!(y < tau_f)) {
            const int pos = atomicAdd(&sh.cnt, 1);
            if (pos < cap_h) buf[pos] = composite(y, i);
          }
        });
        __syncthreads();
        const int m = sh.cnt;
        m_all += m;
        fits = fits && m <= cap_h;
        const int mine = tid < m ? (min(m, cap_h) - tid + NT - 1) / NT : 0;
        if (h == 0)
          cr.n0 = mine;
        else
          cr.n1 = mine;
#pragma unroll
        for (int r = 0; r < CR / 2; ++r)
          if (r < mine) cr.c[h * (CR / 2) + r] = buf[tid + r * NT];
        __syncthreads();  // every candidate of the half is in registers before the buffer is written again
      }
      // (a row whose candidates the binned selection declines, e.g. thousands of equal values around the cut,
      // goes on to the exact passes below like one the sample misled)
      if (fits && m_all >= Zc &&
          binned_select_write<NT>(cr, Zc, buf, reinterpret_cast<uint32_t*>(buf + (Zc + kSelMaxBin)), bs, out, vout))
        return;
    } else {
      if (tid == 0) sh.cnt = 0;
      __syncthreads();
      src([&](float y, uint32_t i) {
        if (!(y < tau_f)) {
          const int pos = atomicAdd(&sh.cnt, 1);
          if (pos < sp.cap) buf[pos] = composite(y, i);
        }
      });
      __syncthreads();
      const int m = sh.cnt;
      if (m >= Zc && m <= sp.cap) {
        constexpr int CR = kCollectRegs;
        CollectedRegs<CR> cr;
        cr.n = tid < m ? (m - tid + NT - 1) / NT : 0;
#pragma unroll
        for (int r = 0; r < CR; ++r)
          if (r < cr.n) cr.c[r] = buf[tid + r * NT];
        __syncthreads();  // every candidate is in registers before the buffer is written again
        if (binned_select_write<NT>(cr, Zc, buf, reinterpret_cast<uint32_t*>(buf + (Zc + kSelMaxBin)), bs, out, vout))
          return;
        __syncthreads();
        const uint64_t cut = radix_select_cut<NT>(cr, Zc, 6, sh);
        collect_sort_write(cr, cut, Zc, P, buf, sh, out, vout);
        return;
      }
    }
    __syncthreads();  // every thread has read sh.cnt before the exact passes reuse it
  }
  const uint64_t cut = radix_select_cut<NT>(src, Zc, 6, sh);
  collect_sort_write(src, cut, Zc, P, buf, sh, out, vout);
}

// ---- lists longer than FM_MAX_Z ------------------------------------------------------------------
// The Zc survivors do not fit LDS.  Per row: the exact cut by radix passes over the row (as above), the
// exactly Zc composites >= cut collected into a slot of the caller's workspace, padded to a power of two,
// and a plain bitonic network over that slot in global memory (it stays in L2: 8 bytes per entry).  A
// workgroup owns one slot and walks rows blockIdx.x, blockIdx.x + gridDim.x, ...  Slow next to the LDS
// forms (about a millisecond per row of 65536) and without any limit on Z or on the values.
constexpr int kBigSlots = 1024;  // workgroups, and workspace slots, of a launch

__global__ __launch_bounds__(kSelThreads) void argtopz_big_kernel(const float* __restrict__ Y, int64_t rows, int N,
                                                                  int64_t ldy, int Zc, int P,
                                                                  int32_t* __restrict__ idx_out,
                                                                  float* __restrict__ val_out,
                                                                  uint64_t* __restrict__ slots) {
  __shared__ SelectShared sh;
  uint64_t* buf = slots + int64_t(blockIdx.x) * P;
  const int tid = threadIdx.x;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    DenseRowT<kSelThreads> src{Y + row * ldy, N};
    const uint64_t cut = radix_select_cut<kSelThreads>(src, Zc, 6, sh);
    if (tid == 0) sh.cnt = 0;
    __syncthreads();
    src([&](float y, uint32_t i) {
      const uint64_t c = composite(y, i);
      if (c >= cut) {
        const int pos = atomicAdd(&sh.cnt, 1);
        if (pos < P) buf[pos] = c;
      }
    });
    for (int i = Zc + tid; i < P; i += kSelThreads) buf[i] = 0;
    __syncthreads();
    for (int k = 2; k <= P; k <<= 1)
      for (int j = k >> 1; j > 0; j >>= 1) {
        for (int t = tid; t < (P >> 1); t += kSelThreads) {
          const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
          const int q = i | j;
          const uint64_t a = buf[i], b = buf[q];
          const bool desc = (i & k) == 0;
          if (desc ? (a < b) : (a > b)) {
            buf[i] = b;
            buf[q] = a;
          }
        }
        __syncthreads();
      }
    for (int i = tid; i < Zc; i += kSelThreads) {
      const uint64_t c = buf[i];
      idx_out[row * Zc + i] = int32_t(0xffffffffu - uint32_t(c));
      if (val_out) val_out[row * Zc + i] = key_to_float(uint32_t(c >> 32));
    }
    __syncthreads();  // the slot and sh are reused by the next row
  }
}

size_t argtopz_big_workspace(int64_t rows, int Zc) {
  if (Zc <= FM_MAX_Z || rows < 1) return 0;
  return size_t(std::min<int64_t>(rows, kBigSlots)) * size_t(next_pow2(Zc)) * sizeof(uint64_t);
}

int launch_argtopz_big(const float* Y, int64_t rows, int N, int64_t ldy, int Zc, int32_t* idx_out, float* val_out,
                       void* ws, size_t ws_bytes, hipStream_t st) {
  FM_REQUIRE(ws && ws_bytes >= argtopz_big_workspace(rows, Zc), FM_ERR_WORKSPACE,
             "arg-top-Z with min(Z, N) = %d > FM_MAX_Z needs a workspace of %zu bytes (fm_argtopz_workspace), got %zu", Zc,
             argtopz_big_workspace(rows, Zc), ws_bytes);
  hipLaunchKernelGGL(argtopz_big_kernel, dim3(unsigned(std::min<int64_t>(rows, kBigSlots))), dim3(kSelThreads), 0, st, Y,
                     rows, N, ldy, Zc, next_pow2(Zc), idx_out, val_out, static_cast<uint64_t*>(ws));
  return launch_status("argtopz(big)");
}

int launch_argtopz(const float* Y, int64_t rows, int N, int64_t ldy, int Zc, int32_t* idx_out, float* val_out,
                   const int32_t* row_map, const int32_t* n_rows_dev, hipStream_t st) {
  const int P = next_pow2(Zc);
  // Two 512-thread workgroups share a CU where one of 1024 threads would have it alone: one row's
  // sort overlaps the other's read.  The narrow form needs the sampled path (its registers then hold
  // all a thread keeps) and lists of at most 4096.
  SamplePlan sp = sample_plan(N, Zc, P, 512);
  const bool narrow = sp.n_lines > 0 && !g_argtopz_exact_only;
  bool wide = false;
  if (!narrow) {
    sp = g_argtopz_exact_only ? SamplePlan{0, 0, 0, 0} : sample_plan(N, Zc, P, kSelThreads);
    if (sp.n_lines == 0 && !g_argtopz_exact_only) {
      sp = sample_plan(N, Zc, P, kSelThreads, true);
      wide = sp.n_lines > 0;
    }
  }
  // SelectShared sits behind the sort buffer / the candidate buffer; the binned selection needs its own extent
  const size_t sh_off = align_up(std::max(sort_lds_bytes(P), (wide ? size_t(sp.cap) / 2 : size_t(sp.cap)) * sizeof(uint64_t)), 16);
  const auto lds_for = [](size_t off, int zc, bool sampled) {
    const size_t binned = sampled ? binned_lds_bytes(zc) : 0;
    return std::max(off + sizeof(SelectShared), binned);
  };
  const size_t lds = lds_for(sh_off, Zc, sp.n_lines > 0);
  const size_t lds_max = lds_for(align_up(std::max(sort_lds_bytes(FM_MAX_Z), size_t(kCollectRegsWide) / 2 * kSelThreads * sizeof(uint64_t)), 16),
                                 FM_MAX_Z, true);
  if (narrow) {
    FM_ALLOW_LDS(argtopz_kernel<512>, lds_max, "argtopz: lds");
    hipLaunchKernelGGL(argtopz_kernel<512>, dim3(unsigned(rows)), dim3(512), lds, st, Y, N, ldy, Zc, P, idx_out,
                       val_out, row_map, n_rows_dev, sp, int(sh_off));
  } else if (wide) {
    FM_ALLOW_LDS((argtopz_kernel<kSelThreads, true>), lds_max, "argtopz: lds");
    hipLaunchKernelGGL((argtopz_kernel<kSelThreads, true>), dim3(unsigned(rows)), dim3(kSelThreads), lds, st, Y, N,
                       ldy, Zc, P, idx_out, val_out, row_map, n_rows_dev, sp, int(sh_off));
  } else {
    FM_ALLOW_LDS(argtopz_kernel<kSelThreads>, lds_max, "argtopz: lds");
    hipLaunchKernelGGL(argtopz_kernel<kSelThreads>, dim3(unsigned(rows)), dim3(kSelThreads), lds, st, Y, N, ldy, Zc,
                       P, idx_out, val_out, row_map, n_rows_dev, sp, int(sh_off));
  }
  return launch_status("argtopz");
}

}  // namespace fm

extern "C" size_t fm_argtopz_workspace(int64_t rows, int N, int Z) {
  if (rows < 1 || N < 1 || Z < 1) return 0;
  return fm::argtopz_big_workspace(rows, Z < N ? Z : N);
}

extern "C" void fm_debug_argtopz_exact_only(int on) {
  if (fm::debug_hooks_enabled()) fm::g_argtopz_exact_only = on != 0;
}

extern "C" int fm_argtopz_f32(const float* Y, int64_t rows, int N, int64_t ldy, int Z,
                              int32_t* idx_out, float* val_out, void* ws, size_t ws_bytes, void* stream) {
  using namespace fm;
  FM_REQUIRE(rows >= 0 && N >= 1 && Z >= 1, FM_ERR_ARG, "fm_argtopz_f32: rows=%lld N=%d Z=%d",
             (long long)rows, N, Z);
  FM_REQUIRE(ldy >= N, FM_ERR_ARG, "fm_argtopz_f32: ldy=%lld < N=%d", (long long)ldy, N);
  if (rows == 0) return FM_OK;
  FM_REQUIRE(Y && idx_out, FM_ERR_ARG, "fm_argtopz_f32: null pointer");
  FM_REQUIRE(rows <= 0x7fffffffLL, FM_ERR_UNSUPPORTED, "fm_argtopz_f32: too many rows");
  const int Zc = Z < N ? Z : N;
  if (Zc > FM_MAX_Z)  // lists that do not fit LDS: sorted in the workspace
    return launch_argtopz_big(Y, rows, N, ldy, Zc, idx_out, val_out, ws, ws_bytes, as_stream(stream));
  return launch_argtopz(Y, rows, N, ldy, Zc, idx_out, val_out, nullptr, nullptr, as_stream(stream));
}
