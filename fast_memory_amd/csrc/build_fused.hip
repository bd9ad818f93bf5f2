// Fused index build (memory.py:260-278 on one device) that never writes the
// projection Y = A.K^T to memory.
//
//   phase 0  per-row threshold.  Y is computed for a strided sample of the keys
//            (every `stride`-th key, 32 Ki - 64 Ki of them) with the ordinary
//            projection kernel, and the `rank`-th largest sampled value of every
//            (head, bucket) row becomes that row's threshold tau; `rank` sits four
//            standard deviations above Z*ns/N, so all but about one row in 30000
//            have at least Z keys reaching tau, and not many more than Z.
//   phase 1  fused_filter_kernel: bf16 MFMA GEMM over all keys with an epilogue
//            that keeps only elements >= tau.  Keys are the M side of the MFMA
//            tile and buckets the N side, so in the accumulator layout one lane
//            owns one bucket column: its threshold, its write cursor and its
//            private segment of the row's candidate buffer live in registers and
//            survivors are appended with plain stores -- no atomics.
//   phase 2  cand_select_kernel: exact top-Z (value desc, index asc) of each
//            row's candidates: radix select + in-LDS bitonic sort, the same code
//            as the dense arg-top-Z kernel, on ~1.2 Z candidates that are read
//            once and then held in registers, instead of the N-element row.
//   phase 3  repair.  A row whose candidate count fell short of Z or overflowed
//            a segment is listed by phase 2; its Y row is recomputed (same MFMA
//            instruction and contraction order) into a small buffer and handed to
//            the dense arg-top-Z kernel.  Up to kMaxRepair rows are repaired on
//            the device; status_dev reports how many were, and how many were left
//            (the caller then falls back to the unfused build).
//
// Results are bit-identical to fm_project + fm_argtopz_f32: both compute every Y
// element with v_mfma_f32_32x32x16_bf16 in ascending 16-element steps with keys
// on the A operand (the third form of phase 1 with v_mfma_f32_16x16x32 in ascending
// 32-element steps, which gives the same sums: the tests compare all forms).
//
// Roofline of phase 1: MFMA, 2*d flops per (key, bucket) pair; K is re-read once
// per 512-bucket slab from L2.  Phases 0, 2, 3 are HBM/L2-bound and small.
#include <atomic>
#include <type_traits>

#include "mfma_tile.hpp"
#include "mma16.hpp"
#include "select.hpp"

namespace fm {

int launch_argtopz(const float* Y, int64_t rows, int N, int64_t ldy, int Zc, int32_t* idx_out, float* val_out,
                   const int32_t* row_map, const int32_t* n_rows_dev, hipStream_t st);

// 0 = the plan decides, 1 = never the form with the epilogue between the MFMAs (tests compare the two)
std::atomic<int> g_fused_filter_form{0};

constexpr int kFD = 128;          // head dimension the fused kernels are built for
constexpr int kFWaves = 8;        // compute waves per workgroup
constexpr int kFThreads = 576;    // + one producer wave
constexpr int kFKeys = 64;        // keys per iteration of a workgroup
constexpr int kFSlab = 512;       // buckets per workgroup (64 per wave)
constexpr int kFLd = kFD + 8;     // LDS row stride in bf16 elements
constexpr int kFDumpLd = 20;      // floats per lane in the dump: 16 registers + 4 (16-byte stores spread over banks)
constexpr int kMaxRepair = 64;
// The sampled threshold is the value of rank mu + kRankSigmas*sqrt(mu) + 3 of the sample (mu = Z*ns/N).
// Four standard deviations: a row misses with probability ~3e-5, i.e. about one repaired row in two
// builds of 16384 rows, and ~18 % more candidates than Z are kept at mu = 512 (six would keep 27 %).
constexpr double kRankSigmas = 4.0;

// Rank (from the top) of the sample value that serves as a row's threshold.  The share of a row's keys above
// the sample's r-th largest value spreads around r / ns by sqrt(r) / ns, so the threshold keeps fewer than Z
// keys (the row is then repaired) with the probability of (r - mu) / sqrt(r) standard deviations, mu = Z ns / N.
// The rank is mu + 4 sqrt(mu) + 3, raised where that is not enough for the build's rows: with small mu the
// 4 sqrt(mu) are fewer than 3.5 deviations of sqrt(r), and a build of many rows needs more of them to leave
// the expected number of repaired rows at about four (64 can be repaired).
// Room, in standard deviations, for the number of candidates a threshold of that rank lets through: five, and
// more for a small rank, whose count (a Gamma variable of that shape) has a long upper tail (at rank 11 one row
// in a thousand exceeded five deviations).
static double room_sigmas(int rank) { return 5.0 + 6.0 / sqrt(double(std::max(rank, 1))); }

static int threshold_rank(double mu, double rows) {
  const double base = mu + kRankSigmas * sqrt(mu) + 3.0;
  const double lp = 2.0 * log(std::max(rows, 64.0) / 4.0);                       // tail 4 / rows
  const double z = std::min(6.0, std::max(3.0, sqrt(lp - log(lp) - 1.8379)));    // its normal quantile
  const double need = mu + 0.5 * z * z + z * sqrt(mu + 0.25 * z * z);            // (r - mu) / sqrt(r) = z
  return int(std::max(base, need));
}

constexpr int kCandRegs = 28;       // candidates a thread of the selection holds, 1024 threads per row
constexpr int kCandRegsSmall = 32;  // ... with 256 or 512 threads per row

struct FusedPlan {
  int ns, stride, rank, n_splits, slabs, n_writers, cap_w, sel_threads;
  bool wide;  // phase 1 takes fused_filter_wide_kernel (slabs of 1024 buckets)
  int ping;   // ... or fused_filter_ping_kernel, in its form 1, 2 or 3 (rounds and passes of the emission); 0 = not
  int64_t ld_s, ldy;
  size_t off_Ks, off_Ys, off_tau, off_cand, off_cnt, off_fail, off_nfail, off_Yf, total;
};

static bool fused_plan(int H, int C, int N, int d, int Z, int dtype, FusedPlan& p) {
  if ((dtype != FM_BF16 && dtype != FM_F16) || d != kFD) return false;
  if (N < 16384 || int64_t(Z) * 8 > N || Z > FM_MAX_Z || Z < 64) return false;  // (the smallest sample is a quarter of 16384 keys)
  // the wide form wherever its 1024-bucket slabs are at least three quarters full
  p.wide = C >= 768 && (C % 1024 == 0 || C % 1024 >= 768 || C >= 4096);
  p.slabs = int(ceil_div(C, p.wide ? 1024 : kFSlab));
  const int64_t ntiles = ceil_div(N, kFKeys);
  int64_t s = ceil_div(256, int64_t(H) * p.slabs);
  s = std::max<int64_t>(1, std::min<int64_t>(32, std::min(s, ntiles)));
  p.n_splits = int(s);
  p.n_writers = 2 * p.n_splits;
  p.ping = 0;
  // Sample size and threads per row of the selection.  A smaller sample makes phase 0 cheaper and the
  // threshold noisier: a row keeps m = rank*stride +- stride*sqrt(rank) candidates, which the
  // selection must hold in registers (R per thread, T = NT / n_writers threads per writer segment,
  // whose share of m spreads by another sqrt).  The sort keeps 16 keys per thread, so P/16 threads
  // are all it can use; fewer threads per row let several rows share a CU.  Of the samples that leave
  // five standard deviations of room or more (room_sigmas; each with the fewest threads that do), take the one with the
  // least expected work; if none does, the large sample with 1024 threads (rows that do not fit are
  // repaired).
  const int P = next_pow2(Z);
  bool found = false;
  double m_exp = 0;
  auto search = [&]() {
    found = false;
    // Among the samples whose candidates the selection holds in registers, the one with the least expected work:
    // phase 0 costs per sampled key and row, the filter's emission and the selection per candidate and row
    // (measured on the 262 144- and the 1 M-key workloads: about 2.7 ps against 10 ps).  A short memory takes
    // a small sample (a 16 K sample would be a quarter of its keys and phase 0 a quarter of the projection), a
    // long one with long lists the 16 K sample that keeps fewer candidates.
    double best = 0;
    int best_ns = 0, best_nt = 0;
    for (int ns_try : {4096, 8192, 16384, 32768, 65536, 131072}) {  // the last two for memories of millions of keys
      const int stride = N / ns_try;
      if (stride < 1) continue;
      const int ns = N / stride;
      const double mu = double(Z) * ns / N;
      const int rank = threshold_rank(mu, double(H) * C);
      if (rank * 4 > ns) continue;
      const double m = double(rank) * N / ns;
      const double per_w = m / p.n_writers;
      const double sd_w = sqrt(pow(double(N) / ns * sqrt(double(rank)) / p.n_writers, 2) + per_w);
      int nt_ok = 0;
      for (int nt = 256; nt <= kSelThreads && !nt_ok; nt *= 2)
        if (nt * 16 >= P &&
            (nt / p.n_writers) * (nt < kSelThreads ? kCandRegsSmall : kCandRegs) >= per_w + room_sigmas(rank) * sd_w)
          nt_ok = nt;
      if (!nt_ok) continue;
      const double cost = 2.7 * ns + 10.0 * m;
      if (!found || cost < best) {
        found = true;
        best = cost;
        best_ns = ns_try;
        best_nt = nt_ok;
      }
    }
    const int ns_take = found ? best_ns : 32768;  // none fits: the large sample, rows that do not fit are repaired
    p.stride = std::max(1, N / ns_take);
    p.ns = N / p.stride;
    const double mu = double(Z) * p.ns / N;
    p.rank = threshold_rank(mu, double(H) * C);
    if (p.rank * 4 > p.ns) return false;
    m_exp = double(p.rank) * N / p.ns;
    p.sel_threads = found ? best_nt : kSelThreads;
    return true;
  };
  // The form with the epilogue between the MFMAs where the wide form applies: a writer is a key split there.
  // Its emission handles a lane's first NR candidates of a group (16 keys x 128 buckets) and the group's first
  // ND * 64 in straight-line code; the forms are (NR, ND) = (4, 1), (6, 2), (7, 3), picked so that 3.5
  // standard deviations of a group's candidates fit the passes.
  const int forced = g_fused_filter_form.load(std::memory_order_relaxed);  // 1: not this form; 2, 3, 4: its ND = 1, 2, 3
  if (p.wide && forced != 1) {
    // With few rows (one or two KV heads: a GPU's share of a model sharded by head) 32 key splits leave most
    // compute units without a workgroup: up to 64 then, a writer each, where the selection's registers still
    // hold a writer's candidates with room (found); otherwise the splits chosen above.
    const int base_splits = p.n_splits;
    const int more_splits = int(std::max<int64_t>(1, std::min<int64_t>(64, std::min(ceil_div(256, int64_t(H) * p.slabs), ntiles))));
    for (int attempt = more_splits > base_splits ? 0 : 1; attempt < 2 && !p.ping; ++attempt) {
      p.n_splits = attempt == 0 ? more_splits : base_splits;
      p.n_writers = p.n_splits;
      if (search() && (found || attempt == 1)) {
        const double per_group = 2048.0 * m_exp / N;
        const int nd = forced >= 2 && forced <= 4 ? forced - 1 : int(ceil((per_group + 3.5 * sqrt(per_group)) / 64.0));
        if (nd >= 1 && nd <= 3) p.ping = nd;
      }
    }
    if (!p.ping) {
      p.n_splits = base_splits;
      p.n_writers = 2 * p.n_splits;
    }
  }
  if (!p.ping && !search()) return false;
  // A writer's segment: its share of the expected candidates with room for five or more standard deviations (the
  // threshold's noise, a relative 1 / sqrt(rank) of all of a row's candidates, plus the spread of a share);
  // the overflow guard keeps 16 slots free.  With a small rank 1.35 times the share is less than that.
  {
    const double per_w = m_exp / p.n_writers;
    const double sd_w = sqrt(pow(double(N) / p.ns * sqrt(double(p.rank)) / p.n_writers, 2) + per_w);
    p.cap_w = int(std::max(1.35 * per_w + 64.0, per_w + room_sigmas(p.rank) * sd_w + 16.0));
  }
  p.ld_s = (int64_t(p.ns) + 3) / 4 * 4;
  p.ldy = (int64_t(N) + 3) / 4 * 4;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    size_t r = o;
    o = align_up(o + bytes, 256);
    return r;
  };
  const size_t rows = size_t(H) * C;
  p.off_Ks = take(size_t(H) * p.ns * d * sizeof(bf16_t));
  p.off_Ys = take(rows * p.ld_s * sizeof(float));
  p.off_tau = take(rows * sizeof(float));
  p.off_cand = take(rows * p.n_writers * size_t(p.cap_w) * sizeof(uint2));
  p.off_cnt = take(rows * p.n_writers * sizeof(int32_t));
  p.off_fail = take(kMaxRepair * sizeof(int32_t));
  p.off_nfail = take(4 * sizeof(int32_t));
  p.off_Yf = take(size_t(kMaxRepair) * p.ldy * sizeof(float));
  p.total = o;
  return true;
}

// The filter stores a candidate's key as a code: first key of its 32-key half-tile (a multiple of
// 32) + 16*(lane half) + accumulator register r; that register holds key row 8*(r/4) + 4*half + r%4.
__device__ __forceinline__ uint32_t fused_key_of_code(uint32_t code) {
  return (code & ~31u) + ((code & 12u) << 1) + ((code & 16u) >> 2) + (code & 3u);
}

// ---- phase 0 ---------------------------------------------------------------
__global__ __launch_bounds__(256) void gather_sample_kernel(const bf16_t* __restrict__ K,
                                                            bf16_t* __restrict__ Ks, int N, int ns,
                                                            int stride) {
  const int h = blockIdx.y;
  const int64_t e = int64_t(blockIdx.x) * 256 + threadIdx.x;  // 16-byte chunk id
  if (e >= int64_t(ns) * (kFD / 8)) return;
  const int i = int(e / (kFD / 8)), ch = int(e % (kFD / 8));
  const uint4* src = reinterpret_cast<const uint4*>(K + (int64_t(h) * N + int64_t(i) * stride) * kFD) + ch;
  reinterpret_cast<uint4*>(Ks + (int64_t(h) * ns + i) * kFD)[ch] = *src;
}

// tau[row] = a lower bound of the rank-th largest value of the sampled row that
// at least `rank` sampled values reach (value bits only: 11+11+10).
constexpr int kTauThreads = 256;  // a sampled row is short: narrow workgroups, several rows per CU in flight
__global__ __launch_bounds__(kTauThreads) void row_threshold_kernel(const float* __restrict__ Ys,
                                                                    int ns, int64_t ld, int rank,
                                                                    float* __restrict__ tau,
                                                                    int32_t* __restrict__ n_fail) {
  __shared__ SelectShared sh;
  if (blockIdx.x == 0 && threadIdx.x < 4) n_fail[threadIdx.x] = 0;
  DenseRowT<kTauThreads> src{Ys + int64_t(blockIdx.x) * ld, ns};
  const uint64_t cut = radix_select_cut<kTauThreads>(src, rank, 3, sh);
  if (threadIdx.x == 0) tau[blockIdx.x] = key_to_float(uint32_t(cut >> 32));
}

// ---- phase 1 ---------------------------------------------------------------
// grid (n_splits, slabs, H); workgroup (sk, slab, h) takes key tiles sk, sk+n_splits, ...
// Candidates are (value bits, key index) pairs in segments [row][writer][cap_w]; a
// writer is one (key split, lane half) pair, i.e. exactly one lane of one wave, so
// cursors are registers and appends need no atomics.
//
// Nine waves.  Wave 8 is the producer: it streams the 64-key tiles from global
// memory into a double-buffered LDS tile, two tiles ahead, and is the only wave
// that ever waits on vector-memory loads.  Waves 0..7 own 64 buckets each (their A
// rows stay in registers as MFMA B fragments) and per 32-key half-tile do
//   * 16 MFMAs (32 keys x 64 buckets x d=128),
//   * the threshold test: per accumulator register one v_cmp and one v_addc that
//     shifts the outcome into a per-lane bit mask -- no exec-mask changes and no
//     memory traffic -- while the accumulators are dumped to a wave-private LDS area,
//   * emission rounds: every lane that still has mask bits pops one, reads that
//     value back from its LDS dump and appends (value, key) to its segment.
// The compute waves issue stores only, so they never stall on a memory counter;
// the two waves that share a SIMD overlap one's MFMAs with the other's VALU work.
template <bool F16>
__global__ __launch_bounds__(kFThreads) void fused_filter_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ K, const float* __restrict__ tau,
    uint2* __restrict__ cand, int32_t* __restrict__ cnt, int C, int N, int n_splits, int cap_w) {
  // one object, so that the dump area is preceded by the key tiles: a lane without candidates
  // reads the word below its dump row, which must stay inside the allocation
  __shared__ __attribute__((aligned(16))) struct {
    bf16_t keys[2][kFKeys * kFLd];
    float dump[kFWaves][2 * 64 * kFDumpLd];  // [wave][column half ni][lane][accumulator register, padded]
  } sm;
  bf16_t(&sK)[2][kFKeys * kFLd] = sm.keys;
  const int sk = blockIdx.x, slab = blockIdx.y, h = blockIdx.z;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int n_writers = 2 * n_splits;
  const bf16_t* Kh = K + int64_t(h) * N * kFD;
  const int ntiles = (N + kFKeys - 1) / kFKeys;
  const int my_tiles = sk < ntiles ? (ntiles - sk + n_splits - 1) / n_splits : 0;  // tiles sk + i*n_splits

  if (w == kFWaves) {
    // ------------------------------ producer wave ------------------------------
    // chunk e = u*64 + l of a tile: row 4u + l/16, 16-byte column l%16 (4 whole rows per instruction)
    uint4 st[2][16];
    auto fetch = [&](int i, uint4 (&r)[16]) {
      const int64_t key0 = (int64_t(sk) + int64_t(i) * n_splits) * kFKeys + (l >> 4);
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int64_t key = key0 + 4 * u;
        r[u] = key < N ? reinterpret_cast<const uint4*>(Kh + key * kFD)[l & 15] : make_uint4(0, 0, 0, 0);
      }
    };
    auto stash = [&](int buf, const uint4 (&r)[16]) {
#pragma unroll
      for (int u = 0; u < 16; ++u)
        *reinterpret_cast<uint4*>(&sK[buf][(4 * u + (l >> 4)) * kFLd + (l & 15) * 8]) = r[u];
    };
    if (my_tiles > 0) {
      fetch(0, st[0]);
      stash(0, st[0]);
    }
    if (my_tiles > 1) fetch(1, st[1]);
    if (my_tiles > 2) fetch(2, st[0]);
    __syncthreads();
    for (int i = 0; i < my_tiles; i += 2) {
      // iteration i: tile i+1 (set 1) -> buffer 1, then tile i+3 into set 1
      if (i + 1 < my_tiles) stash(1, st[1]);
      if (i + 3 < my_tiles) fetch(i + 3, st[1]);
      __syncthreads();
      if (i + 1 >= my_tiles) break;
      // iteration i+1: tile i+2 (set 0) -> buffer 0, then tile i+4 into set 0
      if (i + 2 < my_tiles) stash(0, st[0]);
      if (i + 4 < my_tiles) fetch(i + 4, st[0]);
      __syncthreads();
    }
    return;
  }

  // ------------------------------ compute waves ------------------------------
  const int cb = slab * kFSlab + w * 64;  // this wave's first bucket
  const bool active = cb < C;
  const bf16_t* Ah = A + int64_t(h) * C * kFD;
  // segments of this workgroup's 512 bucket rows; lane offsets below are bytes from here
  const int64_t wg_row0 = int64_t(h) * C + int64_t(slab) * kFSlab;
  char* cbase = reinterpret_cast<char*>(cand + wg_row0 * n_writers * int64_t(cap_w));
  float* dump = sm.dump[w];

  bf16x8 bfrag[2][8];
  float th[2];
  uint32_t off[2], start[2], lim[2];
  int ovf[2] = {0, 0};
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int row = cb + ni * 32 + (l & 31);
    const bool ok = row < C;
    const uint4* pa = reinterpret_cast<const uint4*>(Ah + int64_t(ok ? row : 0) * kFD + (l >> 5) * 8);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      union {
        uint4 u;
        bf16x8 b;
      } cvt;
      cvt.u = ok ? pa[2 * ks] : make_uint4(0, 0, 0, 0);
      bfrag[ni][ks] = cvt.b;
    }
    th[ni] = ok ? tau[int64_t(h) * C + row] : INFINITY;
    const uint32_t rl = uint32_t(w * 64 + ni * 32 + (l & 31));  // row inside the slab
    start[ni] = ((rl * uint32_t(n_writers) + uint32_t(sk * 2 + (l >> 5))) * uint32_t(cap_w)) * 8u;
    off[ni] = start[ni];
    lim[ni] = start[ni] + uint32_t(cap_w - 16) * 8u;
  }
  // make the resident operands "used" here so that the wait for their loads sits before the loop
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) asm volatile("" ::"v"(bfrag[ni][ks]));
    asm volatile("" ::"v"(th[ni]));
  }
  const int lane_code = (l >> 5) << 4;
  uint32_t msk[2];

  // Threshold test of four accumulator registers: mask = 2*mask + (y >= th) for each, and their
  // dump.  The registers of a column half are tested from 15 down to 0, so bit r of the mask
  // belongs to register r.  The dump comes first: it is the compiler-visible read of freshly written MFMA
  // results, so the wait states an MFMA result needs before it can be read are inserted there; the
  // asm (whose operands the hazard logic does not look into) then only ever reads settled registers.
  auto test_dump4 = [&](const f32x16& a, int ni, int q) {
    *reinterpret_cast<float4*>(&dump[(ni * 64 + l) * kFDumpLd + 4 * q]) =
        make_float4(a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]);
#pragma unroll
    for (int j = 3; j >= 0; --j)
      asm volatile("v_cmp_nlt_f32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc"
                   : "+v"(msk[ni])
                   : "v"(a[4 * q + j]), "v"(th[ni])
                   : "vcc", "memory");
  };
  // Emission: every lane pops up to two mask bits per column half (lowest register first), reads
  // those values back from its LDS dump (all four reads in flight together) and appends
  // (value bits, key code) pairs to its segment, both pairs of a column half with one 16-byte store:
  // when only one bit was popped, the second pair lands beyond the cursor and the next append
  // overwrites it (the overflow guard keeps 16 slots free).  The key code is  first key of the
  // half-tile + 16*(l/32) + register; fused_key_of_code() turns it into the key index.  A lane
  // without bits reads a harmless word below its column and stores nothing.
  auto emit = [&](auto check_n, uint32_t code0) {
    bool has[4];
    int r[4];
    float y[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      uint32_t& m = msk[p >> 1];
      if constexpr (decltype(check_n)::value) {  // the ragged last tile: drop the bits of rows past N first
        while (m != 0 && fused_key_of_code(code0 + uint32_t(__builtin_ffs(int(m)) - 1)) >= uint32_t(N)) m &= m - 1u;
      }
      has[p] = m != 0;
      r[p] = __builtin_ffs(int(m)) - 1;
      m &= m - 1u;
    }
#pragma unroll
    for (int p = 0; p < 4; ++p) y[p] = dump[((p >> 1) * 64 + l) * kFDumpLd + r[p]];
    // keep the four reads together ahead of the predicated stores (one LDS round trip, not four)
    asm volatile("" : "+v"(y[0]), "+v"(y[1]), "+v"(y[2]), "+v"(y[3]));
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      if (has[2 * ni]) {
        typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
        const u32x4_t rec = {__float_as_uint(y[2 * ni]), code0 + uint32_t(r[2 * ni]), __float_as_uint(y[2 * ni + 1]),
                             code0 + uint32_t(r[2 * ni + 1])};
        *reinterpret_cast<u32x4_t*>(cbase + off[ni]) = rec;
        off[ni] += has[2 * ni + 1] ? 16u : 8u;
      }
    }
  };

  __syncthreads();  // first tile staged
  for (int i = 0; i < my_tiles; ++i) {
    if (active) {
      const int kbase = (sk + i * n_splits) * kFKeys;
      const bool check_n = kbase + kFKeys > N;
      bf16x8 a_pre[4];  // fragments 0..3 of the second half, read while the first half is emitted
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const bf16_t* pa = &sK[i & 1][(half * 32 + (l & 31)) * kFLd + (l >> 5) * 8];
        bf16x8 a[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
          if (half == 0 || ks >= 4)
            a[ks] = *reinterpret_cast<const bf16x8*>(pa + ks * 16);
          else
            a[ks] = a_pre[ks];
        f32x16 acc[2];
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[ni][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          acc[0] = mfma32<F16>(a[ks], bfrag[0][ks], acc[0]);
          acc[1] = mfma32<F16>(a[ks], bfrag[1][ks], acc[1]);
        }
        if (half == 0) {
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) a_pre[ks] = *reinterpret_cast<const bf16x8*>(pa + 32 * kFLd + ks * 16);
        }
        msk[0] = msk[1] = 0;
        asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");  // all 16 accumulator passes retired
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
          for (int q = 3; q >= 0; --q) test_dump4(acc[ni], ni, q);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
          if (off[ni] > lim[ni]) {  // fewer than 16 free slots: wrap and mark the row for repair
            off[ni] = start[ni];
            ovf[ni] = 1;
          }
        const uint32_t code0 = uint32_t(kbase + half * 32 + lane_code);
        if (check_n) {
          do {
            emit(std::true_type{}, code0);
          } while (__ballot((msk[0] | msk[1]) != 0));
        } else {
          do {
            emit(std::false_type{}, code0);
          } while (__ballot((msk[0] | msk[1]) != 0));
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const int row = cb + ni * 32 + (l & 31);
    if (row < C)
      cnt[(int64_t(h) * C + row) * n_writers + sk * 2 + (l >> 5)] =
          ovf[ni] ? cap_w + 1 : int32_t((off[ni] - start[ni]) >> 3);
  }
}

// ---- phase 1, wide form ------------------------------------------------------
// The same filter for C >= 768: eight waves of 128 buckets each (a slab of 1024), no producer wave.
//   * A key fragment read from LDS feeds four MFMAs instead of two, which halves the LDS read traffic per
//     flop -- the LDS (fragment reads + accumulator dumps) is the busiest unit of the 64-bucket form.
//   * The waves stage the 64-key tiles themselves: two 16-byte chunks per lane and tile, requested two
//     tiles ahead and written to LDS one tile ahead, right after the barrier, when every vector-memory
//     operation of the wave is at least half a tile old (loads and stores complete in issue order, so the
//     wait for a tile's loads is also a wait for the candidate stores issued before them).
//   * The epilogue of a tile's second half is carried over the barrier: the end of a tile period is MFMA
//     work only, its candidate stores are issued at the start of the next period, and the two waves of a
//     SIMD drift half a period apart, one's MFMAs facing the other's test / dump / emission.
// Writers, key codes, segments and counts are those of the 64-bucket form: the selection does not see
// which form ran.  256 registers per lane (128 of them the resident bucket fragments), two waves per SIMD.
constexpr int kFWSlab = 1024;  // buckets per workgroup of the wide form (128 per wave)
constexpr int kFWBT = 4;       // 32-bucket tiles per wave

template <bool F16>
__global__ __launch_bounds__(512) void fused_filter_wide_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ K, const float* __restrict__ tau,
    uint2* __restrict__ cand, int32_t* __restrict__ cnt, int C, int N, int n_splits, int cap_w) {
  __shared__ __attribute__((aligned(16))) struct {
    bf16_t keys[2][kFKeys * kFLd];
    float dump[kFWaves][2 * 64 * kFDumpLd];  // [wave][tile of the pair][lane][accumulator register, padded]
  } sm;
  bf16_t(&sK)[2][kFKeys * kFLd] = sm.keys;
  const int sk = blockIdx.x, slab = blockIdx.y, h = blockIdx.z;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int n_writers = 2 * n_splits;
  const bf16_t* Kh = K + int64_t(h) * N * kFD;
  const int ntiles = (N + kFKeys - 1) / kFKeys;
  const int my_tiles = sk < ntiles ? (ntiles - sk + n_splits - 1) / n_splits : 0;  // tiles sk + i*n_splits

  // staging: chunks tid and tid + 512 of a tile's 1024 16-byte chunks (rows tid/16 and 32 + tid/16)
  uint4 st0, st1;
  auto fetch = [&](int i) {
    const int64_t key0 = (int64_t(sk) + int64_t(i) * n_splits) * kFKeys + (tid >> 4);
    st0 = key0 < N ? reinterpret_cast<const uint4*>(Kh + key0 * kFD)[tid & 15] : make_uint4(0, 0, 0, 0);
    st1 = key0 + 32 < N ? reinterpret_cast<const uint4*>(Kh + (key0 + 32) * kFD)[tid & 15] : make_uint4(0, 0, 0, 0);
  };
  auto stash = [&](int buf) {
    *reinterpret_cast<uint4*>(&sK[buf][(tid >> 4) * kFLd + (tid & 15) * 8]) = st0;
    *reinterpret_cast<uint4*>(&sK[buf][(32 + (tid >> 4)) * kFLd + (tid & 15) * 8]) = st1;
  };

  const int cb = slab * kFWSlab + w * (32 * kFWBT);  // this wave's first bucket
  const bool active = cb < C;
  const bf16_t* Ah = A + int64_t(h) * C * kFD;
  const int64_t wg_row0 = int64_t(h) * C + int64_t(slab) * kFWSlab;
  char* cbase = reinterpret_cast<char*>(cand + wg_row0 * n_writers * int64_t(cap_w));
  float* dump = sm.dump[w];

  bf16x8 bfrag[kFWBT][8];
  float th[kFWBT];
  uint32_t off[kFWBT], start[kFWBT], lim[kFWBT];
  uint32_t ovf = 0;  // bit bt: the segment of tile bt wrapped
#pragma unroll
  for (int bt = 0; bt < kFWBT; ++bt) {
    const int row = cb + bt * 32 + (l & 31);
    const bool ok = row < C;
    const uint4* pa = reinterpret_cast<const uint4*>(Ah + int64_t(ok ? row : 0) * kFD + (l >> 5) * 8);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      union {
        uint4 u;
        bf16x8 b;
      } cvt;
      cvt.u = ok ? pa[2 * ks] : make_uint4(0, 0, 0, 0);
      bfrag[bt][ks] = cvt.b;
    }
    th[bt] = ok ? tau[int64_t(h) * C + row] : INFINITY;
    const uint32_t rl = uint32_t(w * (32 * kFWBT) + bt * 32 + (l & 31));  // row inside the slab
    start[bt] = ((rl * uint32_t(n_writers) + uint32_t(sk * 2 + (l >> 5))) * uint32_t(cap_w)) * 8u;
    off[bt] = start[bt];
    lim[bt] = start[bt] + uint32_t(cap_w - 16) * 8u;
  }
#pragma unroll
  for (int bt = 0; bt < kFWBT; ++bt) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) asm volatile("" ::"v"(bfrag[bt][ks]));
    asm volatile("" ::"v"(th[bt]));
  }
  const int lane_code = (l >> 5) << 4;
  uint32_t msk[2];
  f32x16 acc[kFWBT];

  auto test_dump4 = [&](const f32x16& a, float t, int ni, int q) {
    *reinterpret_cast<float4*>(&dump[(ni * 64 + l) * kFDumpLd + 4 * q]) =
        make_float4(a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]);
#pragma unroll
    for (int j = 3; j >= 0; --j)
      asm volatile("v_cmp_nlt_f32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc"
                   : "+v"(msk[ni])
                   : "v"(a[4 * q + j]), "v"(t)
                   : "vcc", "memory");
  };
  // one emission round over the pair of tiles bt0, bt0 + 1 (see fused_filter_kernel::emit)
  auto emit = [&](auto check_n, auto pair, uint32_t code0) {
    constexpr int bt0 = 2 * decltype(pair)::value;
    bool has[4];
    int r[4];
    float y[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      uint32_t& m = msk[p >> 1];
      if constexpr (decltype(check_n)::value) {
        while (m != 0 && fused_key_of_code(code0 + uint32_t(__builtin_ffs(int(m)) - 1)) >= uint32_t(N)) m &= m - 1u;
      }
      has[p] = m != 0;
      r[p] = __builtin_ffs(int(m)) - 1;
      m &= m - 1u;
    }
#pragma unroll
    for (int p = 0; p < 4; ++p) y[p] = dump[((p >> 1) * 64 + l) * kFDumpLd + r[p]];
    asm volatile("" : "+v"(y[0]), "+v"(y[1]), "+v"(y[2]), "+v"(y[3]));
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      if (has[2 * ni]) {
        typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
        const u32x4_t rec = {__float_as_uint(y[2 * ni]), code0 + uint32_t(r[2 * ni]), __float_as_uint(y[2 * ni + 1]),
                             code0 + uint32_t(r[2 * ni + 1])};
        *reinterpret_cast<u32x4_t*>(cbase + off[bt0 + ni]) = rec;
        off[bt0 + ni] += has[2 * ni + 1] ? 16u : 8u;
      }
    }
  };
  auto epi_pair = [&](auto pair, uint32_t code0, bool check_n) {
    constexpr int bt0 = 2 * decltype(pair)::value;
    msk[0] = msk[1] = 0;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q = 3; q >= 0; --q) test_dump4(acc[bt0 + ni], th[bt0 + ni], ni, q);
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
      if (off[bt0 + ni] > lim[bt0 + ni]) {  // fewer than 16 free slots: wrap and mark the row for repair
        off[bt0 + ni] = start[bt0 + ni];
        ovf |= 1u << (bt0 + ni);
      }
    if (check_n) {
      do {
        emit(std::true_type{}, pair, code0);
      } while (__ballot((msk[0] | msk[1]) != 0));
    } else {
      do {
        emit(std::false_type{}, pair, code0);
      } while (__ballot((msk[0] | msk[1]) != 0));
    }
  };
  // 32 MFMAs: 32 keys (half `half` of tile i) x this wave's 128 buckets
  auto mfma_half = [&](int i, int half) {
    const bf16_t* pa = &sK[i & 1][(half * 32 + (l & 31)) * kFLd + (l >> 5) * 8];
#pragma unroll
    for (int bt = 0; bt < kFWBT; ++bt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bt][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(pa + ks * 16);
#pragma unroll
      for (int bt = 0; bt < kFWBT; ++bt) acc[bt] = mfma32<F16>(a, bfrag[bt][ks], acc[bt]);
    }
  };
  // test, dump and emission of the accumulators of (tile i, half): the pair of tiles 0, 1, then 2, 3
  auto epi_half = [&](int i, int half) {
    const int kbase = (sk + i * n_splits) * kFKeys;
    const bool check_n = kbase + kFKeys > N;
    const uint32_t code0 = uint32_t(kbase + half * 32 + lane_code);
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");  // every accumulator pass retired
    epi_pair(std::integral_constant<int, 0>{}, code0, check_n);
    epi_pair(std::integral_constant<int, 1>{}, code0, check_n);
  };

  if (my_tiles > 0) {
    fetch(0);
    stash(0);
  }
  if (my_tiles > 1) fetch(1);
  __syncthreads();
  for (int i = 0; i < my_tiles; ++i) {
    if (i + 1 < my_tiles) stash((i + 1) & 1);  // into the buffer tile i - 1 was read from
    if (i + 2 < my_tiles) fetch(i + 2);
    if (active) {
      if (i > 0) epi_half(i - 1, 1);
      mfma_half(i, 0);
      epi_half(i, 0);
      mfma_half(i, 1);
    }
    __syncthreads();
  }
  if (active && my_tiles > 0) epi_half(my_tiles - 1, 1);
#pragma unroll
  for (int bt = 0; bt < kFWBT; ++bt) {
    const int row = cb + bt * 32 + (l & 31);
    if (row < C)
      cnt[(int64_t(h) * C + row) * n_writers + sk * 2 + (l >> 5)] =
          ((ovf >> bt) & 1u) ? cap_w + 1 : int32_t((off[bt] - start[bt]) >> 3);
  }
}

// ---- phase 1, form with the epilogue between the MFMAs ----------------------------------------
// The same filter on v_mfma_f32_16x16x32 (the same sums: both instructions contract the 128 dimensions in
// ascending order).  A wave still owns 128 buckets and takes the keys 16 at a time: a *group* is 16 keys x 128
// buckets = eight independent accumulator chains of four k-steps, 32 MFMAs, and the accumulators of two groups fit
// where those of one 32-key half tile were.  While the MFMAs of one group issue, the epilogue of the group
// before it is issued between them, slot by slot (VALU work of a wave that sits between the MFMAs of four or
// more independent chains of the same wave costs next to no time of its own on this hardware; work that
// follows the MFMAs, as in the forms above, is only partly hidden by the SIMD's other wave).  For that the
// epilogue is straight-line code:
//   slots 0-7    threshold test of the group's 32 accumulator registers per lane (two VALU instructions each,
//                the outcomes shifted into a 32-bit mask) and the dump of the registers to the wave's LDS slab;
//   slots 8-9    a wave scan of the lanes' candidate counts: a lane's first NR candidates get places in a queue
//                of the wave;
//   then NR rounds in which every lane writes (lane, register) of one of its candidates to its place;
//   then ND passes in which lane j takes the queue's j-th candidate: value from the dump, its bucket's cursor
//   from LDS by an atomic add (a bucket belongs to one wave: no contention beyond the wave's own lanes), key
//   code and one 8-byte store -- three stages a pass, as far apart as the step allows, each waits for LDS.
//   Every lane stores a candidate, not only those whose bucket column it holds.
// Candidates beyond NR per lane or ND * 64 per group (the plan picks NR and ND from the expected pass rate;
// keys that cluster make such groups less rare than even rates would) are appended by loops after the last slot.
// A writer is a key split, so a row has n_splits segments; records carry the same key codes as above, the
// selection does not see which form ran.
constexpr int kFPDumpLd = 36;   // floats per lane in the dump: 32 accumulator registers + 4 (bank spread of the 16-byte stores)
constexpr int kFPQueue = 448;   // queue places of a group's candidates (64 lanes x at most 7 rounds)

struct FpShared {
  bf16_t keys[2][kFKeys * kFLd];
  float dump[kFWaves][64 * kFPDumpLd];
  uint32_t queue[kFWaves][kFPQueue];
  uint32_t cursor[kFWaves][128 + 64];  // a bucket's candidate count so far; lanes without a candidate add behind them
};

template <int N, typename F>
__device__ __forceinline__ void fp_static_for(F&& f) {
  if constexpr (N > 0) {
    fp_static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// key index -> the code fused_key_of_code() undoes
__device__ __forceinline__ uint32_t fused_code_of_key(uint32_t key) {
  return (key & ~31u) | (key & 3u) | ((key >> 1) & 12u) | ((key << 2) & 16u);
}

template <bool F16, int NR, int ND>
__global__ __launch_bounds__(512) void fused_filter_ping_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ K, const float* __restrict__ tau,
    uint2* __restrict__ cand, int32_t* __restrict__ cnt, int C, int N, int n_splits, int cap_w) {
  __shared__ __attribute__((aligned(16))) FpShared sm;
  const int sk = blockIdx.x, slab = blockIdx.y, h = blockIdx.z;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  const int g = l >> 4, c = l & 15;
  const int n_writers = n_splits;
  const bf16_t* Kh = K + int64_t(h) * N * kFD;
  const int ntiles = (N + kFKeys - 1) / kFKeys;
  const int my_tiles = sk < ntiles ? (ntiles - sk + n_splits - 1) / n_splits : 0;  // tiles sk + i*n_splits

  // staging: chunks tid and tid + 512 of a tile's 1024 16-byte chunks (rows tid/16 and 32 + tid/16)
  uint4 st0, st1;
  auto fetch = [&](int i) {  // rows past the last key repeat it (no branch): the emission drops keys >= N
    const int64_t key0 = (int64_t(sk) + int64_t(i) * n_splits) * kFKeys + (tid >> 4);
    st0 = reinterpret_cast<const uint4*>(Kh + min(key0, int64_t(N) - 1) * kFD)[tid & 15];
    st1 = reinterpret_cast<const uint4*>(Kh + min(key0 + 32, int64_t(N) - 1) * kFD)[tid & 15];
  };
  auto stash = [&](int buf) {
    *reinterpret_cast<uint4*>(&sm.keys[buf][(tid >> 4) * kFLd + (tid & 15) * 8]) = st0;
    *reinterpret_cast<uint4*>(&sm.keys[buf][(32 + (tid >> 4)) * kFLd + (tid & 15) * 8]) = st1;
  };

  const int cb = slab * kFWSlab + w * 128;  // this wave's first bucket
  const bool active = cb < C;
  const bf16_t* Ah = A + int64_t(h) * C * kFD;
  const int64_t wg_row0 = int64_t(h) * C + int64_t(slab) * kFWSlab;
  char* cbase = reinterpret_cast<char*>(cand + (wg_row0 + w * 128) * n_writers * int64_t(cap_w));
  float* dump = sm.dump[w];
  uint32_t* queue = sm.queue[w];
  uint32_t* cursor = sm.cursor[w];
  for (int t = l; t < 128 + 64; t += 64) cursor[t] = 0;

  // resident bucket fragments: bucket cb + 16 bt + c, dimensions 32 ks + 8 g ..
  uint4 bfrag[8][4];
  float th[8];
#pragma unroll
  for (int bt = 0; bt < 8; ++bt) {
    const int row = cb + bt * 16 + c;
    const bool ok = row < C;
    const uint4* pa = reinterpret_cast<const uint4*>(Ah + int64_t(ok ? row : 0) * kFD + g * 8);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bfrag[bt][ks] = ok ? pa[4 * ks] : make_uint4(0, 0, 0, 0);
    th[bt] = ok ? tau[int64_t(h) * C + row] : INFINITY;
  }
#pragma unroll
  for (int bt = 0; bt < 8; ++bt) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
      asm volatile("" ::"v"(bfrag[bt][ks].x), "v"(bfrag[bt][ks].y), "v"(bfrag[bt][ks].z), "v"(bfrag[bt][ks].w));
    asm volatile("" ::"v"(th[bt]));
  }

  f32x4 acc[2][8];  // [group parity][bucket tile]
  uint4 af[2];      // A fragment of a k-step, [k-step parity]
  uint32_t msk = 0, msk0 = 0;
  int n_mine = 0, base = 0, base0 = 0, total = 0;
  bool more = false;
  uint32_t* my_queue = queue;
  // dense passes in flight: descriptor, value, bucket, slot of lane j's candidate
  uint32_t d_desc[ND], d_slot[ND];
  float d_val[ND];
  bool d_ok[ND];

  // LDS address of this lane's A fragment of (buffer, half, key tile kt), k-step 0
  auto frag_ptr = [&](int buf, int grp) -> const bf16_t* {  // grp = 2 half + kt: keys 16 grp .. of the tile
    return &sm.keys[buf][(grp * 16 + c) * kFLd + g * 8];
  };

  // the candidate (lane L, register e) of the group whose first key is key0: checks, cursor and store
  auto emit_one = [&](bool valid, uint32_t L, uint32_t e, float val, uint32_t key0) {
    const uint32_t key = key0 + 4u * (L >> 4) + (e & 3u);
    const uint32_t bl = (e >> 2) * 16u + (L & 15u);
    valid = valid && key < uint32_t(N);
    const uint32_t slot = atomicAdd(&cursor[valid ? bl : 128u + uint32_t(l)], 1u);
    if (valid && slot < uint32_t(cap_w)) {
      const uint2 rec = make_uint2(__float_as_uint(val), fused_code_of_key(key));
      *reinterpret_cast<uint2*>(cbase + ((bl * uint32_t(n_writers) + uint32_t(sk)) * uint32_t(cap_w) + slot) * 8u) = rec;
    }
  };

  // One group step, slot S of 32.  DO_MFMA: the MFMA (k-step S / 8, bucket tile S % 8) of the group at `fp` into
  // acc[P]; DO_EPI: the epilogue of the group before it (acc[1 - P], first key key0_old).
  auto group_step = [&](auto P_, auto DO_MFMA_, auto DO_EPI_, const bf16_t* fp, const bf16_t* fp_next, uint32_t key0_old) {
    constexpr int P = decltype(P_)::value;
    constexpr bool DO_MFMA = decltype(DO_MFMA_)::value, DO_EPI = decltype(DO_EPI_)::value;
    fp_static_for<32>([&](auto S_) {
      constexpr int S = decltype(S_)::value;
      constexpr int ks = S >> 3, bt = S & 7;
      if constexpr (DO_MFMA) {
        if constexpr (bt == 0) {
          if constexpr (ks < 3)
            af[(ks + 1) & 1] = *reinterpret_cast<const uint4*>(fp + (ks + 1) * 32);
          else
            af[0] = *reinterpret_cast<const uint4*>(fp_next);  // always a readable address: a branch here would
                                                                // make the waits behind it count a read that may not have been issued
        }
        acc[P][bt] = Mma<F16>::m16(af[ks & 1], bfrag[bt][ks], ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[P][bt]);
      }
      if constexpr (DO_EPI) {
        constexpr int Q = 1 - P;
        constexpr int kTS = 8;  // slots of the threshold test
        if constexpr (S < 8) {
          // the four registers of bucket tile S: mask bit 31 - (4 bt + i)
          if constexpr (S == 0) msk = 0;
          asm volatile("v_cmp_nlt_f32 vcc, %1, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc\n\t"
                       "v_cmp_nlt_f32 vcc, %3, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc\n\t"
                       "v_cmp_nlt_f32 vcc, %4, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc\n\t"
                       "v_cmp_nlt_f32 vcc, %5, %2\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc"
                       : "+v"(msk)
                       : "v"(acc[Q][S][0]), "v"(th[S]), "v"(acc[Q][S][1]), "v"(acc[Q][S][2]), "v"(acc[Q][S][3])
                       : "vcc");
          *reinterpret_cast<float4*>(&dump[l * kFPDumpLd + 4 * S]) =
              make_float4(acc[Q][S][0], acc[Q][S][1], acc[Q][S][2], acc[Q][S][3]);
        } else if constexpr (S == kTS) {
          msk0 = msk;
          n_mine = __popc(msk);
          base = wave_incl_scan_dpp(min(n_mine, NR));  // the queue takes a lane's first NR candidates
        } else if constexpr (S == kTS + 1) {
          total = __builtin_amdgcn_readlane(base, 63);
          base -= min(n_mine, NR);
          base0 = base;
          more = __ballot(n_mine > NR) != 0ull || total > ND * 64;  // candidates the rounds or the passes do not reach
          my_queue = queue + base;
        } else if constexpr (S < kTS + 2 + NR) {
          // a round: one candidate per lane to its place in the queue (a lane's places are below 64 NR)
          static_assert(NR * 64 <= kFPQueue, "every lane's NR places are inside the queue");
          constexpr int k = S - (kTS + 2);
          if (msk != 0u) my_queue[k] = (uint32_t(l) << 5) | uint32_t(__builtin_ctz(msk));
          msk &= msk - 1u;  // leaves an empty mask empty
        } else {
          // dense passes: three stages a pass, staggered by one slot from pass to pass
          constexpr int S0 = kTS + 2 + NR + 1;  // first stage of pass 0 (a slot after the last round)
          constexpr int gap = (31 - S0 - (ND - 1)) / 2;  // as far apart as the step allows: each stage waits for LDS
          fp_static_for<ND>([&](auto D_) {
            constexpr int D = decltype(D_)::value;
            if constexpr (S == S0 + D) {
              d_ok[D] = D * 64 + l < total;
              d_desc[D] = queue[min(D * 64 + l, kFPQueue - 1)];
            } else if constexpr (S == S0 + D + gap) {
              const uint32_t L = d_desc[D] >> 5, e = 31u - (d_desc[D] & 31u);
              d_val[D] = dump[__umul24(L, kFPDumpLd) + e];
              const uint32_t key = key0_old + 4u * (L >> 4) + (e & 3u);
              d_ok[D] = d_ok[D] && key < uint32_t(N);
              d_slot[D] = atomicAdd(&cursor[d_ok[D] ? (e >> 2) * 16u + (L & 15u) : 128u + uint32_t(l)], 1u);
            } else if constexpr (S == S0 + D + 2 * gap) {
              const uint32_t L = d_desc[D] >> 5, e = 31u - (d_desc[D] & 31u);
              const uint32_t key = key0_old + 4u * (L >> 4) + (e & 3u);
              const uint32_t bl = (e >> 2) * 16u + (L & 15u);
              if (d_ok[D] && d_slot[D] < uint32_t(cap_w)) {
                const uint2 rec = make_uint2(__float_as_uint(d_val[D]), fused_code_of_key(key));
                *reinterpret_cast<uint2*>(cbase + (__umul24(__umul24(bl, uint32_t(n_writers)) + uint32_t(sk), uint32_t(cap_w)) + d_slot[D]) * 8u) = rec;
              }
            }
          });
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (DO_EPI) {
      // What the rounds and passes above did not reach.  A lane's candidates beyond the NR-th are the bits the
      // rounds left in its mask: appended here, a lane a round (keys that cluster make this less rare than even
      // rates would: a bucket then takes most keys of a group).
      static_assert(ND * 64 <= kFPQueue, "the passes read what the queue holds");
      if (more) {
        while (__ballot(msk != 0u)) {
          const bool has = msk != 0u;
          const uint32_t e = 31u - uint32_t(__builtin_ctz(msk | 0x80000000u));
          emit_one(has, uint32_t(l), e, dump[l * kFPDumpLd + e], key0_old);
          msk = has ? (msk & (msk - 1u)) : msk;
        }
        // ... and the candidates whose place in the queue lies beyond the passes' ND * 64 (a group with more than
        // that many candidates in all): the lanes that hold them go through their first NR again
        if (total > ND * 64) {
          uint32_t m = msk0;
          for (int k = 0; k < NR; ++k) {
            const bool has = m != 0u;
            const uint32_t e = 31u - uint32_t(__builtin_ctz(m | 0x80000000u));
            emit_one(has && base0 + k >= ND * 64, uint32_t(l), e, dump[l * kFPDumpLd + e], key0_old);
            m = has ? (m & (m - 1u)) : m;
          }
        }
      }
    }
  };

  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  if (my_tiles > 0) {
    fetch(0);
    stash(0);
  }
  if (my_tiles > 1) fetch(1);
  __syncthreads();
  uint32_t key0_prev = 0;  // first key of the group whose epilogue is pending
  for (int i = 0; i < my_tiles; ++i) {
    if (i + 1 < my_tiles) stash((i + 1) & 1);  // into the buffer tile i - 1 was read from
    if (i + 2 < my_tiles) fetch(i + 2);
    if (active) {
      const int buf = i & 1;
      const uint32_t kbase = uint32_t((sk + i * n_splits) * kFKeys);
      af[0] = *reinterpret_cast<const uint4*>(frag_ptr(buf, 0));
      if (i == 0)
        group_step(B0{}, std::true_type{}, std::false_type{}, frag_ptr(buf, 0), frag_ptr(buf, 1), 0u);
      else
        group_step(B0{}, std::true_type{}, std::true_type{}, frag_ptr(buf, 0), frag_ptr(buf, 1), key0_prev);
      group_step(B1{}, std::true_type{}, std::true_type{}, frag_ptr(buf, 1), frag_ptr(buf, 2), kbase);
      group_step(B0{}, std::true_type{}, std::true_type{}, frag_ptr(buf, 2), frag_ptr(buf, 3), kbase + 16u);
      group_step(B1{}, std::true_type{}, std::true_type{}, frag_ptr(buf, 3), frag_ptr(buf, 0), kbase + 32u);
      key0_prev = kbase + 48u;
    }
    __syncthreads();
  }
  if (active && my_tiles > 0)
    group_step(B0{}, std::false_type{}, std::true_type{}, nullptr, nullptr, key0_prev);
  // candidate counts (beyond cap_w: the segment overflowed, the row is repaired)
  for (int t = l; t < 128; t += 64) {
    const int row = cb + t;
    if (row < C) cnt[(int64_t(h) * C + row) * n_writers + sk] = int32_t(min(cursor[t], uint32_t(cap_w) + 1u));
  }
}

// ---- phase 2 ---------------------------------------------------------------
// Per-writer candidate counts of a row in LDS; returns false (to all threads) if a segment
// overflowed or the row has fewer than Zc candidates, i.e. the sampled threshold failed.
struct CandCounts {
  int counts[64];
  int total, over, maxc;
};
__device__ __forceinline__ bool load_cand_counts(const int32_t* __restrict__ cnt, int64_t row, int n_writers,
                                                 int cap_w, int Zc, CandCounts& cc) {
  if (threadIdx.x < 64) {
    int c = threadIdx.x < n_writers ? cnt[row * n_writers + threadIdx.x] : 0;
    const int over = __any(c > cap_w);
    c = min(c, cap_w);
    cc.counts[threadIdx.x] = c;
    int total = c, mx = c;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      total += __shfl_xor(total, o);
      mx = max(mx, __shfl_xor(mx, o));
    }
    if (threadIdx.x == 0) {
      cc.total = total;
      cc.over = over;
      cc.maxc = mx;
    }
  }
  __syncthreads();
  return !(cc.over || cc.total < Zc);
}

// A row's candidates held in registers: the NT threads are dealt to the writers' segments in
// groups of T = NT / n_writers, and a thread keeps elements t, t + T, t + 2T, ... of its segment
// (at most R of them).  The candidates are read from memory once; the radix passes of
// the selection and the collection into the sort buffer then run from registers.
template <int R>
struct CandRegs {
  uint2 e[R];  // (value bits, key code)
  int n;               // valid entries of this thread
  template <typename F>
  __device__ __forceinline__ void operator()(F f) const {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (r < n) f(__uint_as_float(e[r].x), fused_key_of_code(e[r].y));
  }
};

static inline size_t cand_select_lds_bytes(int Zc, int P) {
  const size_t binned = binned_lds_bytes(Zc);
  const size_t sorted = sort_lds_bytes(P) + sizeof(SelectShared) + 8;
  return std::max(binned, sorted);
}

// Exact top-Z (value desc, index asc) of every row's candidates: radix select of the cut,
// collection of the Zc survivors into LDS, bitonic sort, indices out -- the code of the dense
// arg-top-Z kernel, on ~1.2 Zc register-resident candidates instead of the N-element row.
template <int NT, int R>
__global__ __launch_bounds__(NT) void cand_select_kernel(
    const uint2* __restrict__ cand, const int32_t* __restrict__ cnt, int n_writers, int cap_w, int Zc, int P,
    int32_t* __restrict__ idx_out, float* __restrict__ val_out, int32_t* __restrict__ fail_rows,
    int32_t* __restrict__ n_fail) {
  // dynamic LDS, two uses of the same bytes: [composites of the binned selection | its histogram], or,
  // when that declines the row, [sort buffer of the radix select | its histograms]
  extern __shared__ uint64_t buf[];
  __shared__ CandCounts cc;
  __shared__ BinShared bs;
  const int64_t row = blockIdx.x;
  const int T = NT / n_writers;  // threads per segment
  bool ok = load_cand_counts(cnt, row, n_writers, cap_w, Zc, cc);
  ok = ok && cc.maxc <= T * R;
  if (!ok) {  // threshold missed (or a segment too long to hold): queue the row for repair
    if (threadIdx.x == 0) {
      int pos = atomicAdd(n_fail, 1);
      if (pos < kMaxRepair) fail_rows[pos] = int32_t(row);
    }
    // Until the repair overwrites it the row holds keys 0 .. Zc-1: should more rows fail than the repair
    // takes, a caller that reads the status word late (a recorded graph, a stream it does not wait for)
    // has run its attention over valid key indices, never over uninitialised memory.
    for (int j = threadIdx.x; j < Zc; j += NT) {
      idx_out[row * Zc + j] = j;
      if (val_out) val_out[row * Zc + j] = 0.f;
    }
    return;
  }
  CandRegs<R> src;
  const int w = threadIdx.x / T, t = threadIdx.x - w * T;
  const int cw = w < n_writers ? cc.counts[w] : 0;
  const uint2* seg = cand + (row * n_writers + min(w, n_writers - 1)) * int64_t(cap_w);
  src.n = cw > t ? (cw - t + T - 1) / T : 0;
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (r < src.n) src.e[r] = seg[t + r * T];
  int32_t* out = idx_out + row * Zc;
  float* vout = val_out ? val_out + row * Zc : nullptr;
  uint32_t* hist = reinterpret_cast<uint32_t*>(buf + (Zc + kSelMaxBin));
  if (binned_select_write<NT>(src, Zc, buf, hist, bs, out, vout)) return;
  __syncthreads();
  SelectShared& sh = *reinterpret_cast<SelectShared*>(buf + sort_lds_bytes(P) / sizeof(uint64_t));
  const uint64_t cut = radix_select_cut<NT>(src, Zc, 6, sh);
  collect_sort_write(src, cut, Zc, P, buf, sh, out, vout);
}

// ---- phase 3 ---------------------------------------------------------------
// Y of the listed (head, bucket) rows, one output column per workgroup row-slot.
// grid (up to 128, kMaxRepair): a workgroup walks 128-key tiles (4 waves x 32 keys); with nothing to
// repair the launch is 8192 workgroups that read one word and leave.
template <bool F16>
__global__ __launch_bounds__(256) void project_listed_rows_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ K, const int32_t* __restrict__ fail_rows,
    const int32_t* __restrict__ n_fail, float* __restrict__ Yf, int C, int N, int64_t ldy) {
  const int slot = blockIdx.y;
  if (slot >= min(*n_fail, kMaxRepair)) return;
  const int row = fail_rows[slot];
  const int h = row / C;
  const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
  const uint4* pa = reinterpret_cast<const uint4*>(A + int64_t(row) * kFD + (l >> 5) * 8);
  bf16x8 bfr[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    union {
      uint4 u;
      bf16x8 b;
    } b;
    b.u = (l & 31) == 0 ? pa[2 * ks] : make_uint4(0, 0, 0, 0);  // only column 0 carries the row
    bfr[ks] = b.b;
  }
  for (int tile = blockIdx.x; tile * 128 < N; tile += gridDim.x) {
    const int key = tile * 128 + w * 32 + (l & 31);
    const uint4* pk = reinterpret_cast<const uint4*>(K + (int64_t(h) * N + min(key, N - 1)) * kFD + (l >> 5) * 8);
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      union {
        uint4 u;
        bf16x8 b;
      } a;
      a.u = key < N ? pk[2 * ks] : make_uint4(0, 0, 0, 0);
      acc = mfma32<F16>(a.b, bfr[ks], acc);
    }
    if ((l & 31) == 0) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int n = tile * 128 + w * 32 + acc_row_32(r, l);
        if (n < N) Yf[int64_t(slot) * ldy + n] = acc[r];
      }
    }
  }
}

__global__ __launch_bounds__(64) void fused_status_kernel(const int32_t* __restrict__ n_fail,
                                                          const int32_t* __restrict__ fail_rows,
                                                          int32_t* __restrict__ status) {
  const int f = *n_fail, t = threadIdx.x;
  if (t == 0) {
    status[0] = min(f, kMaxRepair);
    status[1] = max(0, f - kMaxRepair);
  }
  static_assert(FM_FUSED_STATUS_INTS == 2 + kMaxRepair, "the status word names every repaired row");
  status[2 + t] = t < min(f, kMaxRepair) ? fail_rows[t] : -1;  // the repaired (head * C + bucket) rows
}

// optional phase markers for profiling: events recorded after phases 0, 1, 2, 3
// (process-wide and guarded by a mutex: a build that runs while another thread sets or clears the
// markers records into the old set or the new one, never into a half-written pair)
static std::mutex g_phase_mu;
static hipEvent_t* g_phase_events = nullptr;
static int g_n_phase_events = 0;
static inline void mark_phase(int i, hipStream_t st) {
  std::lock_guard<std::mutex> lk(g_phase_mu);
  if (g_phase_events && i < g_n_phase_events) (void)hipEventRecord(g_phase_events[i], st);
}

}  // namespace fm

extern "C" void fm_debug_fused_filter(int form) {
  if (fm::debug_hooks_enabled()) fm::g_fused_filter_form.store(form, std::memory_order_relaxed);
}

extern "C" void fm_debug_set_phase_events(void** events, int n) {
  if (!fm::debug_hooks_enabled()) return;
  std::lock_guard<std::mutex> lk(fm::g_phase_mu);
  fm::g_phase_events = reinterpret_cast<hipEvent_t*>(events);
  fm::g_n_phase_events = events ? n : 0;
}

extern "C" const char* fm_build_index_fused_kernel(int H, int C, int N, int d, int Z, int dtype) {
  fm::FusedPlan p;
  if (H < 1 || C < 1 || N < 1 || !fm::fused_plan(H, C, N, d, Z, dtype, p)) return nullptr;
  return p.ping ? "fused_filter_ping_kernel" : p.wide ? "fused_filter_wide_kernel" : "fused_filter_kernel";
}

extern "C" size_t fm_build_index_fused_workspace(int H, int C, int N, int d, int Z, int dtype) {
  fm::FusedPlan p;
  if (H < 1 || C < 1 || N < 1 || !fm::fused_plan(H, C, N, d, Z, dtype, p)) return 0;
  return p.total;
}

extern "C" int fm_build_index_fused(const void* A, const void* K, int32_t* idx_out, float* val_out, int H,
                                    int C, int N, int d, int Z, int dtype, void* ws, size_t ws_bytes,
                                    int32_t* status_dev, void* stream) {
  using namespace fm;
  FM_REQUIRE(H >= 1 && C >= 1 && N >= 1 && Z >= 1, FM_ERR_ARG, "fm_build_index_fused: H=%d C=%d N=%d Z=%d",
             H, C, N, Z);
  FM_REQUIRE(A && K && idx_out && ws && status_dev, FM_ERR_ARG, "fm_build_index_fused: null pointer");
  FusedPlan p;
  FM_REQUIRE(fused_plan(H, C, N, d, Z, dtype, p), FM_ERR_UNSUPPORTED,
             "fm_build_index_fused: shape not eligible (needs bf16 or fp16, d=128, N >= 65536, 64 <= Z <= N/8)");
  FM_REQUIRE(ws_bytes >= p.total, FM_ERR_WORKSPACE, "fm_build_index_fused: workspace %zu < %zu", ws_bytes,
             p.total);
  FM_REQUIRE(H <= 65535 && int64_t(H) * C <= 0x7fffffffLL, FM_ERR_UNSUPPORTED,
             "fm_build_index_fused: too many rows");
  hipStream_t st = as_stream(stream);
  char* base = static_cast<char*>(ws);
  bf16_t* Ks = reinterpret_cast<bf16_t*>(base + p.off_Ks);
  float* Ys = reinterpret_cast<float*>(base + p.off_Ys);
  float* tau = reinterpret_cast<float*>(base + p.off_tau);
  uint2* cand = reinterpret_cast<uint2*>(base + p.off_cand);
  int32_t* cnt = reinterpret_cast<int32_t*>(base + p.off_cnt);
  int32_t* fail_rows = reinterpret_cast<int32_t*>(base + p.off_fail);
  int32_t* n_fail = reinterpret_cast<int32_t*>(base + p.off_nfail);
  float* Yf = reinterpret_cast<float*>(base + p.off_Yf);
  const int64_t rows = int64_t(H) * C;
  const int Zc = Z;  // Z <= N/8 here

  // phase 0
  mark_phase(0, st);
  hipLaunchKernelGGL(gather_sample_kernel, dim3(unsigned(ceil_div(int64_t(p.ns) * (kFD / 8), 256)), unsigned(H)),
                     dim3(256), 0, st, (const bf16_t*)K, Ks, N, p.ns, p.stride);
  int rc = fm_project(A, Ks, Ys, H, C, p.ns, d, p.ld_s, dtype, stream);
  if (rc) return rc;
  hipLaunchKernelGGL(row_threshold_kernel, dim3(unsigned(rows)), dim3(kTauThreads), 0, st, Ys, p.ns,
                     p.ld_s, p.rank, tau, n_fail);
  // phase 1
  mark_phase(1, st);
  {
    const dim3 grid = dim3(unsigned(p.n_splits), unsigned(p.slabs), unsigned(H));
#define FM_FILTER(KERNEL, THREADS)                                                                          \
  hipLaunchKernelGGL(KERNEL, grid, dim3(THREADS), 0, st, (const bf16_t*)A, (const bf16_t*)K, tau, cand, cnt, C, N, \
                     p.n_splits, p.cap_w)
    if (p.ping == 1 && dtype == FM_F16)
      FM_FILTER((fused_filter_ping_kernel<true, 4, 1>), 512);
    else if (p.ping == 1)
      FM_FILTER((fused_filter_ping_kernel<false, 4, 1>), 512);
    else if (p.ping == 2 && dtype == FM_F16)
      FM_FILTER((fused_filter_ping_kernel<true, 6, 2>), 512);
    else if (p.ping == 2)
      FM_FILTER((fused_filter_ping_kernel<false, 6, 2>), 512);
    else if (p.ping == 3 && dtype == FM_F16)
      FM_FILTER((fused_filter_ping_kernel<true, 7, 3>), 512);
    else if (p.ping == 3)
      FM_FILTER((fused_filter_ping_kernel<false, 7, 3>), 512);
    else if (p.wide && dtype == FM_F16)
      FM_FILTER(fused_filter_wide_kernel<true>, 512);
    else if (p.wide)
      FM_FILTER(fused_filter_wide_kernel<false>, 512);
    else if (dtype == FM_F16)
      FM_FILTER(fused_filter_kernel<true>, kFThreads);
    else
      FM_FILTER(fused_filter_kernel<false>, kFThreads);
#undef FM_FILTER
  }
  // phase 2
  mark_phase(2, st);
  const int P = next_pow2(Zc);
#define FM_CAND_SELECT(NT, R)                                                                           \
  do {                                                                                                  \
    FM_ALLOW_LDS((cand_select_kernel<NT, R>), cand_select_lds_bytes(FM_MAX_Z, FM_MAX_Z), "fm_build_index_fused: lds");   \
    hipLaunchKernelGGL((cand_select_kernel<NT, R>), dim3(unsigned(rows)), dim3(NT), cand_select_lds_bytes(Zc, P), st, cand, cnt, \
                       p.n_writers, p.cap_w, Zc, P, idx_out, val_out, fail_rows, n_fail);                      \
  } while (0)
  if (p.sel_threads == 256)
    FM_CAND_SELECT(256, kCandRegsSmall);
  else if (p.sel_threads == 512)
    FM_CAND_SELECT(512, kCandRegsSmall);
  else
    FM_CAND_SELECT(kSelThreads, kCandRegs);
#undef FM_CAND_SELECT
  // phase 3
  mark_phase(3, st);
  const dim3 rgrid = dim3(unsigned(std::min<int64_t>(ceil_div(N, 128), 128)), kMaxRepair);
  if (dtype == FM_F16)
    hipLaunchKernelGGL(project_listed_rows_kernel<true>, rgrid, dim3(256), 0, st, (const bf16_t*)A, (const bf16_t*)K,
                       fail_rows, n_fail, Yf, C, N, p.ldy);
  else
    hipLaunchKernelGGL(project_listed_rows_kernel<false>, rgrid, dim3(256), 0, st, (const bf16_t*)A, (const bf16_t*)K,
                       fail_rows, n_fail, Yf, C, N, p.ldy);
  rc = launch_argtopz(Yf, kMaxRepair, N, p.ldy, Zc, idx_out, val_out, fail_rows, n_fail, st);
  if (rc) return rc;
  hipLaunchKernelGGL(fused_status_kernel, dim3(1), dim3(64), 0, st, n_fail, fail_rows, status_dev);
  mark_phase(4, st);
  return launch_status("fm_build_index_fused");
}
