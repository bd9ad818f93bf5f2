// Launch of the bucket-gathered attention that gives every work item a wave of its own (attn_wave.hpp): four
// items per workgroup of 256 threads, two workgroups per compute unit, no barriers.  The form for long lists
// with few queries each on a memory whose key rows are listed in many buckets.
#include <atomic>
#include <mutex>
#include <unordered_map>

#include "attn_wave.hpp"

namespace fm {

extern std::atomic<int> g_force_generic;  // attn_api.hip; 13: a launch per row with the sweeps unpaced

// The schedule of a paced launch (WaveClock in attn_wave.hpp) is found by trying, launch after launch, for
// every (memory, lists, row) the library sees: a table of the library's own in device memory, one copy per
// GPU, a slot per (N, C, Sq, the lists' address, the row) -- the host hands the slots out (the 1024 keys seen
// last have one each).  A one-thread kernel behind every launch (wave_pace_step_kernel) takes the launch's
// duration and sets the next launch's schedule.  A launch either keeps its schedule (it ends within 10 % of
// it) or falls off it: the waves that get behind the others no longer find their rows in the L2, get further
// behind, and the launch takes a fifth to a half longer than unpaced.  So:
//   * no schedule yet: the launch runs unpaced; the second such launch (the first on a memory is a cold one)
//     gives the unpaced duration, and the next launch a schedule of 0.92 x that;
//   * searching: a kept schedule is followed by one 2 % faster; the first one missed ends the search -- the
//     slot holds the fastest schedule kept + 2 % (if none was kept: 5 % slower and on with the search);
//   * holding, for 16 launches the first time and twice as long after every search, up to 256: a launch that
//     misses the held schedule makes it 3 % slower; every 129th launch runs unpaced and renews the unpaced
//     duration; then the search goes on from the held schedule;
//   * the held schedule's launches take more than 0.97 x the unpaced duration on average, or a schedule would
//     have to be slower than that: the slot gives up for 1024 launches (they run unpaced and cost nothing),
//     then starts again.
// Calls that use a slot at the same time (two streams on one memory and row) mix their measurements: the
// schedule may then be a poor one, nothing else.
struct WavePaceSlot {
  unsigned long long key;   // whose slot this is (0: nobody's)
  unsigned long long t0;    // start of the launch in flight (0: none, or one without a work item)
  float tpk_used;           // the schedule it runs on (0: unpaced)
  int mode;                 // 0 the next launch runs unpaced and is measured, 1 paced, 2 given up (hold counts down)
  float tpk;                // ticks per key of the next launch's schedule
  float good;               // the fastest schedule kept in the current search (0: none yet)
  float held;               // mean ticks per key of the launches on the held schedule
  float base;               // ticks per key of the unpaced launch
  int hold;                 // launches until the search goes on / until pacing is tried again
  int hold_len;             // how long the next hold lasts
  float last_elapsed;       // the last launch: its ticks per key and the schedule it ran on (diagnostics)
  float last_tpk;
  int refresh;              // 1: the next launch runs unpaced although the slot paces, to renew the unpaced duration
  int since_refresh;        // paced launches since the last such measurement
  int measured;             // unpaced launches measured since the slot (re)started
  int pad;
};
constexpr int kWavePaceSlots = 1024;
static __device__ __align__(256) WavePaceSlot g_wave_pace[kWavePaceSlots];

// What wave_pace_step_kernel does with the slot.  elapsed: ticks since the launch's first wave started;
// tpk_used: the schedule the launch ran on (0: unpaced).
__device__ inline void wave_pace_update(WavePaceSlot* s, unsigned long long key, float elapsed, float tpk_used, int N) {
  const float e = elapsed / float(N);  // ticks per key of this launch
  if (s->key != key) {  // (first use, or another memory's slot: start over)
    s->key = key;
    s->mode = 0;
    s->hold = 0;
    s->measured = 0;
    s->refresh = 0;
  }
  s->last_elapsed = e;
  s->last_tpk = tpk_used;
  auto give_up = [&]() {
    s->mode = 2;
    s->hold = 1024;
    s->tpk = 0.f;
    s->measured = 0;
  };
  if (tpk_used <= 0.f) {
    if (s->mode == 1) {  // the unpaced duration measured again beside the paced launches
      s->base = 0.7f * s->base + 0.3f * e;
      s->refresh = 0;
      s->since_refresh = 0;
      if (s->hold > 0 && s->held > 0.97f * s->base) give_up();
    } else if (s->mode == 2 && --s->hold > 0) {
      s->tpk = 0.f;
      s->measured = 0;
    } else if (++s->measured < 2) {
      s->mode = 0;
    } else {
      s->base = e;
      s->tpk = 0.92f * e;
      s->mode = 1;
      s->good = 0.f;
      s->held = 0.f;
      s->hold = 0;
      s->hold_len = 16;
      s->refresh = 0;
      s->since_refresh = 0;
    }
    return;
  }
  const bool kept = e <= 1.10f * tpk_used;
  if (s->hold == 0) {  // searching
    if (kept) {
      s->good = tpk_used;
      s->tpk = fmaxf(0.98f * tpk_used, 0.4f * s->base);
    } else if (s->good > 0.f) {
      s->tpk = 1.02f * s->good;
      s->held = 1.02f * s->tpk;  // (what a launch on it should take; the launches will tell)
      s->good = 0.f;
      s->hold = s->hold_len;
      s->hold_len = s->hold_len < 128 ? 2 * s->hold_len : 256;
      s->since_refresh = int((key >> 20) & 127);  // (the rows of a memory renew their unpaced durations in different calls)
    } else {
      s->tpk = 1.05f * tpk_used;
    }
  } else {  // holding
    s->held = 0.8f * s->held + 0.2f * e;
    if (kept) {
      if (--s->hold == 0) s->good = 0.f;
    } else {
      s->tpk = 1.03f * tpk_used;
    }
    if (++s->since_refresh >= 128) s->refresh = 1;
    if (s->held > 0.97f * s->base) give_up();
  }
  if (s->mode == 1 && s->tpk > 0.97f * s->base) give_up();
}

// Which work item a wave takes in a launch over one row.  A compute unit holds two workgroups of this kernel,
// and a launch's workgroups i and i + (number of compute units) end up on the same one, wave w of each on the
// same SIMD (measured on 256 compute units; nothing depends on it but speed).  Two waves with two or three tiles
// of queries each keep that SIMD busier than a tile's loads take, two with one tile leave it idle: so the items
// of every 2048 slots are taken heaviest first (by tiles of queries, stable) by the first 1024 slots and lightest
// first by the rest -- slot k then shares its SIMD with slot k + 1024, the heaviest with the lightest.  (Query
// counts drawn at random over 2048 buckets, 16 on average: 7.4 ms per step against 7.9 in bucket order, and
// against 8.0 with like paired with like.)  Every workgroup works the order out for its 2048 slots by itself: a
// counting sort over four classes in LDS the waves have not begun to use.  Called by all threads of the
// workgroup; returns n_it for a slot that has no item.
constexpr int kWavePairSlots = 1024;
__device__ __forceinline__ int wave_paired_item(const fm_item* __restrict__ items, int first, int n_it, int slot,
                                                char* lds) {
  constexpr int kChunk = 2 * kWavePairSlots;
  const int chunk0 = slot / kChunk * kChunk;  // (the same for the four waves: kChunk is a multiple of 4)
  const int m = min(kChunk, n_it - first - chunk0);
  uint16_t* sorted = reinterpret_cast<uint16_t*>(lds);                  // kChunk entries
  long long* scan_tmp = reinterpret_cast<long long*>(lds + 2 * kChunk);  // 17 words
  if (m <= 0) return n_it;  // (all four waves of the workgroup alike)
  // thread t: items 8 t .. 8 t + 7 of the chunk; class = tiles of queries - 1, at most 3 (an item swept twice)
  int cls[8];
  long long mine = 0;  // four 16-bit counts
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = 8 * int(threadIdx.x) + i;
    cls[i] = j < m ? min((items[first + chunk0 + j].n_q - 1) >> 4, 3) : -1;
    if (cls[i] >= 0) mine += 1ll << (16 * cls[i]);
  }
  long long total;
  long long before = block_excl_scan_ll(mine, scan_tmp, &total);
  // heaviest class first
  const int t3 = int(total >> 48) & 0xffff, t2 = int(total >> 32) & 0xffff, t1 = int(total >> 16) & 0xffff;
  const int base[4] = {t3 + t2 + t1, t3 + t2, t3, 0};
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if (cls[i] >= 0) {
      const int pos = base[cls[i]] + (int(before >> (16 * cls[i])) & 0xffff);
      before += 1ll << (16 * cls[i]);
      sorted[pos] = uint16_t(8 * int(threadIdx.x) + i);
    }
  __syncthreads();
  const int k = slot - chunk0;
  const int item = k < m ? first + chunk0 + sorted[k < kWavePairSlots ? k : m - 1 - (k - kWavePairSlots)] : n_it;
  __syncthreads();  // (the waves' tiles take this LDS next)
  return item;
}

template <bool F16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void hash_attn_wave_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const int32_t* __restrict__ k_idx, const int64_t* __restrict__ bucket_off,
    const int32_t* __restrict__ bucket_cnt, const int32_t* __restrict__ q_perm,
    const fm_item* __restrict__ items, const int32_t* __restrict__ n_items,
    bf16_t* __restrict__ out, float* __restrict__ lse, int Sq, int N, int C, float scale2, int only_row,
    WavePaceSlot* __restrict__ pace, unsigned long long pace_key) {
  extern __shared__ __attribute__((aligned(16))) bf16_t wave_lds[];
  int n_it = *n_items;
  int first = 0;
  if (only_row >= 0) {  // a launch per row: the row's items are [first, n_it)
    first = first_item_of_row(items, n_it, only_row);
    n_it = first_item_of_row(items, n_it, only_row + 1);
  }
  const int w = __builtin_amdgcn_readfirstlane(int(threadIdx.x) >> 6);
  int me = first + 4 * int(blockIdx.x) + w;
  if (only_row >= 0 && n_it - first > kWavePairSlots)
    me = wave_paired_item(items, first, n_it, 4 * int(blockIdx.x) + w, reinterpret_cast<char*>(wave_lds));
  if (me >= n_it) return;  // (no barrier from here on: a wave may leave alone)
  const fm_item it = items[me];
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int64_t qbase = int64_t(it.row) * Sq;
  // The launch's schedule (WaveClock).  Every wave takes its own start for the launch's: the waves of a launch
  // start within a microsecond or two of each other (measured), while 2048 of them agreeing on one start through
  // an atomic on one word took the last of them 100 us, which put those behind the schedule before they began.
  WaveClock clk{0, 0.f};
  if (pace) {
    const unsigned long long now = __builtin_amdgcn_s_memrealtime();
    const float tpk = pace->key == pace_key && pace->mode == 1 && !pace->refresh ? pace->tpk : 0.f;
    clk = WaveClock{now, __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, tpk)))};
    if (blockIdx.x == 0 && threadIdx.x == 0) {  // for wave_pace_step_kernel, which follows the launch
      pace->t0 = now;
      pace->tpk_used = tpk;
    }
  }
  // (an item has up to FM_QTILE = 64 queries, a sweep takes 48: the few items with more are swept twice, the
  // second time unpaced)
  for (int q0 = 0; q0 < it.n_q; q0 += 48) {
    attend_wave<3, F16>(q + qbase * kSD, q_perm + it.q_start + q0, min(it.n_q - q0, 48), k + int64_t(it.row) * N * kSD,
                        v + int64_t(it.row) * N * kSD, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                        out + qbase * kSD, lse + qbase, (lds_char_t*)wave_lds + w * kWWaveBytes, clk);
    clk.ticks_per_key = 0.f;
  }
}

// One thread, launched behind every paced launch on its stream: the launch's duration (from the start its
// first wave noted to now) sets the next launch's schedule.
__global__ void wave_pace_step_kernel(WavePaceSlot* __restrict__ pace, unsigned long long pace_key, int N) {
  const unsigned long long now = __builtin_amdgcn_s_memrealtime(), t0 = pace->t0;
  if (t0 == 0 || now <= t0) return;  // (the launch had no work item: nothing was measured)
  wave_pace_update(pace, pace_key, float(now - t0), pace->tpk_used, N);
  pace->t0 = 0;
}

// The table's address on the current device (in host code its name only stands for the symbol); null while it
// is not known and cannot be asked for (a stream that is being captured: the launches then go unpaced).
static WavePaceSlot* wave_pace_table(hipStream_t st) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static WavePaceSlot* table[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!table[dev]) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return nullptr;
    }
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_wave_pace)) == hipSuccess)
      table[dev] = static_cast<WavePaceSlot*>(p);
    else
      (void)hipGetLastError();
  }
  return table[dev];
}

// The slot of a key: the keys in use have a slot each; the 1025th new key takes over the slot handed out
// longest ago (the kernel sees another key in it and starts that slot over).
static int wave_pace_slot(unsigned long long key) {
  static std::mutex mu;
  static std::unordered_map<unsigned long long, int> slot_of;
  static unsigned long long owner[kWavePaceSlots];
  static int next = 0;
  std::lock_guard<std::mutex> lock(mu);
  auto it = slot_of.find(key);
  if (it != slot_of.end()) return it->second;
  const int s = next;
  next = (next + 1) % kWavePaceSlots;
  if (owner[s]) slot_of.erase(owner[s]);
  owner[s] = key;
  slot_of[key] = s;
  return s;
}

static unsigned long long wave_pace_key(int N, int C, int Sq, const void* lists, int row) {
  unsigned long long x = (unsigned long long)(uintptr_t)lists ^ ((unsigned long long)N << 40) ^ ((unsigned long long)C << 20) ^
                         ((unsigned long long)Sq * 0x9E3779B97F4A7C15ull) ^ ((unsigned long long)(row + 1) * 0xC2B2AE3D27D4EB4Full);
  x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27; x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  return x | 1ull;
}

int hash_attn_mfma_wave(const void* q, const void* k, const void* v, const int32_t* k_idx, const int64_t* bucket_off,
                        const int32_t* bucket_cnt, const int32_t* q_perm, const fm_item* items,
                        const int32_t* n_items, int64_t max_items, void* out, float* lse, int Sq, int N, int C,
                        float sm_scale, bool f16, int H, bool per_row, hipStream_t st) {
  // paced sweeps for the launches per row (a single launch over all rows has no common sweep to pace)
  WavePaceSlot* const table = per_row && g_force_generic != 13 ? wave_pace_table(st) : nullptr;
#define FM_WAVE_LAUNCH(F16, ITEMS, ROW)                                                                           \
  do {                                                                                                            \
    FM_ALLOW_LDS((hash_attn_wave_kernel<F16>), kWaveLdsBytes, "fm_hash_attn_fwd: lds");                           \
    hipLaunchKernelGGL((hash_attn_wave_kernel<F16>), dim3(unsigned(ceil_div(int64_t(ITEMS), int64_t(4)))),        \
                       dim3(256), kWaveLdsBytes, st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, k_idx, \
                       bucket_off, bucket_cnt, q_perm, items, n_items, (bf16_t*)out, lse, Sq, N, C,               \
                       sm_scale * kLog2e, ROW, pace_slot, pace_key);                                              \
  } while (0)
  if (per_row) {
    // One launch per row, in row order, for the reason given in attn_mfma_ring.hip: the waves of a launch start
    // together and sweep the row's K and V at about the same pace.
    const int64_t row_items = std::min<int64_t>(max_items, int64_t(C < Sq ? C : Sq) + Sq / FM_QTILE + 1);
    for (int row = 0; row < H; ++row) {
      const unsigned long long pace_key = wave_pace_key(N, C, Sq, k_idx, row);
      WavePaceSlot* const pace_slot = table ? table + wave_pace_slot(pace_key) : nullptr;
      if (f16)
        FM_WAVE_LAUNCH(true, row_items, row);
      else
        FM_WAVE_LAUNCH(false, row_items, row);
      if (pace_slot) hipLaunchKernelGGL(wave_pace_step_kernel, dim3(1), dim3(1), 0, st, pace_slot, pace_key, N);
    }
  } else {
    const unsigned long long pace_key = 0;
    WavePaceSlot* const pace_slot = nullptr;
    if (f16)
      FM_WAVE_LAUNCH(true, max_items, -1);
    else
      FM_WAVE_LAUNCH(false, max_items, -1);
  }
#undef FM_WAVE_LAUNCH
  return launch_status("fm_hash_attn_fwd(mfma, wave)");
}

// out[0..7] = mode, ticks per key of the next launch's schedule, of the fastest schedule kept in the current
// search, of the launches on the held schedule (mean), of the unpaced launch, launches the hold still lasts, the
// last launch's ticks per key and the schedule it ran on, of the slot of (N, C, Sq, lists, row); all zero where there is none yet.  A synchronous copy.
int wave_pace_state(int N, int C, int Sq, const void* lists, int row, float* out) {
  for (int i = 0; i < 8; ++i) out[i] = 0.f;
  WavePaceSlot* const table = wave_pace_table(nullptr);
  if (!table) return FM_ERR_LAUNCH;
  const unsigned long long key = wave_pace_key(N, C, Sq, lists, row);
  WavePaceSlot h;
  if (hipMemcpy(&h, table + wave_pace_slot(key), sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) {
    (void)hipGetLastError();
    return FM_ERR_LAUNCH;
  }
  if (h.key != key) return FM_OK;
  out[0] = float(h.mode); out[1] = h.tpk; out[2] = h.good; out[3] = h.held; out[4] = h.base; out[5] = float(h.hold);
  out[6] = h.last_elapsed; out[7] = h.last_tpk;
  return FM_OK;
}

}  // namespace fm
