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
// last have one each).  The last wave of a launch to finish (every wave counts itself out) takes the launch's
// duration and sets the next launch's schedule -- a descent on the duration itself, which is what counts:
//   * no schedule yet: the launch ran unpaced; the one after the second such launch (the first on a memory is
//     a cold one) gets 0.92 x its duration;
//   * the launch was no slower than the best so far (within 1 %): it is the best now, and unless the schedule is
//     being held the next one is 2 % faster;
//   * it was slower: back to the best schedule, held for 16 launches the first time and twice as long after
//     every such step back, up to 256 (while a schedule is held, the best duration follows what the launches
//     at it take);
//   * while a schedule is held, every 33rd launch runs unpaced and renews the unpaced duration;
//   * the best is no better than 0.97 x the unpaced duration, or four launches in a row were slower than the
//     unpaced one: the slot gives up for 1024 launches (they run unpaced and cost nothing), then starts again.
// A schedule that a launch cannot keep costs that launch up to a third of its time; one it can keep saves up to
// a quarter; once settled a slot tries a faster one every 256 launches.  Calls that use a slot at the same time
// (two streams on one memory and row) mix their measurements: the schedule may then be a poor one, nothing
// else.
struct WavePaceSlot {
  unsigned long long key;   // whose slot this is (0: nobody's)
  unsigned long long t0;    // start of the launch in flight (0: none has started)
  unsigned int done;        // waves of it that have finished
  int mode;                 // 0 the next launch runs unpaced and is measured, 1 paced, 2 given up (hold counts down)
  float tpk;                // ticks per key of the next launch's schedule
  float best_tpk;           // the schedule of the shortest launch so far, and that launch's ticks per key
  float best;
  float base;               // ticks per key of the unpaced launch
  int hold;                 // launches until a faster schedule is tried again / until pacing is tried again
  int hold_len;             // how long the next hold lasts
  int slow;                 // launches in a row slower than the unpaced one
  float last_elapsed;       // the last launch: its ticks per key and the schedule it ran on (diagnostics)
  float last_tpk;
  int refresh;              // 1: the next launch runs unpaced although the slot paces, to measure the unpaced duration again
  int since_refresh;        // paced launches since the last such measurement
  int measured;             // unpaced launches measured since the slot (re)started
};
constexpr int kWavePaceSlots = 1024;
static __device__ __align__(256) WavePaceSlot g_wave_pace[kWavePaceSlots];

// What the last wave of a launch does with the slot (one lane).  elapsed: ticks since the launch's first wave
// started; tpk_used: the schedule the launch ran on (0: unpaced).
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
  if (tpk_used <= 0.f) {
    if (s->mode == 1) {  // the unpaced duration measured again beside the paced launches
      s->base = 0.7f * s->base + 0.3f * e;
      s->refresh = 0;
      s->since_refresh = 0;
    } else if (s->mode == 2 && --s->hold > 0) {
      s->tpk = 0.f;
      s->measured = 0;
    } else if (++s->measured < 2) {  // (the first launch on a memory is a cold one: the second counts)
      s->mode = 0;
    } else {
      s->base = e;
      s->tpk = 0.92f * e;
      s->mode = 1;
      s->best = 0.f;
      s->best_tpk = 0.f;
      s->hold = 0;
      s->hold_len = 16;
      s->slow = 0;
      s->refresh = 0;
      s->since_refresh = 0;
    }
    if (s->mode == 1 && s->hold > 0 && s->best > 0.97f * s->base) {
      s->mode = 2;
      s->hold = 1024;
      s->tpk = 0.f;
      s->measured = 0;
    }
    return;
  }
  if (++s->since_refresh >= 32 && s->hold > 0) s->refresh = 1;
  s->slow = e > s->base ? s->slow + 1 : 0;
  if (s->best <= 0.f || e <= 1.01f * s->best) {
    if (s->best <= 0.f || e < s->best || tpk_used == s->best_tpk) {
      s->best = (tpk_used == s->best_tpk && s->best > 0.f) ? 0.8f * s->best + 0.2f * e : e;
      s->best_tpk = tpk_used;
    }
    if (s->hold > 0)
      --s->hold;
    else
      s->tpk = fmaxf(0.98f * s->best_tpk, 0.4f * s->base);
  } else if (tpk_used == s->best_tpk) {  // the best schedule itself has become slower: follow it
    s->best = 0.8f * s->best + 0.2f * e;
    if (s->hold > 0) --s->hold;
  } else {
    s->tpk = s->best_tpk;
    s->hold = s->hold_len;
    s->hold_len = s->hold_len < 128 ? 2 * s->hold_len : 256;
  }
  if (s->slow >= 4 || (s->hold > 0 && s->best > 0.97f * s->base)) {
    s->mode = 2;
    s->hold = 1024;
    s->tpk = 0.f;
    s->measured = 0;
  }
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
  const int me = first + 4 * int(blockIdx.x) + w;
  if (me >= n_it) return;  // (no barrier anywhere: a wave may leave alone)
  const fm_item it = items[me];
  const int64_t bkt = int64_t(it.row) * C + it.bucket;
  const int64_t qbase = int64_t(it.row) * Sq;
  // The launch's schedule and start (WaveClock): the first wave to come sets the start.
  WaveClock clk{0, 0.f};
  float tpk_used = 0.f;
  if (pace) {
    unsigned long long t0 = 0;
    float tpk = 0.f;
    if ((threadIdx.x & 63) == 0) {
      const unsigned long long now = __builtin_amdgcn_s_memrealtime();
      unsigned long long old = atomicCAS(&pace->t0, 0ull, now);
      if (old && now - old > (1ull << 28)) {  // a start 2.7 s old: a launch never counted itself out (two calls
        // mixed on the slot with different numbers of waves); start over
        if (atomicCAS(&pace->t0, old, now) == old) atomicExch(&pace->done, 0u);
        old = 0;
      }
      t0 = old ? old : now;
      tpk = pace->key == pace_key && pace->mode == 1 && !pace->refresh ? pace->tpk : 0.f;
    }
    t0 = (uint64_t(__builtin_amdgcn_readfirstlane(uint32_t(t0 >> 32))) << 32) | __builtin_amdgcn_readfirstlane(uint32_t(t0));
    tpk_used = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, tpk)));
    clk = WaveClock{t0, tpk_used};
  }
  // (an item has up to FM_QTILE = 64 queries, a sweep takes 48: the few items with more are swept twice, the
  // second time unpaced)
  for (int q0 = 0; q0 < it.n_q; q0 += 48) {
    attend_wave<3, F16>(q + qbase * kSD, q_perm + it.q_start + q0, min(it.n_q - q0, 48), k + int64_t(it.row) * N * kSD,
                        v + int64_t(it.row) * N * kSD, k_idx + bucket_off[bkt], bucket_cnt[bkt], N, scale2,
                        out + qbase * kSD, lse + qbase, (lds_char_t*)wave_lds + w * kWWaveBytes, clk);
    clk.ticks_per_key = 0.f;
  }
  // Every wave counts itself out; the last one sets the next launch's schedule and clears the way for it.
  if (pace && (threadIdx.x & 63) == 0) {
    const unsigned int n_waves = unsigned(n_it - first);
    if (atomicAdd(&pace->done, 1u) + 1u == n_waves) {
      const unsigned long long now = __builtin_amdgcn_s_memrealtime();
      const unsigned long long t0 = atomicAdd(&pace->t0, 0ull);
      wave_pace_update(pace, pace_key, float(now - t0), tpk_used, N);
      __threadfence();
      pace->done = 0u;
      atomicExch(&pace->t0, 0ull);
    }
  }
}

// The table's address on the current device (in host code its name only stands for the symbol).
static WavePaceSlot* wave_pace_table() {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static WavePaceSlot* table[kMaxDevices];
  static bool asked[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!asked[dev]) {
    asked[dev] = true;
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
  WavePaceSlot* const table = per_row && g_force_generic != 13 ? wave_pace_table() : nullptr;
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

// out[0..7] = mode, ticks per key of the next launch's schedule, of the best schedule and of the launch that
// ran on it, of the unpaced launch, launches until the next try, the last launch's ticks per key and the
// schedule it ran on, of the slot of (N, C, Sq, lists, row); all zero where there is none yet.  A synchronous copy.
int wave_pace_state(int N, int C, int Sq, const void* lists, int row, float* out) {
  for (int i = 0; i < 8; ++i) out[i] = 0.f;
  WavePaceSlot* const table = wave_pace_table();
  if (!table) return FM_ERR_LAUNCH;
  const unsigned long long key = wave_pace_key(N, C, Sq, lists, row);
  WavePaceSlot h;
  if (hipMemcpy(&h, table + wave_pace_slot(key), sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) {
    (void)hipGetLastError();
    return FM_ERR_LAUNCH;
  }
  if (h.key != key) return FM_OK;
  out[0] = float(h.mode); out[1] = h.tpk; out[2] = h.best_tpk; out[3] = h.best; out[4] = h.base; out[5] = float(h.hold);
  out[6] = h.last_elapsed; out[7] = h.last_tpk;
  return FM_OK;
}

}  // namespace fm
