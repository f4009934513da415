// Negative-sample pass of skip-gram negative sampling, and its forward-only twin.
//
// Semantics follow the reference CPU path, jni/src/BIDMach_CPUMACH.c:186-264 (word2vecNeg) and
// :429-483 (word2vecEvalNeg): group i holds nwa words WA[i*nwa + j] (columns of A) and nwb words
// WB[i*nwb + k] (columns of B); for every (j, k):
//   s = A[:,wa_j] . B[:,wb_k];  g = -lrate * sigmoid(s)
//   dB_k += bscale_k * g * A[:,wa_j];   dA_j += ascale_j * g * B[:,wb_k]
// and every dot product of the group uses the columns as they were when the group started; the
// nwa + nwb accumulated deltas are scattered once each.
//
// One wavefront owns one group at a time.  The nwb B columns and their nwb accumulators stay in
// registers; A columns stream through CHA at a time (all loads of a chunk issued before its first
// dot).  The CHA*nwb pre-activations of a chunk are parked one per lane so that the sigmoid (a
// double exp) is evaluated once per chunk; each A delta leaves as float atomics right after its
// chunk and the B deltas after the last chunk, so every column is read once and updated once per
// group.
//
// The update kernel is persistent: a fixed number of workgroups each walk a contiguous range of
// groups, which bounds the number of groups in flight (and with it the staleness of the Hogwild
// updates) by the launch size.  The atomics for the hottest columns go to their shadow copies
// (w2v_device.h), so their same-line atomics spread over several lines, and the columns of words
// that are rare within the launch are updated with a device-scope read-modify-write instead of
// atomics (prepare_rare_words below), which takes a third or more of the load off the float-atomic
// units that bound the pass.
//
// The reference reads WA/WB without a validity test (:213-214,220-221); here a negative id
// skips every pair it takes part in, so a bad id cannot become an out-of-bounds access.
#include <atomic>

#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

// Forward-only twin: sum over the group's pairs of log(max(1 - sigmoid(s), floor)).
// Persistent: workgroup b walks groups [b*groups_per_wg, (b+1)*groups_per_wg), one group per wave
// at a time, and a wave fetches the word ids of its next group while it works on the current
// one, so that the only memory latency left on its critical path is that of the column gathers.
template <int R, int MAXB, int CHA>
__global__ void __launch_bounds__(kBlock)
neg_eval_kernel(int d, int ngroups, int nwa, int nwb, int64_t groups_per_wg,
                const int* __restrict__ WA, const int* __restrict__ WB,
                const float* __restrict__ A, const float* __restrict__ B, double floorv,
                double* __restrict__ partials) {
  static_assert(MAXB * CHA <= kWave, "one lane per pre-activation of a chunk");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t g_begin = (int64_t)blockIdx.x * groups_per_wg;
  const int64_t g_end = min(g_begin + groups_per_wg, (int64_t)ngroups);
  double lsum = 0.0;

  int64_t unit = g_begin + wave;
  int wbl = -1, wal0 = -1;
  if (unit < g_end) {
    if (lane < nwb) wbl = WB[unit * nwb + lane];
    if (lane < nwa) wal0 = WA[unit * nwa + lane];
  }
  for (; unit < g_end; unit += kWavesPerBlock) {
    // ids of this wave's next group, in flight while this group is scored
    const int64_t next = unit + kWavesPerBlock;
    int wbl_next = -1, wal_next = -1;
    if (next < g_end) {
      if (lane < nwb) wbl_next = WB[next * nwb + lane];
      if (lane < nwa) wal_next = WA[next * nwa + lane];
    }
    // MAXB columns of B at a time (one trip unless nwb > MAXB)
    for (int kb = 0; kb < nwb; kb += MAXB) {
    float b[MAXB][R];
    int wb[MAXB];
#pragma unroll
    for (int k = 0; k < MAXB; ++k) {
      wb[k] = -1;
      if (kb + k < nwb) {
        wb[k] = read_lane(wbl, kb + k);
        if (wb[k] >= 0) load_col<R>(b[k], B + (int64_t)wb[k] * d, lane, d);
      }
    }
    for (int jbase = 0; jbase < nwa; jbase += kWave) {
      int wal = wal0;
      if (jbase > 0) {
        wal = -1;
        if (jbase + lane < nwa) wal = WA[unit * nwa + jbase + lane];
      }
      const int jend = min(nwa - jbase, kWave);
      for (int j0 = 0; j0 < jend; j0 += CHA) {
        float a[CHA][R];
        int wa[CHA];
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          wa[c] = -1;
          if (j0 + c < jend) {
            wa[c] = read_lane(wal, j0 + c);
            if (wa[c] >= 0) load_col<R>(a[c], A + (int64_t)wa[c] * d, lane, d);
          }
        }
        // Pre-activation of (c, k) parks in lane c*MAXB + k; only those lanes contribute.
        float pre = 0.0f;
        bool live = false;
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          if (wa[c] >= 0) {
#pragma unroll
            for (int k = 0; k < MAXB; ++k) {
              if (wb[k] >= 0) {
                const float s = wave_sum(dot_partial<R>(a[c], b[k]));
                const bool mine = lane == c * MAXB + k;
                pre = mine ? s : pre;
                live = mine ? true : live;
              }
            }
          }
        }
        if (live) lsum += log(fmax(1.0 - (double)sat_sigmoid(pre), floorv));
      }
    }
    }
    wbl = wbl_next;
    wal0 = wal_next;
  }
  block_store_partial(wave_sum_f64(lsum), partials);
}

constexpr int64_t kMinEvalGroupsPerWg = 64;

constexpr int kNegWaves = 4;
constexpr int kNegThreads = kNegWaves * kWave;
constexpr int kMinGroupsPerWg = 512;  // a workgroup walks at least this many consecutive groups
constexpr int kMinGroupsPerWgWide = 32;  // the same for a launch without hot words
// Waves per SIMD the update kernel is compiled for.  The pass is bound by atomic latency, so it
// wants waves in flight more than it wants registers per wave.
#ifndef W2V_NEG_WAVES_PER_EU
#define W2V_NEG_WAVES_PER_EU 3
#endif

template <int R, int MAXB, int CHA>
__global__ void __launch_bounds__(kNegThreads, W2V_NEG_WAVES_PER_EU)
neg_train_kernel(int d, int ngroups, int idlimit, int nwa, int nwb, int64_t groups_per_wg_hot,
                 int64_t groups_per_wg_wide, int64_t groups_per_wg_ordered,
                 const int* __restrict__ WA, const int* __restrict__ WB, float* A, float* B,
                 float lrate, float vexp, int smode, Shadow shadow_arg) {
  static_assert(MAXB * CHA <= kWave, "one lane per pre-activation of a chunk");
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slot = blockIdx.x;  // picks the shadow copy this workgroup writes to

  int64_t groups_per_wg = launch_is_cold(shadow_arg, shadow) ? groups_per_wg_wide
                                                              : groups_per_wg_hot;
  if (launch_is_ordered(shadow_arg, shadow)) {
    if (groups_per_wg_ordered == 0) return;   // neg_rows_kernel does this launch
    groups_per_wg = groups_per_wg_ordered;    // no ordered instance for this shape: few workers
  }
  const int64_t g_begin = (int64_t)blockIdx.x * groups_per_wg;
  const int64_t g_end = min(g_begin + groups_per_wg, (int64_t)ngroups);

  for (int64_t unit = g_begin + wave; unit < g_end; unit += kNegWaves) {
    // Lane k < nwb holds B word k and its scale.
    int wbl = -1;
    if (lane < nwb) wbl = WB[unit * nwb + lane];
    if (wbl >= idlimit) wbl = -1;  // word2vecNegFilt: ids beyond the resident columns are skipped
    const float sbl = wbl >= 0 ? scale_of(wbl, vexp, smode) : 0.0f;
    // a word that occurs twice in the group would have two plain updates in flight: not rare
    bool lone_b = true;
    if (nwb <= MAXB) {
#pragma unroll
      for (int k = 0; k < MAXB; ++k)
        if (k < nwb && k != lane && read_lane(wbl, k) == wbl) lone_b = false;
    } else {
      for (int k = 0; k < nwb; ++k)
        if (k != lane && read_lane(wbl, k) == wbl) lone_b = false;
    }
    const uint64_t rare_b = __ballot(wbl >= 0 && lone_b && is_rare(shadow, wbl));
    // tickets for the writes to hot B columns at the end of the group, taken now
    const unsigned tkb = hot_ticket(shadow, 0, slot, (wbl >= 0 && wbl < kHotWords) ? wbl : -1);

    // MAXB columns of B at a time.  The launcher sends groups with nwb > MAXB to the kernel of
    // w2v_neg_wide.hip, so this loop makes one trip: with more, the A columns would be read again
    // on every trip with the group's own earlier deltas in them, which the reference's order
    // (A written after the group's last dot, BIDMach_CPUMACH.c:248-254) does not allow.
    for (int kb = 0; kb < nwb; kb += MAXB) {
    float b[MAXB][R];
    float dbb[MAXB][R];
    int wb[MAXB];
#pragma unroll
    for (int k = 0; k < MAXB; ++k) {
      wb[k] = -1;
      if (kb + k < nwb) {
        wb[k] = read_lane(wbl, kb + k);
        if (wb[k] >= 0) {
          if ((rare_b >> (kb + k)) & 1)
            load_col_fresh<R>(b[k], B + (int64_t)wb[k] * d, lane, d);
          else
            load_col_ref<R>(b[k], table_ref(B, wb[k], d), shadow, 0, lane, d);
        }
        zero_col<R>(dbb[k]);
      }
    }

    for (int jbase = 0; jbase < nwa; jbase += kWave) {
      int wal = -1;
      if (jbase + lane < nwa) wal = WA[unit * nwa + jbase + lane];
      if (wal >= idlimit) wal = -1;
      const float sal = wal >= 0 ? scale_of(wal, vexp, smode) : 0.0f;
      const int jend = min(nwa - jbase, kWave);
      bool lone_a = true;
      if (shadow.rare_max > 0) {
        for (int j = 0; j < jend; ++j)
          if (j != lane && read_lane(wal, j) == wal) lone_a = false;
      }
      // (an A word updated on several trips is not rare: its plain updates would be in flight
      // together)
      const uint64_t rare_a =
          __ballot(wal >= 0 && lone_a && nwb <= MAXB && is_rare_a(shadow, wal));
      const unsigned tka = hot_ticket(shadow, 1, slot, (wal >= 0 && wal < kHotWords) ? wal : -1);

      for (int j0 = 0; j0 < jend; j0 += CHA) {
        float a[CHA][R];
        int wa[CHA];
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          wa[c] = -1;
          if (j0 + c < jend) {
            wa[c] = read_lane(wal, j0 + c);
            if (wa[c] >= 0) {
              if ((rare_a >> (j0 + c)) & 1)
                load_col_fresh<R>(a[c], A + (int64_t)wa[c] * d, lane, d);
              else
                load_col_ref<R>(a[c], table_ref(A, wa[c], d), shadow, 1, lane, d);
            }
          }
        }
        float pre = 0.0f;
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          if (wa[c] >= 0) {
#pragma unroll
            for (int k = 0; k < MAXB; ++k) {
              if (wb[k] >= 0) {
                const float s = wave_sum(dot_partial<R>(a[c], b[k]));
                pre = (lane == c * MAXB + k) ? s : pre;
              }
            }
          }
        }
        const float gl = -lrate * sat_sigmoid(pre);
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          if (wa[c] >= 0) {
            const float as = read_lane(sal, j0 + c);
            float daa[R];
            zero_col<R>(daa);
#pragma unroll
            for (int k = 0; k < MAXB; ++k) {
              if (wb[k] >= 0) {
                const float g = read_lane(gl, c * MAXB + k);
                const float bs = read_lane(sbl, kb + k);
                axpy<R>(dbb[k], bs * g, a[c]);
                axpy<R>(daa, as * g, b[k]);
              }
            }
            if ((rare_a >> (j0 + c)) & 1)
              store_sum_col<R>(A + (int64_t)wa[c] * d, a[c], daa, lane, d);
            else
              scatter_add_ref<R>(table_ref(A, wa[c], d), shadow, 1, slot, daa, lane, d,
                                 read_lane(tka, j0 + c));
          }
        }
      }
    }

    // A rare B column was read when the group began, a whole group's work ago: it is read
    // again now (into the registers of the old value, which no dot needs any more), so that what
    // another wave wrote to it in the meantime is kept and only a write that falls into the last
    // few microseconds can be lost.
#pragma unroll
    for (int k = 0; k < MAXB; ++k) {
      if (wb[k] >= 0 && ((rare_b >> (kb + k)) & 1))
        load_col_fresh<R>(b[k], B + (int64_t)wb[k] * d, lane, d);
    }
#pragma unroll
    for (int k = 0; k < MAXB; ++k) {
      if (wb[k] >= 0) {
        if ((rare_b >> (kb + k)) & 1)
          store_sum_col<R>(B + (int64_t)wb[k] * d, b[k], dbb[k], lane, d);
        else
          scatter_add_ref<R>(table_ref(B, wb[k], d), shadow, 0, slot, dbb[k], lane, d,
                             read_lane(tkb, kb + k));
      }
    }
    }
  }
}

// Clears the occurrence counters (a kernel, not a memset, so that callers may capture the call).
__global__ void __launch_bounds__(kBlock) clear_occurs_kernel(int4* __restrict__ p, int n4) {
  for (int i = blockIdx.x * kBlock + threadIdx.x; i < n4; i += gridDim.x * kBlock)
    p[i] = make_int4(0, 0, 0, 0);
}

// Counts how often each word occurs among the two id arrays of a launch, exactly up to rare_max
// and saturating soon after: a slot that is already above rare_max is left alone, so the words that
// occur hundreds of thousands of times do not queue that many atomics on one address.  Words that
// may have shadow copies are never rare and are not counted.  Four ids per thread and trip, so
// that the dependent id -> slot -> atomic chains of a thread overlap.
__device__ __forceinline__ void count_occurrence(int w, int seen, int idlimit, int* occurs,
                                                 int rare_max) {
  if (w >= kHotWords && w < idlimit && seen <= rare_max)
    __hip_atomic_fetch_add(occurs + (w & (kOccurSlots - 1)), 1, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ int peek_occurrence(int w, int idlimit, const int* occurs) {
  // A plain load: an XCD sees the other XCDs' increments of a slot at the latest after its own
  // next increment of it, so every XCD stops soon after the slot has passed rare_max.
  return (w >= kHotWords && w < idlimit)
             ? *const_cast<const volatile int*>(occurs + (w & (kOccurSlots - 1)))
             : 0;
}

// `every` (a power of two): only every `every`-th run of 16 consecutive ids is looked at.  The id
// arrays of the negative pass are in random order, so this is an unbiased sample, and the caller
// scales its threshold accordingly.
__global__ void __launch_bounds__(kBlock)
count_occurs_kernel(const int* __restrict__ ids, int64_t n, int every, int idlimit, int* occurs,
                    int rare_max) {
  const bool aligned = (reinterpret_cast<uintptr_t>(ids) & 15u) == 0;
  const int64_t runs = n / 16;                        // whole runs of 16 ids
  const int64_t kept = (runs + every - 1) / every;    // runs 0, every, 2 * every, ...
  if (aligned) {
    const int4* ids4 = reinterpret_cast<const int4*>(ids);
    for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < kept * 4;
         j += (int64_t)gridDim.x * kBlock) {
      const int4 w = ids4[(j >> 2) * every * 4 + (j & 3)];
      const int s0 = peek_occurrence(w.x, idlimit, occurs);
      const int s1 = peek_occurrence(w.y, idlimit, occurs);
      const int s2 = peek_occurrence(w.z, idlimit, occurs);
      const int s3 = peek_occurrence(w.w, idlimit, occurs);
      count_occurrence(w.x, s0, idlimit, occurs, rare_max);
      count_occurrence(w.y, s1, idlimit, occurs, rare_max);
      count_occurrence(w.z, s2, idlimit, occurs, rare_max);
      count_occurrence(w.w, s3, idlimit, occurs, rare_max);
    }
  } else {
    for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < kept * 16;
         j += (int64_t)gridDim.x * kBlock) {
      const int w = ids[(j >> 4) * every * 16 + (j & 15)];
      count_occurrence(w, peek_occurrence(w, idlimit, occurs), idlimit, occurs, rare_max);
    }
  }
  // the ids after the last whole run, when every id is looked at
  if (every == 1) {
    for (int64_t i = runs * 16 + (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * kBlock) {
      const int w = ids[i];
      count_occurrence(w, peek_occurrence(w, idlimit, occurs), idlimit, occurs, rare_max);
    }
  }
}

static std::atomic<int> g_rare_update_mode{-1};
void set_rare_update_mode(int mode) { g_rare_update_mode.store(mode >= 0 ? mode : -1); }
int get_rare_update_mode() { return g_rare_update_mode.load(); }

// Decides how many occurrences still make a word of this launch "rare" and counts the words.  A
// launch of `units` work units keeps `waves` of them in flight, so a word with n occurrences has
// about n * waves / units updates in flight together; words for which that is below 1/8 are
// updated without atomics.  Small launches get 0: everything stays atomic and nothing is counted.
// The count is a scattered read-modify-write per id, which is what the device is slowest at, so for
// thresholds that allow it only every 2nd, 4th or 8th run of ids is counted and the threshold
// scaled down: the threshold is a soft one, and a word somewhat above it that slips through is as
// harmless as one just below it.
constexpr int kRareConcurrencyDen = 8;
constexpr int kRareMaxCap = 64;
constexpr int kRareMinSampledMax = 2;   // the scaled threshold is kept at or above this
hipError_t prepare_rare_words(hipStream_t stream, const int* ids_a, int64_t na, const int* ids_b,
                              int64_t nb, int idlimit, int64_t units, int64_t waves,
                              Shadow* shadow, int cap) {
  shadow->rare_max = 0;
  const int mode = g_rare_update_mode.load();
  if (mode == 0 || shadow->occurs == nullptr || waves <= 0) return hipSuccess;
  int64_t most = mode >= 2 ? mode : units / (kRareConcurrencyDen * waves);
  if (cap <= 0 || cap > kRareMaxCap) cap = kRareMaxCap;
  if (most > cap) most = cap;
  if (most < 1) return hipSuccess;
  int every = 1;
  while (every < 8 && most / (2 * every) >= kRareMinSampledMax) every *= 2;
  // a sample needs something to sample from (forced thresholds on small calls)
  while (every > 1 && (nb > 0 && nb < na ? nb : na) / (16 * every) < 4096) every /= 2;
  const int sampled_max = (int)(most / every);
  hipLaunchKernelGGL(clear_occurs_kernel, dim3(256), dim3(kBlock), 0, stream,
                     reinterpret_cast<int4*>(shadow->occurs), kOccurSlots / 4);
  hipLaunchKernelGGL(count_occurs_kernel, dim3(1024), dim3(kBlock), 0, stream, ids_a, na, every,
                     idlimit, shadow->occurs, sampled_max);
  if (nb > 0)
    hipLaunchKernelGGL(count_occurs_kernel, dim3(1024), dim3(kBlock), 0, stream, ids_b, nb, every,
                       idlimit, shadow->occurs, sampled_max);
  shadow->rare_max = sampled_max;
  return hipGetLastError();
}

// Workers of the group-at-a-time kernel when a launch is ordered and the row-by-row kernel has
// no instance for its shape: that order needs 32 or fewer for 1 % of held-out loss.
constexpr int kNegFallbackChains = 32;
constexpr int kMaxTileB = 8;     // B columns a wave holds in registers at once
constexpr int kMaxNwb = kWave;   // lane k of a wave holds the group's k-th B word
int max_nwb() { return kMaxNwb; }

// A columns gathered per chunk, sized so that b, dbb and the chunk stay near 100 registers.
template <int R, int MAXB>
struct NegChunk {
  static constexpr int budget = (100 - 2 * MAXB * R) / R;
  static constexpr int capped = budget > 5 ? 5 : budget;
  static constexpr int value = capped < 1 ? 1 : capped;
};

template <int R, int MAXB>
static hipError_t launch_neg_eval_rb(hipStream_t stream, int d, int ngroups, int nwa, int nwb,
                                     const int* WA, const int* WB, float* A, float* B,
                                     double floorv, double* partials, int64_t* nparts) {
  auto kern = neg_eval_kernel<R, MAXB, NegChunk<R, MAXB>::value>;
  int64_t nwg = 0;
  hipError_t err = persistent_grid(reinterpret_cast<const void*>(kern), kBlock, 0, ngroups,
                                   kMinEvalGroupsPerWg, &nwg);
  if (err != hipSuccess) return err;
  int64_t cap = eval_partials_needed(ngroups);   // what the caller's buffer holds,
  if (*nparts > 0 && *nparts < cap) cap = *nparts;   // unless the caller says it holds less
  if (nwg > cap) nwg = cap;
  const int64_t groups_per_wg = ((int64_t)ngroups + nwg - 1) / nwg;
  nwg = ((int64_t)ngroups + groups_per_wg - 1) / groups_per_wg;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, ngroups, nwa, nwb,
                     groups_per_wg, WA, WB, A, B, floorv, partials);
  *nparts = nwg;
  return hipGetLastError();
}

int64_t ordered_neg_chains(int waves_per_wg, int builtin) {
  int64_t chains = ordered_neg_workers() > 0 ? ordered_neg_workers() : builtin;
  const int limit = get_max_workgroups();
  if (limit > 0 && chains > (int64_t)limit * waves_per_wg) chains = (int64_t)limit * waves_per_wg;
  return chains;
}

template <int R, int MAXB>
static hipError_t launch_neg_train_rb(hipStream_t stream, int d, int ngroups, int idlimit, int nwa,
                                      int nwb, const int* WA, const int* WB, float* A, float* B,
                                      float lrate, float vexp, Shadow shadow) {
  auto kern = neg_train_kernel<R, MAXB, NegChunk<R, MAXB>::value>;
  GridSplit g;
  hipError_t err = split_grid(reinterpret_cast<const void*>(kern), kNegThreads, 0, ngroups,
                              kMinGroupsPerWg, kMinGroupsPerWgWide, &g);
  if (err != hipSuccess) return err;
  // word2vecNegFilt with fewer resident columns than hot ids: no read copies, which are filled
  // from the columns of every hot id the launch holds, resident or not
  const bool copies = idlimit >= kHotWords;
  err = prepare_hot_mode(stream, WB, (int64_t)ngroups * nwb, WA, (int64_t)ngroups * nwa,
                         copies ? A : nullptr, copies ? B : nullptr, d, g.nwg, kNegWaves, &shadow);
  if (err != hipSuccess) return err;
  // only a launch that counts its hot words can turn out cold
  const int64_t nwg = shadow.hot_total > 0 ? g.nwg_wide : g.nwg;
  err = prepare_rare_words(stream, WA, (int64_t)ngroups * nwa, WB, (int64_t)ngroups * nwb, idlimit,
                           ngroups, nwg * kNegWaves, &shadow);
  if (err != hipSuccess) return err;
  // ordered launches: the row-by-row kernel where it has an instance for the shape, else this
  // kernel on a few workgroups
  const bool rows = shadow.ordered != 0 && neg_rows_available(d, nwa);
  const int64_t chains = ordered_neg_chains(kNegWaves, kNegRowWorkers);
  const int limit = get_max_workgroups();
  int64_t per_wg_ordered = 0;
  if (shadow.ordered != 0 && !rows) {
    int64_t wgs = kNegFallbackChains / kNegWaves;
    if (limit > 0 && wgs > limit) wgs = limit;
    if (wgs > nwg) wgs = nwg;   // the grid that is launched
    per_wg_ordered = ((int64_t)ngroups + wgs - 1) / wgs;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kNegThreads), 0, stream, d, ngroups, idlimit,
                     nwa, nwb, g.per_wg, g.per_wg_wide, per_wg_ordered, WA, WB, A, B, lrate, vexp,
                     scale_mode(vexp), shadow);
  err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (rows) {
    err = launch_neg_rows(stream, d, ngroups, idlimit, nwa, nwb, WA, WB, A, B, lrate, vexp, chains,
                          shadow);
    if (err != hipSuccess) return err;
  }
  return launch_fold(stream, A, B, shadow, d);
}

template <int R, bool TRAIN>
static hipError_t launch_neg_r(hipStream_t stream, int d, int ngroups, int idlimit, int nwa, int nwb,
                               const int* WA, const int* WB, float* A, float* B, float lrate,
                               float vexp, double floorv, double* partials, int64_t* nparts,
                               Shadow shadow) {
#define W2V_NEG_DISPATCH(MAXB_)                                                                  \
  return TRAIN ? launch_neg_train_rb<R, MAXB_>(stream, d, ngroups, idlimit, nwa, nwb, WA, WB, A, \
                                               B, lrate, vexp, shadow)                           \
               : launch_neg_eval_rb<R, MAXB_>(stream, d, ngroups, nwa, nwb, WA, WB, A, B, floorv, \
                                              partials, nparts)
  if (nwb <= 2) W2V_NEG_DISPATCH(2);
  if (nwb <= 5) W2V_NEG_DISPATCH(5);
  if (nwb <= kMaxNwb) W2V_NEG_DISPATCH(kMaxTileB);
#undef W2V_NEG_DISPATCH
  return hipErrorInvalidValue;
}

hipError_t launch_neg(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                      const int* WA, const int* WB, float* A, float* B, float lrate, float vexp,
                      Shadow shadow) {
  if (nwb > kMaxTileB)
    return launch_neg_wide(stream, nrows, ncols, idlimit, nwa, nwb, WA, WB, A, B, lrate, vexp,
                           shadow);
  const int rounds = (nrows + kWave - 1) / kWave;
  int64_t unused = 0;
#define CALL(R)                                                                                   \
  return launch_neg_r<R, true>(stream, nrows, ncols, idlimit, nwa, nwb, WA, WB, A, B, lrate, vexp, \
                               0.0, nullptr, &unused, shadow)
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
}

hipError_t launch_eval_neg(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                           const int* WA, const int* WB, const float* A, const float* B,
                           double floorv, double* partials, float* Retval32, double* Retval64,
                           int64_t partials_capacity) {
  const int rounds = (nrows + kWave - 1) / kWave;
  hipError_t err = hipSuccess;
  int64_t nparts = partials_capacity;   // in: capacity of `partials` (0: the default), out: used
#define CALL(R)                                                                                   \
  err = launch_neg_r<R, false>(stream, nrows, ncols, 0, nwa, nwb, WA, WB, const_cast<float*>(A),  \
                               const_cast<float*>(B), 0.0f, 0.0f, floorv, partials, &nparts,      \
                               Shadow{});                                                         \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, nparts, Retval32, Retval64);
}

}  // namespace w2v
