// Device-side building blocks shared by the SGNS kernels (gfx950, wave64).
//
// Work decomposition: one wavefront owns one work unit (a centre token for the
// positive pass, a group of nwa x nwb words for the negative pass).  An embedding
// column of d floats is held by the wave as R = ceil(d/64) registers per lane in
// "dword-strided" layout: lane l holds elements l, l+64, l+128, ...  Every memory
// instruction of the wave (load or float atomic) therefore covers 64 consecutive
// floats = 256 contiguous bytes, so each atomic request that reaches L2 touches
// whole cache lines instead of one dword in every fourth slot.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace w2v {

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWave * kWavesPerBlock;
constexpr int kXcds = 8;       // MI355X: 8 accelerator dies, each with a private L2
constexpr int kMaxRounds = 20; // d <= 1280 on the register-resident path

// vexp handling: scale = (1 + id) ** vexp, evaluated in double then rounded to float
// (jni/src/BIDMach_CPUMACH.c:33,42,215,222 of the reference).
enum ScaleMode : int { kScaleOne = 0, kScaleSqrt = 1, kScaleLinear = 2, kScalePow = 3 };

__device__ __forceinline__ float scale_of(int id, float vexp, int mode) {
  if (mode == kScaleOne) return 1.0f;
  const double x = (double)(1 + id);
  if (mode == kScaleSqrt) return (float)sqrt(x);
  if (mode == kScaleLinear) return (float)x;
  return (float)pow(x, (double)vexp);
}

// Saturating logistic function of the reference CPU path (BIDMach_CPUMACH.c:48-55):
// exactly 1 above 16, exactly 0 below -16, otherwise e/(1+e) with e = (float)exp((double)s).
__device__ __forceinline__ float sat_sigmoid(float s) {
  if (s > 16.0f) return 1.0f;
  if (s < -16.0f) return 0.0f;
  const float e = (float)exp((double)s);
  return e / (1.0f + e);
}

// The same function with the exponential in single precision (v_exp_f32 on s * log2(e), a few
// units in the last place over |s| <= 16) and a reciprocal instead of a division: the value
// differs from sat_sigmoid's by at most a few 1e-7, which the update kernels' tolerance (1e-4 of
// a step that is lrate times it) does not see, and it takes a handful of instructions instead
// of the double-precision exp's sixty.  For the ordered update kernels, whose workers run one
// wave per SIMD with nothing to hide an instruction's latency behind; the forward kernels, whose
// sums of logarithms are held to 1e-5, keep sat_sigmoid.
__device__ __forceinline__ float sat_sigmoid_fast(float s) {
  if (s > 16.0f) return 1.0f;
  if (s < -16.0f) return 0.0f;
  const float e = __expf(s);
  return e * __frcp_rn(1.0f + e);
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

__device__ __forceinline__ float read_lane(float x, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

__device__ __forceinline__ int read_lane(int x, int lane) {
  return __builtin_amdgcn_readlane(x, lane);
}

// Sum over the 64 lanes, result in every lane (and wave-uniform).
// Four DPP rotate-and-add steps inside each 16-lane row (row_ror:8,4,2,1), then the four row
// totals are read out with v_readlane and added.
__device__ __forceinline__ float wave_sum(float x) {
  x += dpp_move<0x128>(x);
  x += dpp_move<0x124>(x);
  x += dpp_move<0x122>(x);
  x += dpp_move<0x121>(x);
  const float r0 = read_lane(x, 0);
  const float r1 = read_lane(x, 16);
  const float r2 = read_lane(x, 32);
  const float r3 = read_lane(x, 48);
  return (r0 + r1) + (r2 + r3);
}

__device__ __forceinline__ double wave_sum_f64(double x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, kWave);
  return x;
}

// Blocks are handed to the 8 XCDs round-robin by the hardware dispatcher.  Remapping the block
// index so that each XCD walks one contiguous range of work units keeps the columns shared by
// neighbouring centre tokens (overlapping windows) inside one XCD's L2.
__device__ __forceinline__ int64_t xcd_contiguous_block(int64_t per_xcd) {
  const int64_t b = blockIdx.x;
  return (b % kXcds) * per_xcd + b / kXcds;
}

template <int R>
__device__ __forceinline__ void load_col(float (&x)[R], const float* __restrict__ col, int lane,
                                         int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    x[r] = (r < R - 1 || e < d) ? col[e] : 0.0f;
  }
}

template <int R>
__device__ __forceinline__ void zero_col(float (&x)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) x[r] = 0.0f;
}

template <int R>
__device__ __forceinline__ float dot_partial(const float (&a)[R], const float (&b)[R]) {
  float s = 0.0f;
#pragma unroll
  for (int r = 0; r < R; ++r) s = fmaf(a[r], b[r], s);
  return s;
}

// y += alpha * x for the lane's slice.
template <int R>
__device__ __forceinline__ void axpy(float (&y)[R], float alpha, const float (&x)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) y[r] = fmaf(alpha, x[r], y[r]);
}

// Hogwild scatter of a column held in the dword-strided register layout: col[e] += x[e] with
// hardware float atomics (global_atomic_add_f32, no return value, no compare-and-swap loop).
//
// The L2 retires atomics per 128-byte line request, and a column starts wherever w*d*4 falls,
// so a wave instruction that covers elements [64r, 64r+64) of the column straddles three lines.
// The lanes are therefore rotated by the column's misalignment (ds_bpermute) so that every
// instruction covers exactly two whole lines: lane l of round r' handles element
// 64*r' + l - mis, where mis = (column start / 4) mod 32.  One extra, mostly empty, round pays
// for roughly a third fewer line requests.
template <int R>
__device__ __forceinline__ void atomic_add_col(float* __restrict__ col, const float (&x)[R],
                                               int lane, int d) {
  const int mis = (int)((reinterpret_cast<uintptr_t>(col) >> 2) & 31u);
  const int src = (lane - mis) & (kWave - 1);
  float prev = 0.0f;
#pragma unroll
  for (int r = 0; r <= R; ++r) {
    float cur = 0.0f;
    if (r < R) cur = __shfl(x[r], src, kWave);
    const float v = (lane >= mis) ? cur : prev;
    const int e = r * kWave + lane - mis;
    if (e >= 0 && e < d) unsafeAtomicAdd(col + e, v);
    prev = cur;
  }
}

// The Hogwild update without atomic adds, for words that occur so rarely in a launch that two
// updates of one column are practically never in flight together (see Shadow::occurs): the column
// is read with load_col_fresh where other columns are read with load_col, and written back as
// fresh + delta.  Both sides bypass the XCD-local L2 (device-scope loads and stores), because plain
// stores of one XCD are not visible to the others while a kernel runs.  What other writers add
// between the load and the store is overwritten.  Without a concurrent writer the result is
// bit-identical to the atomic update.
template <int R>
__device__ __forceinline__ void load_col_fresh(float (&x)[R], const float* col, int lane, int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    x[r] = (r < R - 1 || e < d)
               ? __hip_atomic_load(col + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
               : 0.0f;
  }
}

template <int R>
__device__ __forceinline__ void store_sum_col(float* col, const float (&fresh)[R],
                                              const float (&x)[R], int lane, int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    if (r < R - 1 || e < d)
      __hip_atomic_store(col + e, fresh[r] + x[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int R>
__device__ __forceinline__ void atomic_axpy_col(float* __restrict__ col, float alpha,
                                                const float (&x)[R], int lane, int d) {
  float y[R];
#pragma unroll
  for (int r = 0; r < R; ++r) y[r] = alpha * x[r];
  atomic_add_col<R>(col, y, lane, d);
}

// Shadow copies of the hottest columns.
//
// Word ids are frequency ranks, so under a Zipf law the first few ids each receive hundreds of
// thousands of column updates per call.  Atomics to one cache line retire one after the other in
// L2 (about 36 ns each), and reads of that line queue behind them, which would make those few
// columns the critical path of the whole pass.  The atomics for a hot column therefore go to one
// of several shadow copies of it (chosen by the workgroup index) in a scratch buffer that is zero
// between calls, so the same-line queue is spread over several lines.  A small kernel moves what
// is left in the copies into the table at the end of the call.  Three modes (HotMode):
//
//   off: no shadow copies; every column is read and updated in place.  Chosen inside the kernel,
//       for each of the two tables, when the ids read from that table hold few hot words (counted
//       by a small kernel beforehand, see ids_are_hot), as after frequent-word subsampling.
//   exact (Shadow::combine == 0): while a pass runs, the value of hot column w is
//       table[w] + sum of its copies, and a reader sums them all.  No update is delayed, but the
//       readers of word 0 fetch 17 columns instead of one.  Words 0..7 are hot, with 16, 8, 8, 4,
//       4, 4, 4, 2 copies (the Zipf shares).
//   combining (Shadow::combine == 1): readers read neither the copies nor the table column but a
//       read copy of it (load_col_ref), or the table column where there are no read copies.  What
//       piles up in a copy is moved into the table by its writers: each copy has a write counter, and the
//       writer that brings it to a multiple of kFoldEvery swaps the copy to zero (an atomic
//       exchange, so no concurrent add is lost or counted twice) and adds what it got to the
//       table column.  A reader misses the updates parked in the copies, fewer than kFoldEvery
//       per copy.  Words 0..15 are hot, with 32, 16, 16, 8 x 4, 4 x 8, 2 copies.  The launchers
//       choose this mode only for launches with thousands of work units in flight, where the
//       parked updates are a small addition to the updates that are invisible anyway because
//       their work units are still running.
constexpr int kHotWords = 16;  // hot words of the combining mode; the buffers are sized for it
constexpr int kShadows = 32;   // copies of word 0 in the combining mode
constexpr int kHotWordsExact = 8;
constexpr int kShadowsExact = 16;
constexpr int kFoldEvery = 8;  // power of two; 16 is 6 % faster and parks twice as many updates

constexpr int kCounterStride = 32;  // one write counter per 128-byte line

enum HotMode : int { kHotExact = 0, kHotCombining = 1, kHotOff = 2 };
constexpr int kHotShareDen = 16;  // shadows are used if >= 1/16 of a launch's ids are hot words
constexpr int kHotZeroShareDen = 48;  // or if >= 1/48 of them are id 0
constexpr int kHotCountSlots = 256;  // blocks of the counting kernel, one partial count each

struct Shadow {
  float* a;         // [kShadows][kHotWords][d] for table A
  float* b;         // same for table B
  unsigned* count;  // [2][kShadows][kHotWords][kCounterStride] write counters (B then A); they
                    // only ever count up, so they need no clearing between calls
  // Counted on the device before the launch (count_heavy_kernel), kHotCountSlots partial counts
  // each: how many of the hot_total word ids read from table B belong to the kHotWords most
  // frequent words of the launch, how many to the most frequent one, and the same two for the
  // hot_total_a ids read from table A (0: table A follows table B).  The counts are of
  // occurrences, so they do not depend on how the vocabulary is numbered.  hot_total == 0: not
  // counted, the modes below stand.
  int* hot_seen;
  long long hot_total;
  long long hot_total_a;
  int combine;    // table B: kHotExact or kHotCombining (kHotOff once resolved in a kernel)
  int combine_a;  // table A
  // Rare words.  The float-atomic units are what bounds the update passes, and most of their work
  // is spent on columns that are touched a handful of times per launch, where two updates of the
  // same column are practically never in flight together.  occurs[w & (kOccurSlots - 1)] holds how
  // often word w occurs in the launch (counted on the device beforehand, saturating just above
  // rare_max; slots shared by several words only err towards atomics); a word with at most
  // rare_max occurrences is updated with a plain read-modify-write.  rare_max == 0: every update
  // is atomic.
  int* occurs;
  int rare_max;
  // Read copies of the hot columns for the combining mode: [kXcds][kHotWords][d] per table, one
  // per XCD, or null (then readers read the table).  See load_col_ref.
  float* pub_a;
  float* pub_b;
  int* hot_mask;  // [2][kHotCountSlots] partial bit masks of the hot ids seen: table B's, then A's
  int xcc;        // the XCD this wave runs on (filled in by resolve_hot_mode)
  // Ordered form of the update passes (see launch_is_ordered): 0 never, 1 when the device-side
  // count finds the launch full of frequent words, 2 always.
  int ordered;
  // Ordered form: the frequent columns are kept as grid_c x grid_r delta slots (see
  // load_col_ordered); grid_c == 0: read and updated in place.
  int grid_c;
  int grid_r;
};

constexpr int kOccurSlots = 1 << 20;

// Whether word w (>= 0) of this launch is updated without atomics.  The words that may have
// shadow copies never are.
__device__ __forceinline__ bool is_rare(const Shadow& sh, int w) {
  return sh.rare_max > 0 && w >= kHotWords && sh.occurs[w & (kOccurSlots - 1)] <= sh.rare_max;
}

// The throughput kernels hold a rare A column between its read and its write for the time of a
// chunk of dot products and cannot shorten that by reading it again, as they do for the B columns
// (neg_train_kernel): the A words are held to a limit one count lower, which takes their lost
// share of all contributions below that of the B words.
__device__ __forceinline__ bool is_rare_a(const Shadow& sh, int w) {
  const int limit = sh.rare_max > 1 ? sh.rare_max - 1 : sh.rare_max;
  return sh.rare_max > 0 && w >= kHotWords && sh.occurs[w & (kOccurSlots - 1)] <= limit;
}

// The same in two steps, for a worker that must not wait for the counter where it asks for it:
// rare_seen requests the counter of word w (a value no threshold reaches if w cannot be rare),
// and the word is rare if what arrives is at most sh.rare_max.
__device__ __forceinline__ int rare_seen(const Shadow& sh, int w) {
  return (sh.rare_max > 0 && w >= kHotWords) ? sh.occurs[w & (kOccurSlots - 1)] : 0x7fffffff;
}

// The mode a kernel runs in: the launcher's, unless the ids of this launch hold too few hot words
// for shadow copies to pay (subsampled or re-numbered vocabularies), in which case every column is
// read and updated in place.
// The XCD (0..7) the calling wave runs on: bits 3:0 of hardware register XCC_ID (id 20).
__device__ __forceinline__ int xcc_id() {
  return (int)(__builtin_amdgcn_s_getreg((3 << 11) | 20) & (kXcds - 1));
}

// Sum over the kHotCountSlots partial counts at `part`, the same value in every lane.
__device__ __forceinline__ long long sum_hot_counts(const int* part) {
  int t = 0;
  for (int k = threadIdx.x & 63; k < kHotCountSlots; k += kWave) t += part[k];
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) t += __shfl_xor(t, m, kWave);
  return __builtin_amdgcn_readfirstlane(t);
}

// Whether `total` word ids, `low` of them occurrences of the kHotWords most frequent words and
// `zero` of them of the most frequent one, are full of frequent words: the 16 most frequent are a
// sixteenth of all, or the most frequent alone is a 48th (its atomics retire one after the other,
// and at 5 ids per group a 48th of them already lasts about half as long as the whole pass).
__host__ __device__ __forceinline__ bool ids_are_hot(long long low, long long zero, long long total) {
  return low * kHotShareDen >= total || zero * kHotZeroShareDen >= total;
}

__device__ __forceinline__ Shadow resolve_hot_mode(Shadow sh) {
  sh.xcc = xcc_id();
  if (sh.hot_total > 0) {
    const bool hot_b = ids_are_hot(sum_hot_counts(sh.hot_seen),
                                   sum_hot_counts(sh.hot_seen + kHotCountSlots), sh.hot_total);
    bool hot_a = hot_b;
    if (sh.hot_total_a > 0)
      hot_a = ids_are_hot(sum_hot_counts(sh.hot_seen + 2 * kHotCountSlots),
                          sum_hot_counts(sh.hot_seen + 3 * kHotCountSlots), sh.hot_total_a);
    if (!hot_b) sh.combine = kHotOff;
    if (!hot_a) sh.combine_a = kHotOff;
  }
  return sh;
}

// The mode of table `which` (0 = B, 1 = A).
__device__ __forceinline__ int hot_mode_of(const Shadow& sh, int which) {
  return which ? sh.combine_a : sh.combine;
}

// True if the launch counted its hot words and found too few: such a launch has no column that a
// large share of the units in flight would update, so it may spread over the whole device.
__device__ __forceinline__ bool launch_is_cold(const Shadow& asked, const Shadow& resolved) {
  return asked.hot_total > 0 && asked.combine != kHotOff && resolved.combine == kHotOff &&
         resolved.combine_a == kHotOff;
}

// Keeps the compiler from moving a worker's later reads above its earlier adds.  It is NOT a
// wait: a workgroup-scope release fence emits no s_waitcnt on this target.  What the ordered
// kernels rely on is that requests of one wave to one address are performed in the order they
// were issued (a device-scope load that follows a device-scope atomic add of the same wave to the
// same address returns the sum), which the one-worker sequential-equivalence tests pin; a real
// wait for the adds' acknowledgements is __builtin_amdgcn_s_waitcnt(0), which the team kernel uses
// where the next reader of a column may be another wave.  (An agent-scope release fence adds a
// write-back of the XCD's L2, 6 ms per 1M-token pass, for nothing: every write of these kernels
// is a device-scope atomic, performed at the memory side.)
__device__ __forceinline__ void wait_for_own_writes() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
}

// Teams of wavefronts in the ordered positive kernels (pos_chain_kernel, pos_team_bf16_kernel): a
// wave's lanes look at the window offsets -kChainLook .. kChainLook - 1 of the centre token.
constexpr int kChainLook = 32;

// The wave of a team of `tw` (a power of two) that reads and writes the A column of word `w`.
__device__ __forceinline__ int team_wave(int w, int tw) {
  return (int)(((unsigned)w * 2654435761u) >> 16) & (tw - 1);
}

// A team deals the window's positions to its waves by their place in the token stream (a word
// that stands at several positions belongs, with all of them, to the wave of the first), so a
// column is read and written by one wave while its position moves through consecutive windows,
// and requests of one wave to one address are performed in order.  The order is NOT given where
// a word that this token's window holds, and that has just been updated by the wave of its
// position, belongs to another wave in the next token's window: that wave reads the column a
// fraction of a microsecond after the other wave's add was issued.  True if that can happen, i.e.
// the team has to wait for its adds' acknowledgements before it goes on.  `wl` is the word this
// lane's position holds in this token's window (-1 if none), `wnear` the word at the position
// whatever the window, `nlo`..`nhi` the next token's window (offsets of the next token, clipped
// to the minibatch), `tw` the team's waves.  Only words with one occurrence in this window are
// looked at (after a window with a repeated word the team waits anyway): such a word changes
// hands if a position that the next window newly reaches holds it and becomes its first
// position there, on another wave - because the old position has left the window, or the new
// one lies before it.  A next window beyond the lanes' reach counts as a change of hands.
__device__ __forceinline__ bool window_hands_over(int wl, int wnear, int lane, int nlo, int nhi,
                                                  int tw) {
  if (nlo < -kChainLook || nhi >= kChainLook - 1) return true;
  const int jn = lane - kChainLook - 1;   // this lane's position as an offset of the next token
  const bool in_next = jn >= nlo && jn <= nhi && jn != 0;
  const unsigned long long stays = __ballot(wl >= 0 && in_next);
  unsigned long long enter = __ballot(wl < 0 && wnear >= 0 && in_next);
  while (enter != 0ull) {
    const int e = __builtin_ctzll(enter);
    enter &= enter - 1ull;
    const int we = __builtin_amdgcn_readlane(wnear, e);
    const unsigned long long held = __ballot(wl == we);
    if (held != 0ull) {
      const int p = __builtin_ctzll(held);           // its (first) position in this window
      const bool keeps = ((stays >> p) & 1ull) != 0 && p < e;   // still first in the next window
      if (!keeps && ((p ^ e) & (tw - 1)) != 0) return true;
    }
  }
  return false;
}

// Whether this launch runs in its ordered form.  A launch that is full of frequent words (a raw,
// un-subsampled Zipf stream: a tenth of all tokens are word 0) trains at the edge of stability at
// the reference's step size, and what its result then depends on is how many updates of the
// frequent words' columns a reader misses.  The reference's CPU threads miss a handful (one pair
// per thread in flight); thousands of work units in flight on a whole GPU miss thousands, and a
// tile of adjacent tokens that shares one snapshot of its context columns misses every update
// its own tokens make.  The held-out loss then lands many percent (or many hundred percent) away
// from the reference's.  The ordered kernels (pos_chain_kernel, neg_rows_kernel) keep the
// reference's order inside a worker - a wave walks its tokens / groups one after the other, reads
// every column afresh and adds a B delta to the table before the next read - and keep the number
// of workers at a few dozen, like a large multi-core host.  They run in place of the throughput
// kernels, which return at once, when the count made on the device before the launch finds hot
// words; launches without them (after frequent-word subsampling) keep the throughput kernels.
__device__ __forceinline__ bool launch_is_ordered(const Shadow& asked, const Shadow& resolved) {
  if (asked.ordered == 2) return true;
  return asked.ordered == 1 && asked.hot_total > 0 &&
         !(resolved.combine == kHotOff && resolved.combine_a == kHotOff);
}

__device__ __forceinline__ int shadow_copies(int w, int combine) {
  const int c = (combine == kHotCombining ? kShadows : kShadowsExact) >> (31 - __builtin_clz(w + 1));
  return c < 2 ? 2 : c;
}

// ---- where a word's column lives -------------------------------------------------------------
//
// The kernels that serve both the single-table model and the sliced, multi-part model see the
// model through a small policy object: it turns a word id into a ColRef and answers the two
// questions the sliced model adds (is this pair trained? may this column be written?).

constexpr int kMine = 1;  // sliced model: a tail word this worker owns; single table: any word
constexpr int kHead = 2;  // sliced model: a head word, resident on every worker

struct ColRef {
  float* col;  // start of the column
  int hot;     // index of its shadow copies, or -1 if the column has none
  int flags;   // 0: not resident (skip the word), else kMine or kHead
};

// The shadow index of `ref` in the mode of `shadow`, or -1.
__device__ __forceinline__ int hot_index(const ColRef& ref, int combine) {
  if (combine == kHotOff) return -1;
  return (combine == kHotCombining || ref.hot < kHotWordsExact) ? ref.hot : -1;
}

// ---- the frequent columns in the ordered kernels ------------------------------------------------
//
// What bounds the ordered kernels once they have a few hundred workers is the memory-side queue of
// the few cache lines that hold the most frequent words' columns: every device-scope read and
// every add of one line takes its turn (about 36 ns), and on a raw Zipf stream word 0 alone is
// read 0.4 M times and added to 0.4 M times per 1M-token pass.  While an ordered launch runs, a
// frequent column (ColRef::hot >= 0) is therefore not touched in the table at all.  Its value is
//     table column (unchanged during the launch: plain, cacheable loads)
//   + the sum over c < grid_c of delta slot (c, r),   for any one r < grid_r,
// where the grid_c x grid_r slots live in the shadow buffer of the table (zero between calls).  A
// writer adds its delta to the grid_r slots (c, 0 .. grid_r - 1) of the c its worker number
// selects: the slots (c, r) of one c are replicas of each other up to the order of the float
// adds.  A reader sums the grid_c slots (0 .. grid_c - 1, r) of the r its worker number selects,
// so it sees every update made so far, and one line takes 1/grid_c of the adds and 1/grid_r of the
// reads.  grid_fold_kernel, launched right after the ordered kernel, adds the slots (c, 0) to the
// table and clears them all.
constexpr int kGridMaxC = 8;

__device__ __forceinline__ float* grid_slot(const Shadow& sh, int which, int c, int r, int hot,
                                            int d) {
  return (which ? sh.a : sh.b) + ((int64_t)(c * sh.grid_r + r) * kHotWords + hot) * d;
}

// The column `ref` of table `which` (0 = B, 1 = A) as worker `worker` of an ordered launch sees it.
template <int R>
__device__ __forceinline__ void load_col_ordered(float (&x)[R], const ColRef& ref,
                                                 const Shadow& sh, int which, int64_t worker,
                                                 int lane, int d) {
  if (ref.hot < 0 || sh.grid_c == 0) {
    load_col_fresh<R>(x, ref.col, lane, d);
    return;
  }
  const int twin = (int)((worker / sh.grid_c) % sh.grid_r);
  float y[kGridMaxC][R];
#pragma unroll
  for (int c = 0; c < kGridMaxC; ++c) {
    if (c < sh.grid_c) load_col_fresh<R>(y[c], grid_slot(sh, which, c, twin, ref.hot, d), lane, d);
  }
  load_col<R>(x, ref.col, lane, d);
#pragma unroll
  for (int c = 0; c < kGridMaxC; ++c) {
    if (c < sh.grid_c) {
#pragma unroll
      for (int r = 0; r < R; ++r) x[r] += y[c][r];
    }
  }
}

// col(ref) += x by worker `worker` of an ordered launch.
template <int R>
__device__ __forceinline__ void add_col_ordered(const ColRef& ref, const Shadow& sh, int which,
                                                int64_t worker, const float (&x)[R], int lane,
                                                int d) {
  if (ref.hot < 0 || sh.grid_c == 0) {
    atomic_add_col<R>(ref.col, x, lane, d);
    return;
  }
  const int c = (int)(worker % sh.grid_c);
  for (int r = 0; r < sh.grid_r; ++r)
    atomic_add_col<R>(grid_slot(sh, which, c, r, ref.hot, d), x, lane, d);
}

// The read copy of hot column `hot` of table `which` (0 = B, 1 = A) for this wave's XCD, or null.
__device__ __forceinline__ float* read_copy(const Shadow& sh, int which, int hot, int d) {
  float* const pub = which ? sh.pub_a : sh.pub_b;
  return pub == nullptr ? nullptr : pub + ((int64_t)sh.xcc * kHotWords + hot) * d;
}

// Reads the column `ref` of table `which` (0 = B, 1 = A) as the mode of `sh` sees it.
//   exact: the table column plus all its shadow copies.
//   combining: the table column of a hot word receives the atomics of every fold, and reads of a
//       line queue with the atomics to it, which made these few columns the critical path of the
//       pass.  Readers therefore read a copy that no atomic ever touches: one per XCD (so that
//       plain loads and stores through that XCD's L2 are coherent), filled from the table before
//       the kernel for the hot ids the launch holds and rewritten by every fold done on the XCD
//       with the value its atomic add to the table produced.
template <int R>
__device__ __forceinline__ void load_col_ref(float (&x)[R], const ColRef& ref, const Shadow& sh,
                                             int which, int lane, int d) {
  const int mode = hot_mode_of(sh, which);
  if (mode == kHotCombining && ref.hot >= 0) {
    const float* const pub = read_copy(sh, which, ref.hot, d);
    if (pub != nullptr) {
      load_col<R>(x, pub, lane, d);
      return;
    }
  }
  load_col<R>(x, ref.col, lane, d);
  if (mode == kHotExact && ref.hot >= 0 && ref.hot < kHotWordsExact) {
    // two copies per trip: enough loads in flight without inflating the register count of the
    // callers, which inline this many times
    const float* const shadow = which ? sh.a : sh.b;
    const int copies = shadow_copies(ref.hot, 0);
#pragma unroll 1
    for (int s = 0; s < copies; s += 2) {
      float y0[R], y1[R];
      load_col<R>(y0, shadow + ((int64_t)s * kHotWords + ref.hot) * d, lane, d);
      load_col<R>(y1, shadow + ((int64_t)(s + 1) * kHotWords + ref.hot) * d, lane, d);
#pragma unroll
      for (int r = 0; r < R; ++r) x[r] += y0[r] + y1[r];
    }
  }
}

// Moves what has piled up in a shadow copy into the table column it shadows and, if the column
// has a read copy on this XCD (`pub`, may be null), leaves the column's new value there.
template <int R>
__device__ __forceinline__ void fold_copy(float* __restrict__ copy, float* __restrict__ col,
                                          float* __restrict__ pub, int lane, int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    if (r < R - 1 || e < d) {
      const float v =
          __hip_atomic_exchange(copy + e, 0.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (v != 0.0f) {
        if (pub != nullptr) {
          const float before = unsafeAtomicAdd(col + e, v);
          pub[e] = before + v;
        } else {
          unsafeAtomicAdd(col + e, v);
        }
      }
    }
  }
}

// Announces a write to the column with shadow index `hot` (ColRef::hot; -1 for none) and returns
// the value of its copy's write counter before this write.  Lanes may ask for different columns.
// The returning atomic takes a few microseconds, so callers take the ticket well before the write
// it belongs to.  0 when the write will not go to a combining shadow copy.
__device__ __forceinline__ unsigned hot_ticket(const Shadow& sh, int which, int wg, int hot) {
  if (hot_mode_of(sh, which) != kHotCombining || hot < 0) return 0u;
  const int slot = wg & (shadow_copies(hot, kHotCombining) - 1);
  unsigned* const counter =
      sh.count + (((int64_t)which * kShadows + slot) * kHotWords + hot) * kCounterStride;
  return __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ unsigned read_lane(unsigned x, int lane) {
  return (unsigned)__builtin_amdgcn_readlane((int)x, lane);
}

// col(ref) += x with float atomics.  `which` says which table ref belongs to (0 = B, 1 = A), `wg`
// picks the shadow copy, `ticket` is the wave-uniform result of hot_ticket for this write.
// ref.hot must be wave-uniform.
template <int R>
__device__ __forceinline__ void scatter_add_ref(const ColRef& ref, const Shadow& sh, int which,
                                                int wg, const float (&x)[R], int lane, int d,
                                                unsigned ticket) {
  const int mode = hot_mode_of(sh, which);
  const int hot = hot_index(ref, mode);
  if (hot < 0) {
    atomic_add_col<R>(ref.col, x, lane, d);
    return;
  }
  const int slot = wg & (shadow_copies(hot, mode) - 1);
  float* const copy = (which ? sh.a : sh.b) + ((int64_t)slot * kHotWords + hot) * d;
  atomic_add_col<R>(copy, x, lane, d);
  if (mode == kHotCombining && ((ticket + 1u) & (kFoldEvery - 1)) == 0)
    fold_copy<R>(copy, ref.col, read_copy(sh, which, hot, d), lane, d);
}

// The same for callers on a rarely taken path: takes the ticket on the spot.
template <int R>
__device__ __forceinline__ void scatter_add_ref(const ColRef& ref, const Shadow& sh, int which,
                                                int wg, const float (&x)[R], int lane, int d) {
  const unsigned mine = lane == 0 ? hot_ticket(sh, which, wg, ref.hot) : 0u;
  const unsigned ticket = (unsigned)__builtin_amdgcn_readfirstlane((int)mine);
  scatter_add_ref<R>(ref, sh, which, wg, x, lane, d, ticket);
}

template <int R>
__device__ __forceinline__ void scatter_axpy_ref(const ColRef& ref, const Shadow& sh, int which,
                                                 int wg, float alpha, const float (&x)[R],
                                                 int lane, int d, unsigned ticket) {
  float y[R];
#pragma unroll
  for (int r = 0; r < R; ++r) y[r] = alpha * x[r];
  scatter_add_ref<R>(ref, sh, which, wg, y, lane, d, ticket);
}

template <int R>
__device__ __forceinline__ void scatter_axpy_ref(const ColRef& ref, const Shadow& sh, int which,
                                                 int wg, float alpha, const float (&x)[R],
                                                 int lane, int d) {
  float y[R];
#pragma unroll
  for (int r = 0; r < R; ++r) y[r] = alpha * x[r];
  scatter_add_ref<R>(ref, sh, which, wg, y, lane, d);
}

// Column w of one table, shadowed iff w < kHotWords (for kernels that address a pair of tables by
// word id).
__device__ __forceinline__ ColRef table_ref(float* table, int w, int d) {
  return ColRef{table + (int64_t)w * d, w < kHotWords ? w : -1, kMine};
}

// One pair of tables: word w is column w of A / of B; every pair is trained, every column written.
struct PlainTables {
  float* A;
  float* B;
  static constexpr bool kSliced = false;
  __device__ __forceinline__ ColRef a(int w, int d) const {
    return ColRef{A + (int64_t)w * d, w < kHotWords ? w : -1, w >= 0 ? kMine : 0};
  }
  __device__ __forceinline__ ColRef b(int w, int d) const {
    return ColRef{B + (int64_t)w * d, w < kHotWords ? w : -1, w >= 0 ? kMine : 0};
  }
  __device__ __forceinline__ bool trained(int, int) const { return true; }
  __device__ __forceinline__ bool written(int) const { return true; }
  // the table whose first columns are the frequent (shadowed) ones: 0 = B, 1 = A
  __device__ __forceinline__ float* hot_base(int which) const { return which ? A : B; }
};

// A sliced, multi-part model (jni/src/BIDMach_CPUMACH.c:80-88 of the reference).  The vocabulary
// is split over nslices workers: ids below nhead ("head") are resident on every worker, an id
// >= nhead ("tail") on worker id % nslices only.  A worker packs its resident words densely
// (head, then its tail words in id order: packed column nhead + (id - nhead) / nslices) and cuts
// the packed table into parts of maxcols columns, each part a separate allocation; part m has
// its B table at mats[2m] and its A table at mats[2m+1].  Passed to kernels by value.
constexpr int kMaxSliceParts = 32;
struct SliceMap {
  float* mats[2 * kMaxSliceParts];
  int nparts;   // parts present; a word whose packed column falls beyond them is skipped
  int islice;   // this worker
  int nslices;  // workers the tail of the vocabulary is dealt to
  int nhead;    // ids below this are resident on every worker
  int maxcols;  // columns per part
  int dohead;   // 0: head columns read-only, 1: written, 2: written and head-head pairs trained
};

struct SlicedTables {
  SliceMap m;
  static constexpr bool kSliced = true;
  // which: 0 = B table of the part, 1 = A table
  __device__ __forceinline__ ColRef place(int w, int which, int d) const {
    ColRef r{nullptr, -1, 0};
    if (w < 0) return r;
    const bool head = w < m.nhead;
    const bool mine = !head && (w % m.nslices == m.islice);
    if (!head && !mine) return r;
    const int packed = head ? w : (w - m.nhead) / m.nslices + m.nhead;
    const int part = packed / m.maxcols;
    if (part >= m.nparts) return r;
    r.col = m.mats[2 * part + which] + (int64_t)(packed - part * m.maxcols) * d;
    r.hot = (part == 0 && packed < kHotWords) ? packed : -1;  // the first columns of part 0
    r.flags = head ? kHead : kMine;
    return r;
  }
  __device__ __forceinline__ ColRef a(int w, int d) const { return place(w, 1, d); }
  __device__ __forceinline__ ColRef b(int w, int d) const { return place(w, 0, d); }
  // Rules of the reference (:137-157, :315-349); both words are resident when these are asked.
  __device__ __forceinline__ bool trained(int fa, int fb) const {
    return (((fa | fb) & kMine) != 0) || m.dohead > 1;
  }
  __device__ __forceinline__ bool written(int f) const {
    return f == kMine || (f == kHead && m.dohead > 0);
  }
  __device__ __forceinline__ float* hot_base(int which) const { return m.mats[which ? 1 : 0]; }
};

// After an ordered kernel: adds the delta slots (c, 0) of frequent column blockIdx.x of table
// blockIdx.y (0 = B, 1 = A) to the table column and clears all its slots (load_col_ordered).  A
// column no worker touched has all-zero slots and is left alone, so the vocabulary may be smaller
// than kHotWords.  Does nothing when the launch did not run in its ordered form.
template <class Tables>
__global__ void __launch_bounds__(kBlock)
grid_fold_kernel(Tables tables, Shadow shadow_arg, int d) {
  if (shadow_arg.grid_c == 0) return;
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  if (!launch_is_ordered(shadow_arg, shadow)) return;
  const int w = blockIdx.x, which = blockIdx.y;
  float* const col = tables.hot_base(which) + (int64_t)w * d;
  for (int e = threadIdx.x; e < d; e += kBlock) {
    float sum = 0.0f;
    bool any = false;
    for (int c = 0; c < shadow.grid_c; ++c) {
      for (int r = 0; r < shadow.grid_r; ++r) {
        float* const p = grid_slot(shadow, which, c, r, w, d) + e;
        const float v = *p;
        if (v != 0.0f) {
          any = true;
          if (r == 0) sum += v;
          *p = 0.0f;
        }
      }
    }
    if (any) col[e] += sum;
  }
}

// Block-level sum of one double per wave, written as one partial per block.
__device__ __forceinline__ void block_store_partial(double wave_total, double* __restrict__ partials) {
  __shared__ double s_part[kWavesPerBlock];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  if (lane == 0) s_part[wave] = wave_total;
  __syncthreads();
  if (threadIdx.x == 0) {
    double t = 0.0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) t += s_part[w];
    partials[blockIdx.x] = t;
  }
}

// Launch geometry: 4 waves (work units) per block, grid rounded up to a multiple of the XCD count.
inline int64_t blocks_per_xcd(int64_t units) {
  const int64_t nblocks = (units + kWavesPerBlock - 1) / kWavesPerBlock;
  return (nblocks + kXcds - 1) / kXcds;
}

inline int scale_mode(float vexp) {
  if (vexp == 0.0f) return kScaleOne;
  if (vexp == 0.5f) return kScaleSqrt;
  if (vexp == 1.0f) return kScaleLinear;
  return kScalePow;
}

}  // namespace w2v
