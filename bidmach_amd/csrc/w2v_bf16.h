// Device-side building blocks of the reduced-precision storage variant: both tables are
// bfloat16, every column is widened to fp32 when it is read, all arithmetic is the fp32 (double
// inside exp / pow / log) arithmetic of the fp32 kernels, and a column is narrowed again with
// stochastic rounding when it is written back.  There are no floating-point atomics on bf16
// pairs that round stochastically, so the write-back is a compare-and-swap of the 4-byte word
// (add_col16 below).
//
// Register layout: a column of d elements is held by the wave as RP = ceil(d / 128) element
// pairs per lane: lane l holds elements 128 r + 2 l and 128 r + 2 l + 1.  With an even d and
// 4-byte aligned tables every column starts on a 4-byte boundary, so a pair is one dword and each
// memory instruction of the wave covers 256 contiguous bytes; otherwise the two halves are moved
// separately.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "w2v_device.h"

namespace w2v {

constexpr int kMaxPairRounds = 10;  // d <= 1280, as for the fp32 tables

// Dispatch on RP; a value without an instance of its own uses the next larger one (the extra
// registers hold zeros and are never stored).
#define W2V_PAIR_ROUNDS_SWITCH(RP_, CALL)                                                   \
  switch (RP_) {                                                                            \
    case 1: CALL(1); case 2: CALL(2); case 3: CALL(3); case 4: CALL(4); case 5: CALL(5);    \
    case 6: CALL(6); case 7: case 8: CALL(8); case 9: case 10: CALL(10);                    \
    default: return hipErrorInvalidValue;                                                   \
  }

__host__ __device__ __forceinline__ uint64_t sr_mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ULL;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

__device__ __forceinline__ uint32_t sr_fmix32(uint32_t h) {
  h ^= h >> 16;
  h *= 0x85EBCA6BU;
  h ^= h >> 13;
  h *= 0xC2B2AE35U;
  h ^= h >> 16;
  return h;
}

// Key of one column write: `unit` is the token (positive pass) or group (negative pass) of the
// call, `slot` the write inside it, `seed` the caller's seed of the call.
__device__ __forceinline__ uint32_t sr_key(uint64_t seed, uint32_t unit, uint32_t slot) {
  return (uint32_t)(sr_mix64(seed ^ sr_mix64(((uint64_t)unit << 32) | slot)) >> 32);
}

// fp32 -> bf16 with 16 random bits added below the kept mantissa: the magnitude rounds up with
// probability (dropped bits) / 65536, so the expectation of the stored value is x.
__device__ __forceinline__ uint32_t sr_narrow(float x, uint32_t key, uint32_t row) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  if ((u & 0x7F800000U) == 0x7F800000U)  // infinity or NaN: keep the class
    return (u >> 16) | ((u & 0x007FFFFFU) ? 0x40U : 0U);
  return (u + (sr_fmix32(key ^ (row * 0x9E3779B9U)) >> 16)) >> 16;
}

// Table columns are read with plain loads, like the fp32 kernels'.  A plain load may be served
// from the CU's own L1 or the XCD's own L2, which other CUs' and XCDs' writes do not reach, so a
// column that stays resident there is read as it was the first time.  That is harmless here for
// two reasons.  The columns that do stay resident are the frequent words', and a frequent word's
// table column does not change while a call runs: its updates go to its side buffer, which is
// read with device-scope loads (add_side_col).  Every other column's line lives in an L2 for tens
// of microseconds at most, and its write-back does not trust what was read: the exchange compares
// against memory and repeats with the value found.  (With plain loads AND plain stores a frequent
// column ended as whichever wave wrote last had left it.)
template <int RP, bool ALIGNED>
__device__ __forceinline__ void load_col16(float (&x)[2 * RP], const uint16_t* col, int lane,
                                           int d) {
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    const int e = r * 128 + 2 * lane;
    if (ALIGNED) {
      uint32_t v = 0;
      if (e < d) v = *reinterpret_cast<const uint32_t*>(col + e);
      x[2 * r] = __builtin_bit_cast(float, v << 16);
      x[2 * r + 1] = __builtin_bit_cast(float, v & 0xFFFF0000U);
    } else {
      const uint32_t lo = (e < d) ? col[e] : 0U;
      const uint32_t hi = (e + 1 < d) ? col[e + 1] : 0U;
      x[2 * r] = __builtin_bit_cast(float, lo << 16);
      x[2 * r + 1] = __builtin_bit_cast(float, hi << 16);
    }
  }
}

// The same with device-scope loads, for the ordered kernels (launch_is_ordered, w2v_device.h),
// whose workers must see each other's, and their own, latest exchanges.
template <int RP, bool ALIGNED>
__device__ __forceinline__ void load_col16_fresh(float (&x)[2 * RP], const uint16_t* col, int lane,
                                                 int d) {
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    const int e = r * 128 + 2 * lane;
    if (ALIGNED) {
      uint32_t v = 0;
      if (e < d)
        v = __hip_atomic_load(reinterpret_cast<const uint32_t*>(col + e), __ATOMIC_RELAXED,
                              __HIP_MEMORY_SCOPE_AGENT);
      x[2 * r] = __builtin_bit_cast(float, v << 16);
      x[2 * r + 1] = __builtin_bit_cast(float, v & 0xFFFF0000U);
    } else {
      // each element out of the aligned word that holds it
      uint32_t lo = 0, hi = 0;
      if (e < d) {
        const uintptr_t addr = reinterpret_cast<uintptr_t>(col + e);
        const uint32_t w = __hip_atomic_load(reinterpret_cast<const uint32_t*>(addr & ~(uintptr_t)3),
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        lo = (addr & 2) ? (w >> 16) : (w & 0xFFFFU);
      }
      if (e + 1 < d) {
        const uintptr_t addr = reinterpret_cast<uintptr_t>(col + e + 1);
        const uint32_t w = __hip_atomic_load(reinterpret_cast<const uint32_t*>(addr & ~(uintptr_t)3),
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        hi = (addr & 2) ? (w >> 16) : (w & 0xFFFFU);
      }
      x[2 * r] = __builtin_bit_cast(float, lo << 16);
      x[2 * r + 1] = __builtin_bit_cast(float, hi << 16);
    }
  }
}

__device__ __forceinline__ uint32_t cas_word(uint32_t* p, uint32_t expected, uint32_t desired) {
  __hip_atomic_compare_exchange_strong(p, &expected, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
  return expected;  // the value found: equal to the guess iff the exchange took place
}

// col[e] = narrow(widen(col[e]) + delta[e]) for the lane's elements, as a compare-and-swap on the
// 4-byte word that holds them, so that no update of the column by another wave is lost: a store
// of "what I read plus my delta" would wipe out whatever was added in between, and with
// thousands of waves in flight the frequent words would lose most of their updates.  `seen` is
// the column as this wave read it (the first guess; the exchange fails and is repeated with the
// value found if the column has changed since).  The random bits depend on (key, row) only, so a
// repeated attempt rounds the same way.
// First round of the exchange for a column of 4-byte words: the words are issued and their
// results left in `found`, not waited for, so that a caller can put the exchanges of several
// columns (or a load it will need next) in flight before the first result is looked at.
template <int RP>
__device__ __forceinline__ void cas_first(uint16_t* col, const float (&seen)[2 * RP],
                                          const float (&delta)[2 * RP], int lane, int d,
                                          uint32_t key, uint32_t (&guess)[RP],
                                          uint32_t (&found)[RP]) {
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    const int e = r * 128 + 2 * lane;
    guess[r] = (__builtin_bit_cast(uint32_t, seen[2 * r]) >> 16) |
               (__builtin_bit_cast(uint32_t, seen[2 * r + 1]) & 0xFFFF0000U);
    found[r] = guess[r];
    if (e < d) {
      const float lo = seen[2 * r] + delta[2 * r];
      const float hi = seen[2 * r + 1] + delta[2 * r + 1];
      const uint32_t want = sr_narrow(lo, key, (uint32_t)e) |
                            (sr_narrow(hi, key, (uint32_t)(e + 1)) << 16);
      found[r] = cas_word(reinterpret_cast<uint32_t*>(col + e), guess[r], want);
    }
  }
}

// Looks at the results of cas_first and repeats the words that found another value, with that
// value as the new guess, until every word has been exchanged.
template <int RP>
__device__ __forceinline__ void cas_rest(uint16_t* col, const float (&delta)[2 * RP], int lane,
                                         int d, uint32_t key, uint32_t (&guess)[RP],
                                         uint32_t (&found)[RP]) {
  bool open[RP];
  bool any = false;
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    open[r] = found[r] != guess[r];   // words beyond d were never issued: found == guess
    guess[r] = found[r];
    any = any || open[r];
  }
  while (any) {
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      if (open[r]) {
        const int e = r * 128 + 2 * lane;
        const float lo = __builtin_bit_cast(float, guess[r] << 16) + delta[2 * r];
        const float hi = __builtin_bit_cast(float, guess[r] & 0xFFFF0000U) + delta[2 * r + 1];
        const uint32_t want = sr_narrow(lo, key, (uint32_t)e) |
                              (sr_narrow(hi, key, (uint32_t)(e + 1)) << 16);
        found[r] = cas_word(reinterpret_cast<uint32_t*>(col + e), guess[r], want);
      }
    }
    any = false;
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      if (open[r]) {
        open[r] = found[r] != guess[r];
        guess[r] = found[r];
        any = any || open[r];
      }
    }
  }
}

// cas_rest for a delta of the form scale * x, formed again where a word has to be repeated, so
// that a caller with many exchanges in flight need not keep their deltas.
template <int RP>
__device__ __forceinline__ void cas_rest_axpy(uint16_t* col, float scale, const float (&x)[2 * RP],
                                              int lane, int d, uint32_t key, uint32_t (&guess)[RP],
                                              uint32_t (&found)[RP]) {
  bool any = false;
#pragma unroll
  for (int r = 0; r < RP; ++r) any = any || found[r] != guess[r];
  if (__ballot(any) == 0ull) return;   // the usual case: every word was exchanged at once
  float delta[2 * RP];
#pragma unroll
  for (int r = 0; r < 2 * RP; ++r) delta[r] = scale * x[r];
  cas_rest<RP>(col, delta, lane, d, key, guess, found);
}

template <int RP, bool ALIGNED>
__device__ __forceinline__ void add_col16(uint16_t* col, const float (&seen)[2 * RP],
                                          const float (&delta)[2 * RP], int lane, int d,
                                          uint32_t key) {
  if (ALIGNED) {
    uint32_t guess[RP], found[RP];
    cas_first<RP>(col, seen, delta, lane, d, key, guess, found);
    cas_rest<RP>(col, delta, lane, d, key, guess, found);
  } else {
    // columns on 2-byte boundaries: each element is exchanged inside the aligned word that
    // holds it, the other half of the word being written back as found
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) {
      const int e = (r >> 1) * 128 + 2 * lane + (r & 1);
      if (e < d) {
        const uintptr_t addr = reinterpret_cast<uintptr_t>(col + e);
        uint32_t* word = reinterpret_cast<uint32_t*>(addr & ~(uintptr_t)3);
        const int shift = (addr & 2) ? 16 : 0;
        uint32_t guess = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (;;) {
          const float x = __builtin_bit_cast(float, ((guess >> shift) & 0xFFFFU) << 16) + delta[r];
          const uint32_t want = (guess & ~(0xFFFFU << shift)) |
                                (sr_narrow(x, key, (uint32_t)e) << shift);
          const uint32_t found = cas_word(word, guess, want);
          if (found == guess) break;
          guess = found;
        }
      }
    }
  }
}

// col[e] = narrow(seen[e] + delta[e]) for the lane's elements with plain device-scope stores: no
// exchange, nothing to wait for.  What another wave added to the column between this wave's read
// of `seen` and this store is overwritten, so this is for the words that are rare within a launch
// of the ordered kernels (a few hundred workers, each between a column's read and its write for a
// few microseconds: two updates of a word that occurs a handful of times practically never
// overlap), and it is the closest this library gets to the atomic-free stochastic-rounded
// write-back of bfloat16 tables.  Same random bits as the exchange: without an overlapping update
// the stored bits are the same.
template <int RP, bool ALIGNED>
__device__ __forceinline__ void store_col16(uint16_t* col, const float (&seen)[2 * RP],
                                            const float (&delta)[2 * RP], int lane, int d,
                                            uint32_t key) {
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    const int e = r * 128 + 2 * lane;
    if (e < d) {
      const uint32_t lo = sr_narrow(seen[2 * r] + delta[2 * r], key, (uint32_t)e);
      if (ALIGNED) {
        // (an odd d is never ALIGNED, so e + 1 < d here)
        const uint32_t hi = sr_narrow(seen[2 * r + 1] + delta[2 * r + 1], key, (uint32_t)(e + 1));
        __hip_atomic_store(reinterpret_cast<uint32_t*>(col + e), lo | (hi << 16), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      } else {
        __hip_atomic_store(col + e, (uint16_t)lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (e + 1 < d)
          __hip_atomic_store(col + e + 1,
                             (uint16_t)sr_narrow(seen[2 * r + 1] + delta[2 * r + 1], key,
                                                 (uint32_t)(e + 1)),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

// Frequent words.  Word ids are frequency ranks, so the first few hundred ids take most of the
// updates of a call, and a compare-and-swap on a column that thousands of waves update at once
// fails nearly every time.  The columns of the words below `n` therefore have an fp32 side
// buffer each (sa for table A, sb for table B; side_columns(n) x side_stride(d) floats, zero
// between calls): while a call
// runs, the value of such a column is widen(table) + side buffer, readers add the two in fp32,
// and writers add their delta to the side buffer with float atomics, which need no retry.  A small
// kernel at the end of the call narrows table + side buffer back into the table (one stochastic
// rounding per element and call instead of one per update) and clears the side buffer.
struct HotCols {
  float* sa;
  float* sb;
  int n;
};

// Inside a side buffer a column is stored in the order the wave holds it: the lane's first
// elements of a round, then its second ones (element 128 r + 2 l + h sits at 128 r + 64 h + l),
// padded to whole rounds.  A float-atomic instruction of the wave then covers 64 consecutive
// floats, two whole cache lines, and an update touches every line of the column once; in element
// order it would touch every line twice, and the updates of the most frequent word, which retire
// one after the other on each of its lines, are the critical path of a call.
__host__ __device__ __forceinline__ int side_stride(int d) { return (d + 127) / 128 * 128; }

template <int RP>
__device__ __forceinline__ void add_side_col(float (&x)[2 * RP], const float* side, int lane,
                                             int d) {
#pragma unroll
  for (int r = 0; r < 2 * RP; ++r) {
    const int e = (r >> 1) * 128 + 2 * lane + (r & 1);
    if (e < d)
      x[r] += __hip_atomic_load(side + (r >> 1) * 128 + (r & 1) * 64 + lane, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
  }
}

// The same in two steps, for callers that want several columns in flight before the first value
// is used: side_col_request leaves the side column's values in s (zero beyond d), side_col_add adds
// them.  (add_side_col uses each value as it names it, so a caller that gathers column after
// column with it waits for every column before it asks for the next.)
template <int RP>
__device__ __forceinline__ void side_col_request(float (&s)[2 * RP], const float* side, int lane,
                                                 int d) {
#pragma unroll
  for (int r = 0; r < 2 * RP; ++r) {
    const int e = (r >> 1) * 128 + 2 * lane + (r & 1);
    s[r] = 0.0f;
    if (e < d)
      s[r] = __hip_atomic_load(side + (r >> 1) * 128 + (r & 1) * 64 + lane, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int RP>
__device__ __forceinline__ void side_col_add(float (&x)[2 * RP], const float (&s)[2 * RP]) {
#pragma unroll
  for (int r = 0; r < 2 * RP; ++r) x[r] += s[r];
}

template <int RP>
__device__ __forceinline__ void atomic_add_side_col(float* side, const float (&delta)[2 * RP],
                                                    int lane, int d) {
#pragma unroll
  for (int r = 0; r < 2 * RP; ++r) {
    const int e = (r >> 1) * 128 + 2 * lane + (r & 1);
    if (e < d) atomicAdd(side + (r >> 1) * 128 + (r & 1) * 64 + lane, delta[r]);
  }
}

// The few most frequent words.  Requests to one cache line retire one after the other, and the
// reads and float atomics of the most frequent word's side-buffer lines are the longest such
// chain of a call.  The first kTopWords words therefore have kTopCopies side columns each (the
// main one and kTopCopies - 1 more, stored after the hot.n main columns: copy c >= 1 of word w is
// column hot.n + (c - 1) kTopWords + w): a writer adds to the copy its wave index selects, a
// reader sums all copies, so the value read is still every update made so far while a line takes
// a quarter of the atomics.  Used when hot.n >= kTopWords.
constexpr int kTopWords = 8;
constexpr int kTopCopies = 4;

__host__ __device__ __forceinline__ int side_columns(int hot_n) {
  return hot_n + (hot_n >= kTopWords ? (kTopCopies - 1) * kTopWords : 0);
}

template <int RP>
__device__ __forceinline__ void read_side(float (&x)[2 * RP], const float* base, int hot_n, int w,
                                          int lane, int d) {
  const int64_t stride = side_stride(d);
  add_side_col<RP>(x, base + (int64_t)w * stride, lane, d);
  if (w < kTopWords && hot_n >= kTopWords) {
#pragma unroll
    for (int c = 1; c < kTopCopies; ++c)
      add_side_col<RP>(x, base + ((int64_t)hot_n + (c - 1) * kTopWords + w) * stride, lane, d);
  }
}

// The ordered kernels (a few hundred workers) read and write the main side column only, with one
// exception: the row-by-row kernel of the negative pass uses the kTopCopies side columns of table
// B's kTopWords most frequent words as a 2 x 2 grid of delta slots: slot g = 2 c + r is the main
// column for g = 0 and extra column g - 1 otherwise; a writer adds its delta to both twins
// r = 0, 1 of the copy c its worker number selects, a reader sums one twin r of both copies.
// Every reader still sees every update made so far, and a column takes half of the adds and half
// of the reads.  On a raw Zipf(1.1) stream one word is 13 % of the context words, and the
// requests to its columns are served one after the other: from about 400 workers on the pass
// does not get faster (55 ms per 1.2M groups at vocab 3M, with the slots 41 ms at 576 workers and
// 37 ms at 768).  The positive kernel, whose workers are fewer, only pays for the second column
// (teams of 160: 71 ms with the slots, 65 ms without) and stays with the main column.  The
// end-of-call narrowing then sums twin 0 of both copies (fold_bf16_kernel).
static_assert(kTopCopies == 4, "the ordered kernels lay the copies out as 2 x 2");

__device__ __forceinline__ int64_t side_slot_column(int hot_n, int w, int g) {
  return g == 0 ? (int64_t)w : (int64_t)hot_n + (g - 1) * kTopWords + w;
}

__device__ __forceinline__ bool has_side_slots(int hot_n, int w) {
  return w < kTopWords && hot_n >= kTopWords;
}

// Requests what a reader of frequent word w needs (side_col_request: nothing is used yet): the
// main side column into s, or twin r of both copies into s and s2.
template <int RP>
__device__ __forceinline__ void side_request_ordered(float (&s)[2 * RP], float (&s2)[2 * RP],
                                                     const float* base, int hot_n, int w,
                                                     int64_t worker, int lane, int d) {
  const int64_t stride = side_stride(d);
  if (has_side_slots(hot_n, w)) {
    const int r = (int)(worker >> 1) & 1;
    side_col_request<RP>(s, base + side_slot_column(hot_n, w, r) * stride, lane, d);
    side_col_request<RP>(s2, base + side_slot_column(hot_n, w, 2 + r) * stride, lane, d);
  } else {
    side_col_request<RP>(s, base + (int64_t)w * stride, lane, d);
  }
}

template <int RP>
__device__ __forceinline__ void side_add_ordered(float (&x)[2 * RP], const float (&s)[2 * RP],
                                                 const float (&s2)[2 * RP], int hot_n, int w) {
  side_col_add<RP>(x, s);
  if (has_side_slots(hot_n, w)) side_col_add<RP>(x, s2);
}

// Table A in the ordered kernels (the centre words and the negatives: no word takes a large
// share of its updates) keeps to the main side column.
template <int RP>
__device__ __forceinline__ void write_side_main(float* base, int w, const float (&delta)[2 * RP],
                                                int lane, int d) {
  atomic_add_side_col<RP>(base + (int64_t)w * side_stride(d), delta, lane, d);
}

template <int RP>
__device__ __forceinline__ void write_side_ordered(float* base, int hot_n, int w, int64_t worker,
                                                   const float (&delta)[2 * RP], int lane, int d) {
  const int64_t stride = side_stride(d);
  if (has_side_slots(hot_n, w)) {
    const int c = (int)worker & 1;
    atomic_add_side_col<RP>(base + side_slot_column(hot_n, w, 2 * c) * stride, delta, lane, d);
    atomic_add_side_col<RP>(base + side_slot_column(hot_n, w, 2 * c + 1) * stride, delta, lane, d);
  } else {
    atomic_add_side_col<RP>(base + (int64_t)w * stride, delta, lane, d);
  }
}

template <int RP>
__device__ __forceinline__ void write_side(float* base, int hot_n, int w, int copy,
                                           const float (&delta)[2 * RP], int lane, int d) {
  const int64_t stride = side_stride(d);
  int64_t column = w;
  if (w < kTopWords && hot_n >= kTopWords && copy > 0)
    column = (int64_t)hot_n + (copy - 1) * kTopWords + w;
  atomic_add_side_col<RP>(base + column * stride, delta, lane, d);
}

// Slot of the end-of-call narrowing of a frequent word's column in the random-bit key (the unit
// is 0xFFFFFFFF, which no token or group index reaches).
__host__ __device__ __forceinline__ uint32_t fold_slot(int table_b, int word) {
  return ((uint32_t)table_b << 31) | (uint32_t)word;
}

// Launchers (enqueue only).  Tables are bf16, nrows x vocab, column-major.
// `hot` holds zeroed side buffers of side_columns(hot.n) x side_stride(nrows) floats each (hot.n may be 0); the update
// launchers leave them zeroed (they enqueue the narrowing kernel after the update kernel).
// `shadow` lends the launch the thread's hot-word counters: a launch that its device-side count
// finds full of frequent words runs in its ordered form (launch_is_ordered, w2v_device.h).
hipError_t launch_pos_bf16(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                           const int* LB, const int* UB, uint16_t* A, uint16_t* B, float lrate,
                           float vexp, uint64_t seed, HotCols hot, Shadow shadow);
hipError_t launch_neg_bf16(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                           const int* WA, const int* WB, uint16_t* A, uint16_t* B, float lrate,
                           float vexp, uint64_t seed, HotCols hot, Shadow shadow);
// Ordered form of the positive pass (w2v_bf16_pos_chain.hip): counts the words that are rare
// within the launch and enqueues the worker kernel; `aligned` as pair_aligned() found the tables.
hipError_t launch_pos_chain_bf16(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                                 const int* LB, const int* UB, uint16_t* A, uint16_t* B,
                                 float lrate, float vexp, uint64_t seed, HotCols hot,
                                 const Shadow& shadow, bool aligned);
// Ordered form of the negative pass (w2v_bf16_neg_rows.hip); false if the shape has no instance.
bool neg_rows_bf16_available(int nrows, int nwa);
hipError_t launch_neg_rows_bf16(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                const int* WA, const int* WB, uint16_t* A, uint16_t* B,
                                float lrate, float vexp, uint64_t seed, HotCols hot,
                                int64_t chains, const Shadow& shadow);
hipError_t launch_neg_rows_bf16_unaligned(hipStream_t stream, int nrows, int ncols, int nwa,
                                          int nwb, const int* WA, const int* WB, uint16_t* A,
                                          uint16_t* B, float lrate, float vexp, uint64_t seed,
                                          HotCols hot, int64_t chains, const Shadow& shadow);
// `slots_if_ordered`: the launch's ordered kernel (if the device-side decision is for it) used the
// most frequent words' side columns as delta slots with twins (side_request_ordered).
hipError_t launch_fold_bf16(hipStream_t stream, int nrows, uint16_t* A, uint16_t* B, uint64_t seed,
                            HotCols hot, const Shadow& shadow, bool slots_if_ordered);
// The forward twins add their sum into the device double Retval[0].
hipError_t launch_eval_pos_bf16(hipStream_t stream, int nrows, int ncols, const int* W,
                                const int* LB, const int* UB, const uint16_t* A,
                                const uint16_t* B, double floorv, double* Retval);
hipError_t launch_eval_neg_bf16(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                const int* WA, const int* WB, const uint16_t* A,
                                const uint16_t* B, double floorv, double* Retval);

// Whole-table conversions: fp32 -> bf16 rounds to nearest, ties to even; bf16 -> fp32 is exact.
hipError_t launch_f32_to_bf16(hipStream_t stream, size_t n, const float* src, uint16_t* dst);
hipError_t launch_bf16_to_f32(hipStream_t stream, size_t n, const uint16_t* src, float* dst);

}  // namespace w2v
