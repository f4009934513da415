// Ordered form of the negative-sample pass (launch_is_ordered, w2v_device.h): the row-by-row
// order of the reference's CPU loop, jni/src/BIDMach_CPUMACH.c:210-254.
//
// The reference walks a group one B word at a time: it reads that word's column, dots it with the
// group's A columns, and adds the row's delta to the table before it turns to the next B word
// (:219-246); the A columns are written after the last row (:248-254).  The B words of a raw Zipf
// stream are the frequent ones (a tenth of them word 0), so the time between a worker's read of a
// B column and its write is what decides how many updates of that column other workers miss.  The
// throughput kernel (w2v_neg.hip) reads a group's B columns together and writes them after the
// group's last dot; here a wave keeps the group's A columns (the negatives, drawn from the
// flatter unigram^0.75 law) and their accumulators in registers and streams the B columns through
// one row at a time: fresh device-scope read, nwa dots, sigmoid, delta added to the table at
// once.  The next row's column is requested while the current row is worked on.  A lockstep
// simulation of this order stays within 0.2 % of the sequential held-out loss with 256 workers,
// where the group-at-a-time order is 5 % off.
//
// A wave is one worker and walks a contiguous range of groups, as a thread of the reference does
// (:197-201).  Registers matter more than occupancy here (a few hundred waves run in all), so up
// to 16 A columns stay resident.
#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

namespace {

// What bounds this kernel once it has a few hundred workers is the memory-side queue of the lines
// that hold the most frequent B words' columns: every read and every add of a line takes its turn
// (about 36 ns), and on a raw Zipf stream word 0 alone is read 0.4 M times and added to 0.4 M times
// per 1.2 M groups.  The kHotWords most frequent columns of B therefore have kRowTwins twins each
// (the per-XCD read copies of the throughput kernel, filled from the table before the launch,
// serve as the memory): every writer adds its delta to the table column AND to every twin, so a
// twin is the table column up to the order of the float adds, and a reader reads the twin its
// worker number selects: a line then takes all the adds but only a quarter of the reads.  The
// negative pass of a 1.2 M-group launch: 45 ms without twins however many workers, 30 ms with
// four twins on 512 workers, 36 ms on the 384 the library uses.  (Launches large enough for the
// read copies to exist; in a sliced model the frequent columns are the first ones of part 0; the
// twins are not read after the launch.)
constexpr int kRowTwins = 4;
static_assert((kRowTwins & (kRowTwins - 1)) == 0 && kRowTwins <= kXcds, "a power of two of the copies");

// `tables` places a word's column and, for a sliced model, says which pairs are trained and
// which columns are written (BIDMach_CPUMACH.c:315-349 and :369-381).
template <int R, int MAXA, class Tables>
__global__ void __launch_bounds__(kBlock, 1)
neg_rows_kernel(int d, int ngroups, int idlimit, int nwa, int nwb, int64_t per_chain,
                const int* __restrict__ WA, const int* __restrict__ WB, Tables tables,
                float lrate, float vexp, int smode, Shadow shadow_arg) {
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  if (!launch_is_ordered(shadow_arg, shadow)) return;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t chain = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t g_begin = chain * per_chain;
  const int64_t g_end = min(g_begin + per_chain, (int64_t)ngroups);

  int wal = -1, wbl = -1;
  auto fetch = [&](int64_t g) {
    wal = wbl = -1;
    if (g < g_end) {
      if (lane < nwa) wal = WA[g * nwa + lane];
      if (lane < nwb) wbl = WB[g * nwb + lane];
    }
  };
  fetch(g_begin);
  for (int64_t unit = g_begin; unit < g_end; ++unit) {
    int wa_l = wal, wb_l = wbl;
    fetch(unit + 1);
    if (wa_l >= idlimit) wa_l = -1;
    if (wb_l >= idlimit) wb_l = -1;
    const float sal = wa_l >= 0 ? scale_of(wa_l, vexp, smode) : 0.0f;
    const float sbl = wb_l >= 0 ? scale_of(wb_l, vexp, smode) : 0.0f;

    float a[MAXA][R], daa[MAXA][R];
    float* acol[MAXA];
    int fa[MAXA];
#pragma unroll
    for (int j = 0; j < MAXA; ++j) {
      fa[j] = 0;
      acol[j] = nullptr;
      if (j < nwa) {
        const ColRef ra = tables.a(read_lane(wa_l, j), d);
        fa[j] = ra.flags;
        acol[j] = ra.col;
      }
      if (fa[j] != 0) load_col_fresh<R>(a[j], acol[j], lane, d);
      zero_col<R>(daa[j]);
    }

    // a B word that was a B word of an earlier row of this group is read only after that row's
    // delta has been added
    bool seen_before = false;
    for (int k = 0; k < nwb; ++k)
      if (k < lane && read_lane(wb_l, k) == wb_l) seen_before = true;
    const unsigned long long repeats = __ballot(seen_before && wb_l >= 0);

    // Twins of the most frequent B columns (see kRowTwins): a reader takes the twin its worker
    // number selects, a writer adds to the table and to every twin.
    const bool twins = shadow.pub_b != nullptr;
    auto read_b = [&](float (&x)[R], const ColRef& r) {
      const float* src = r.col;
      if (twins && r.hot >= 0)
        src = shadow.pub_b + ((int64_t)(chain & (kRowTwins - 1)) * kHotWords + r.hot) * d;
      load_col_fresh<R>(x, src, lane, d);
    };
    float bn[R];
    ColRef rbn = tables.b(read_lane(wb_l, 0), d);
    if (rbn.flags != 0) read_b(bn, rbn);
    for (int k = 0; k < nwb; ++k) {
      const ColRef rb = rbn;
      float b[R];
#pragma unroll
      for (int r = 0; r < R; ++r) b[r] = bn[r];
      bool again = false;
      if (k + 1 < nwb) {
        rbn = tables.b(read_lane(wb_l, k + 1), d);
        again = rbn.flags != 0 && ((repeats >> (k + 1)) & 1ull) != 0;
        if (rbn.flags != 0 && !again) read_b(bn, rbn);
      }
      if (rb.flags != 0) {
        float pre = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXA; ++j) {
          if (fa[j] != 0 && tables.trained(fa[j], rb.flags)) {
            const float s = wave_sum(dot_partial<R>(a[j], b));
            pre = (lane == j) ? s : pre;
          }
        }
        const float gl = -lrate * sat_sigmoid(pre);
        const float bs = read_lane(sbl, k);
        float dbb[R];
        zero_col<R>(dbb);
#pragma unroll
        for (int j = 0; j < MAXA; ++j) {
          if (fa[j] != 0 && tables.trained(fa[j], rb.flags)) {
            const float g = read_lane(gl, j);
            axpy<R>(dbb, bs * g, a[j]);
            axpy<R>(daa[j], read_lane(sal, j) * g, b);
          }
        }
        if (tables.written(rb.flags)) {
          atomic_add_col<R>(rb.col, dbb, lane, d);
          if (twins && rb.hot >= 0) {
#pragma unroll
            for (int c = 0; c < kRowTwins; ++c)
              atomic_add_col<R>(shadow.pub_b + ((int64_t)c * kHotWords + rb.hot) * d, dbb, lane, d);
          }
        }
      }
      if (again) {
        wait_for_own_writes();
        read_b(bn, rbn);
      }
    }
#pragma unroll
    for (int j = 0; j < MAXA; ++j)
      if (fa[j] != 0 && tables.written(fa[j])) atomic_add_col<R>(acol[j], daa[j], lane, d);
  }
}

constexpr int64_t kMinGroupsPerChain = 16;

template <int R, int MAXA, class Tables>
hipError_t launch_rows(hipStream_t stream, int d, int ngroups, int idlimit, int nwa, int nwb,
                       const int* WA, const int* WB, const Tables& tables, float lrate, float vexp,
                       int64_t chains, const Shadow& shadow) {
  const int64_t by_size = ((int64_t)ngroups + kMinGroupsPerChain - 1) / kMinGroupsPerChain;
  if (chains > by_size) chains = by_size;
  if (chains < 1) chains = 1;
  const int64_t per_chain = ((int64_t)ngroups + chains - 1) / chains;   // waves beyond: empty range
  hipLaunchKernelGGL((neg_rows_kernel<R, MAXA, Tables>),
                     dim3((unsigned)((chains + kWavesPerBlock - 1) / kWavesPerBlock)),
                     dim3(kBlock), 0, stream, d, ngroups, idlimit, nwa, nwb, per_chain, WA, WB,
                     tables, lrate, vexp, scale_mode(vexp), shadow);
  return hipGetLastError();
}

template <class Tables>
hipError_t launch_rows_for(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                           const int* WA, const int* WB, const Tables& tables, float lrate,
                           float vexp, int64_t chains, const Shadow& shadow) {
  const int rounds = (nrows + kWave - 1) / kWave;
  if (nwa <= 5) {
#define CALL(R)                                                                                \
  return launch_rows<R, 5>(stream, nrows, ncols, idlimit, nwa, nwb, WA, WB, tables, lrate, vexp, \
                           chains, shadow)
    W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  }
  if (nwa <= 16 && rounds <= 8) {
    switch (rounds) {
#define CALL(R)                                                                                  \
  case R:                                                                                        \
    return launch_rows<R, 16>(stream, nrows, ncols, idlimit, nwa, nwb, WA, WB, tables, lrate, vexp, \
                              chains, shadow)
      CALL(1); CALL(2); CALL(3); CALL(4); CALL(5); CALL(6); CALL(7); CALL(8);
#undef CALL
      default: break;
    }
  }
  return hipErrorInvalidValue;
}

}  // namespace

bool neg_rows_available(int nrows, int nwa) {
  const int rounds = (nrows + kWave - 1) / kWave;
  return nwa <= 5 || (nwa <= 16 && rounds <= 8);
}

hipError_t launch_neg_rows(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                           const int* WA, const int* WB, float* A, float* B, float lrate,
                           float vexp, int64_t chains, const Shadow& shadow) {
  return launch_rows_for(stream, nrows, ncols, idlimit, nwa, nwb, WA, WB, PlainTables{A, B}, lrate,
                         vexp, chains, shadow);
}

hipError_t launch_slice_neg_rows(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                 const int* WA, const int* WB, const SliceMap& m, float lrate,
                                 float vexp, int64_t chains, const Shadow& shadow) {
  return launch_rows_for(stream, nrows, ncols, 0x7fffffff, nwa, nwb, WA, WB, SlicedTables{m}, lrate,
                         vexp, chains, shadow);
}

}  // namespace w2v
