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
// once.
//
// A wave is one worker and walks a contiguous range of groups, as a thread of the reference does
// (:197-201).  What the held-out loss bounds is the number of rows that are between their read and
// their add at any time, summed over the device, and the pass runs at that number divided by the
// time a row spends there: about 2 us for the column to arrive, then the dots, the sigmoid and the
// add.  A row's column is therefore requested only when the row before it is done (requesting
// it one row ahead doubles the rows in flight per worker: the same loss needs half the workers
// and the pass takes 1.4 times as long), and the number of workers is the knob:  held-out loss of
// the 10k-vocabulary configuration on a raw stream against the sequential oracle, 128 positive
// workers: 384: +0.36 %, 480: +0.15 %, 576: -0.06 %, 640: -0.35 %, 768: -0.5 %.
// Registers matter more than occupancy here (a few hundred waves run in all), so up to 16 A
// columns stay resident.
#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

namespace {

// What bounds this kernel once it has a few hundred workers is the memory-side queue of the lines
// that hold the most frequent B words' columns, so those columns are read and updated through the
// delta slots of load_col_ordered / add_col_ordered (w2v_device.h): a line then takes a fraction
// of the adds and a fraction of the reads, and no reader misses an update.  The A columns (the
// negatives) are read and updated in place.
// `tables` places a word's column and, for a sliced model, says which pairs are trained and
// which columns are written (BIDMach_CPUMACH.c:315-349 and :369-381).
template <int R, int MAXA, class Tables>
__global__ void __launch_bounds__(kWave, 1)
neg_rows_kernel(int d, int ngroups, int idlimit, int nwa, int nwb, int64_t per_chain,
                const int* __restrict__ WA, const int* __restrict__ WB, Tables tables,
                float lrate, float vexp, int smode, Shadow shadow_arg) {
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  if (!launch_is_ordered(shadow_arg, shadow)) return;
  const int lane = threadIdx.x;
  const int64_t chain = blockIdx.x;   // a workgroup is one wave is one worker
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

    // Every row's column is read after the adds of the rows before it were issued: requests of
    // one wave to one address are performed in order, so a B word that was a B word of an
    // earlier row of this group is read as that row left it.
    for (int k = 0; k < nwb; ++k) {
      const ColRef rb = tables.b(read_lane(wb_l, k), d);
      if (rb.flags == 0) continue;
      float b[R];
      load_col_ordered<R>(b, rb, shadow, 0, chain, lane, d);
      float pre = 0.0f;
#pragma unroll
      for (int j = 0; j < MAXA; ++j) {
        if (fa[j] != 0 && tables.trained(fa[j], rb.flags)) {
          const float s = wave_sum(dot_partial<R>(a[j], b));
          pre = (lane == j) ? s : pre;
        }
      }
      const float gl = -lrate * sat_sigmoid_fast(pre);
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
      if (tables.written(rb.flags)) add_col_ordered<R>(rb, shadow, 0, chain, dbb, lane, d);
      wait_for_own_writes();
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
  hipLaunchKernelGGL((neg_rows_kernel<R, MAXA, Tables>), dim3((unsigned)chains), dim3(kWave), 0,
                     stream, d, ngroups, idlimit, nwa, nwb, per_chain, WA, WB, tables, lrate, vexp,
                     scale_mode(vexp), shadow);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  return launch_grid_fold(stream, tables, shadow, d);
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
