// Host-side declarations shared between the launchers and the C-ABI file.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Dispatch on R = ceil(nrows / 64), the registers per lane that hold one column.
#define W2V_ROUNDS_SWITCH(R_, CALL)                                                        \
  switch (R_) {                                                                            \
    case 1: CALL(1); case 2: CALL(2); case 3: CALL(3); case 4: CALL(4); case 5: CALL(5);   \
    case 6: CALL(6); case 7: CALL(7); case 8: CALL(8); case 9: CALL(9); case 10: CALL(10); \
    case 11: CALL(11); case 12: CALL(12); case 13: CALL(13); case 14: CALL(14);            \
    case 15: CALL(15); case 16: CALL(16); case 17: CALL(17); case 18: CALL(18);            \
    case 19: CALL(19); case 20: CALL(20);                                                  \
    default: return hipErrorInvalidValue;                                                  \
  }

#include "w2v_device.h"

namespace w2v {

// Bytes of one shadow buffer (one per table): kShadows copies of kHotWords columns of up to
// max_rows() floats.  The caller of launch_pos / launch_neg provides both buffers zeroed; the
// launchers leave them zeroed.
size_t shadow_bytes();
// Bytes of the write counters of both tables' shadow copies plus the partial hot-word counts of a
// launch (zero-initialised once; the counters are never cleared, the counts are rewritten by every
// counting launch).
size_t shadow_counter_bytes();

// Grid size of a persistent kernel: the workgroups that fit on the device at once, but no more
// than `units / min_units_per_wg` (a workgroup walks at least that many work units, so a small
// minibatch is not spread over the whole device: fewer units in flight means less stale Hogwild
// updates), and no more than the caller's limit (set_max_workgroups, 0 = none).
struct GridSplit {
  int64_t nwg, per_wg;            // bounded grid: workgroups and units per workgroup
  int64_t nwg_wide, per_wg_wide;  // device-filling grid (never smaller than the bounded one)
};
hipError_t split_grid(const void* kernel, int threads, size_t lds_bytes, int64_t units,
                      int64_t min_units, int64_t min_units_wide, GridSplit* out);
hipError_t persistent_grid(const void* kernel, int threads, size_t lds_bytes, int64_t units,
                           int64_t min_units_per_wg, int64_t* nwg);
void set_max_workgroups(int n);
int get_max_workgroups();

// How the hottest columns are updated (w2v_device.h): -1 chosen per launch (the default), 0 exact,
// 1 combining.  prepare_hot_mode fills in the mode fields of `shadow` for a launch of nwg workgroups
// of waves_per_wg waves over the n word ids `ids` (device memory); in the default mode it first
// enqueues the count of hot words among them.
void set_hot_update_mode(int mode);
int get_hot_update_mode();
void set_rare_update_mode(int mode);
int get_rare_update_mode();
size_t occurs_bytes();
// `ids` are the words read from table B (and counted), `ids2` those read from table A (null: the
// same); A and B are the tables whose hot columns get read copies in the combining mode (null:
// none, readers read the tables).
hipError_t prepare_hot_mode(hipStream_t stream, const int* ids, int64_t n, const int* ids2,
                            int64_t n2, const float* A, const float* B, int d, int64_t nwg,
                            int waves_per_wg, Shadow* shadow);
// What prepare_hot_mode left for the calling thread's most recent update launch (the counters it
// points to are the launch's own until the thread's next update launch): for w2v_last_launch_form.
// Null before the thread's first update launch.
const Shadow* last_launch_shadow();
void note_last_launch(const Shadow& shadow);
// The same for a sliced model, whose shadowed columns are the first columns of part 0.
hipError_t prepare_hot_mode_sliced(hipStream_t stream, const int* ids, int64_t n, const int* ids2,
                                   int64_t n2, const SliceMap& m, int d, int64_t nwg,
                                   int waves_per_wg, Shadow* shadow);
size_t read_copy_bytes();
// Decides which words of a launch over `units` work units, `waves` of them in flight, are rare
// enough for plain read-modify-write updates (Shadow::rare_max) and enqueues the count of the
// words in the two id arrays (ids at or beyond idlimit are ignored).
// cap: the largest number of occurrences that may still count as rare (0: the built-in 64).
hipError_t prepare_rare_words(hipStream_t stream, const int* ids_a, int64_t na, const int* ids_b,
                              int64_t nb, int idlimit, int64_t units, int64_t waves,
                              Shadow* shadow, int cap = 0);
// For kernels that only read: no shadow copies anywhere.
inline Shadow no_shadow() {
  Shadow s{};
  s.combine = kHotOff;
  s.combine_a = kHotOff;
  return s;
}

// Adds the shadow copies of the hot columns into A and B and zeroes them.
hipError_t launch_fold(hipStream_t stream, float* A, float* B, Shadow shadow, int d);

// Enqueued right after an ordered kernel: moves its delta slots into the tables (grid_fold_kernel).
template <class Tables>
inline hipError_t launch_grid_fold(hipStream_t stream, const Tables& tables, const Shadow& shadow,
                                   int d) {
  if (shadow.grid_c == 0) return hipSuccess;
  hipLaunchKernelGGL((grid_fold_kernel<Tables>), dim3(kHotWords, 2), dim3(kBlock), 0, stream,
                     tables, shadow, d);
  return hipGetLastError();
}
// Delta slots of the frequent columns in the ordered kernels (load_col_ordered): copies x twins,
// copies * twins <= 32, copies <= 8; copies == 0 switches them off.
void set_ordered_copies(int copies, int twins);
void get_ordered_copies(int* copies, int* twins);

// Number of per-block partial sums an Eval launch over `units` work units writes.
int64_t eval_partials_needed(int64_t units);

// All launchers enqueue on `stream` and return the launch status; none of them synchronises.
// `shift` is the caller's maximum window half-width; it sizes the halo a tile stages in LDS.
// Offsets beyond it are still processed (gathered from memory), so any LB/UB is accepted.
hipError_t launch_pos(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                      const int* LB, const int* UB, float* A, float* B, float lrate, float vexp,
                      Shadow shadow);

// Word ids >= idlimit (and negative ids) are skipped with every pair they take part in.
hipError_t launch_neg(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                      const int* WA, const int* WB, float* A, float* B, float lrate, float vexp,
                      Shadow shadow);

// The same pass for groups with more than 8 B words (w2v_neg_wide.hip): the group's A columns are
// staged in LDS, so nwa * ceil(nrows / 64) is bounded (hipErrorInvalidValue beyond, about 300).
// `shadow` lends the launch the hot-word counters: a launch full of frequent words goes to the
// row-by-row kernel below where that has an instance for the shape.
hipError_t launch_neg_wide(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                           const int* WA, const int* WB, float* A, float* B, float lrate,
                           float vexp, const Shadow& shadow);
hipError_t launch_slice_neg_wide(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                 const int* WA, const int* WB, const SliceMap& m, float lrate,
                                 float vexp, const Shadow& shadow);

// Ordered form of the negative pass (w2v_neg_rows.hip), for launches whose device-side count
// finds them full of frequent words: `chains` waves walk the groups row by row in the
// reference's order.  It keeps the group's A columns in registers, so not every shape has an
// instance (neg_rows_available).  Launched after the throughput kernel, which returns at once
// when the launch is ordered, as this one does when it is not.
bool neg_rows_available(int nrows, int nwa);
// Workers of the ordered kernels: the caller's built-in number (or what w2v_set_ordered_workers
// asks for), within the bound on workgroups.
constexpr int kNegRowWorkers = 576;        // fp32 row-by-row kernel, one row in flight per worker
constexpr int kNegRowWorkersBf16 = 384;    // bfloat16 row-by-row kernel, which requests a row ahead
// Ordered bfloat16 kernels: a word with at most this many occurrences in the launch is written back
// with a plain store instead of a compare-and-swap (w2v_bf16.h, store_col16).
constexpr int kRareCapOrderedBf16 = 16;
constexpr int kPosTeams = 192;             // fp32 positive kernel, teams of kTeamWaves waves
constexpr int kPosChainsBf16 = 128;        // bfloat16 positive kernel, single waves
constexpr int kPosTeamsBf16 = 160;         // bfloat16 positive kernel, teams of kTeamWaves waves
constexpr int kTeamWaves = 4;
int64_t ordered_neg_chains(int waves_per_wg, int builtin);
int64_t ordered_pos_chains(int ncols, int shift, int builtin);
hipError_t launch_neg_rows(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                           const int* WA, const int* WB, float* A, float* B, float lrate,
                           float vexp, int64_t chains, const Shadow& shadow);
hipError_t launch_slice_neg_rows(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                 const int* WA, const int* WB, const SliceMap& m, float lrate,
                                 float vexp, int64_t chains, const Shadow& shadow);
// Ordered form: -1 (default) chosen per launch on the device, 0 never, 1 always.
void set_ordered_mode(int mode);
int get_ordered_mode();
int ordered_flag(bool forced_hot_mode);   // the value of Shadow::ordered for a launch
// Workers (wavefronts) of the ordered kernels; 0 = the built-in numbers.
void set_ordered_workers(int pos, int neg);
int ordered_pos_workers();
int ordered_neg_workers();

// Eval launchers write one double per block into `partials` (capacity >= eval_partials_needed)
// and then fold them, in a fixed order, into Retval32[0] (float, added into) and/or
// Retval64[0] (double, added into).  Either output pointer may be null.
hipError_t launch_eval_pos(hipStream_t stream, int nrows, int ncols, const int* W, const int* LB,
                           const int* UB, const float* A, const float* B, double floorv,
                           double* partials, float* Retval32, double* Retval64);

// partials_capacity: doubles `partials` holds, if fewer than eval_partials_needed (0: that many).
hipError_t launch_eval_neg(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                           const int* WA, const int* WB, const float* A, const float* B,
                           double floorv, double* partials, float* Retval32, double* Retval64,
                           int64_t partials_capacity = 0);

hipError_t launch_finalize(hipStream_t stream, double* partials, int64_t n, float* Retval32,
                           double* Retval64);

int max_slice_parts();
// Capacity the Eval launchers below need in `partials`.
int64_t slice_eval_partials_needed();

// Update passes over a sliced, multi-part model (SliceMap, w2v_device.h).  The shadow buffers
// serve the first kHotWords packed columns of part 0 and are left zeroed.
hipError_t launch_slice_pos(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                            const int* LB, const int* UB, const SliceMap& m, float lrate,
                            float vexp, Shadow shadow);
hipError_t launch_slice_neg(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                            const int* WA, const int* WB, const SliceMap& m, float lrate,
                            float vexp, Shadow shadow);
// The tiled positive pass on a sliced model; *launched is false (and nothing was enqueued) when
// no tile fits in LDS for this nrows / shift.
// The ordered positive kernel on a sliced model, for the launcher of the per-centre kernel.
hipError_t launch_slice_pos_chain(hipStream_t stream, int nrows, int ncols, int shift,
                                  const int* W, const int* LB, const int* UB, const SliceMap& m,
                                  float lrate, float vexp, const Shadow& shadow);
hipError_t launch_slice_pos_tiled(hipStream_t stream, int nrows, int ncols, int shift,
                                  const int* W, const int* LB, const int* UB, const SliceMap& m,
                                  float lrate, float vexp, Shadow shadow, bool* launched);
hipError_t launch_slice_eval_pos(hipStream_t stream, int nrows, int ncols, const int* W,
                                 const int* LB, const int* UB, const SliceMap& m, double floorv,
                                 double* partials, float* Retval32, double* Retval64);
hipError_t launch_slice_eval_neg(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                 const int* WA, const int* WB, const SliceMap& m, double floorv,
                                 double* partials, float* Retval32, double* Retval64);

// The operators for any shape (w2v_any_shape.hip): one wave per work unit, columns walked in
// chunks, untuned.  Taken for nrows beyond max_rows(), nwb beyond max_nwb(), and wide groups whose
// A columns do not fit in LDS (neg_wide_fits).  neg_any_fits: the group's nwa x nwb steps and one
// chunk of A deltas fit in LDS (else the negative operators fail with hipErrorInvalidValue).
bool neg_wide_fits(int nrows, int nwa);
bool neg_any_fits(int nwa, int nwb);
hipError_t launch_pos_any(hipStream_t stream, int nrows, int ncols, const int* W, const int* LB,
                          const int* UB, float* A, float* B, float lrate, float vexp);
hipError_t launch_eval_pos_any(hipStream_t stream, int nrows, int ncols, const int* W,
                               const int* LB, const int* UB, const float* A, const float* B,
                               double floorv, double* partials, float* Retval32,
                               double* Retval64);
hipError_t launch_neg_any(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                          const int* WA, const int* WB, float* A, float* B, float lrate,
                          float vexp);
hipError_t launch_eval_neg_any(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                               const int* WA, const int* WB, const float* A, const float* B,
                               double floorv, double* partials, float* Retval32, double* Retval64,
                               int64_t partials_capacity);

// Largest nrows / nwb the register-resident kernels take; the single-table fp32 operators go to
// the any-shape kernels beyond them, the sliced and bfloat16 operators fail with
// hipErrorInvalidValue.
int max_rows();
int max_nwb();

}  // namespace w2v
