// Negative-sample pass for groups with more B words than a wavefront can hold in registers
// (nwb > 8, up to 64): the reference's GPU launcher runs (nwa, nwb) = (5, 10)
// (jni/src/DNN127.cu:1434,1446) and its CPU path takes any shape (jni/src/BIDMach_CPUMACH.c:212).
//
// Semantics are those of BIDMach_CPUMACH.c:186-264: every dot of a group uses the A columns as
// they were when the group started (A is written after the group's last dot, :248-254) and a B
// column as it was when its own tile of rows started (read with device-scope loads, so that a
// word of an earlier tile is seen as that tile's adds left it).  Walking the B columns in tiles and re-reading A for
// every tile would break the first rule (a later tile would see the deltas of the earlier ones,
// an error of the order of the squared step, which is not small for the large steps that
// vexp > 0 gives rare words).  So the group's A columns are staged once, in LDS, next to an fp32
// accumulator for each of them; the B columns then pass through registers eight (four for long
// columns) at a time, each tile reading its B columns, dotting them with the staged A columns,
// adding its share to the A accumulators and scattering its own B deltas; the A deltas leave
// after the last tile.  Every column is read once and updated once, as in the narrow kernel.
//
// One wavefront per workgroup and group at a time; a lane only ever touches its own slots of the
// staged columns (elements lane, lane + 64, ...), so the column data needs no barrier.  All
// updates are float atomics (no shadow copies, no rare-word path): this shape is rare, and the
// narrow kernel stays the one that is tuned.
#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

namespace {

constexpr size_t kWideMaxLds = 160 * 1024 - 512;

template <int R>
__device__ __forceinline__ void load_col_any(float (&x)[R], const float* col, int lane, int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    x[r] = e < d ? col[e] : 0.0f;
  }
}

// The same with device-scope loads, for the B columns: a B word that occurs in two tiles of one
// group (or in two groups of this workgroup) was updated with a device-scope add, which a plain
// load could still answer from this CU's L1 with the value from before.
template <int R>
__device__ __forceinline__ void load_col_any_fresh(float (&x)[R], const float* col, int lane,
                                                   int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    x[r] = e < d ? __hip_atomic_load(col + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
  }
}

// R here is an upper bound of ceil(d / 64): rounds beyond d hold zeros and are never stored.
template <int R, int MAXB, typename Tables>
__global__ void __launch_bounds__(kWave)
neg_wide_kernel(int d, int ngroups, int idlimit, int nwa, int nwb, int64_t per_wg_all,
                int64_t per_wg_ordered, const int* __restrict__ WA, const int* __restrict__ WB,
                Tables tables, float lrate,
                float vexp, int smode, Shadow shadow_arg) {
  // a launch full of frequent words is done by neg_rows_kernel (launch_is_ordered, w2v_device.h),
  // or, where that has no instance for the shape, by this kernel on a few workgroups
  int64_t per_wg = per_wg_all;
  if (shadow_arg.ordered != 0 && launch_is_ordered(shadow_arg, resolve_hot_mode(shadow_arg))) {
    if (per_wg_ordered == 0) return;
    per_wg = per_wg_ordered;
  }
  extern __shared__ float lds[];
  constexpr int RS = R * kWave;
  float* const a_old = lds;                          // [nwa][RS]
  float* const a_acc = lds + (size_t)nwa * RS;       // [nwa][RS]
  int* const a_id = reinterpret_cast<int*>(lds + (size_t)2 * nwa * RS);   // [nwa], -1 = skipped
  const int lane = threadIdx.x;
  const int64_t g_begin = (int64_t)blockIdx.x * per_wg;
  const int64_t g_end = min(g_begin + per_wg, (int64_t)ngroups);

  for (int64_t unit = g_begin; unit < g_end; ++unit) {
    // stage the group's A columns and clear their accumulators
    __syncthreads();   // the previous group's readers of a_id are done
    for (int jbase = 0; jbase < nwa; jbase += kWave) {
      int wal = -1;
      if (jbase + lane < nwa) wal = WA[unit * nwa + jbase + lane];
      if (wal >= idlimit) wal = -1;
      const ColRef pal = tables.a(wal, d);
      if (jbase + lane < nwa) a_id[jbase + lane] = pal.flags != 0 ? wal : -1;
    }
    __syncthreads();
    for (int j = 0; j < nwa; ++j) {
      const int w = a_id[j];
      float a[R];
      if (w >= 0) {
        load_col_any<R>(a, tables.a(w, d).col, lane, d);
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) a[r] = 0.0f;
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        a_old[(size_t)j * RS + r * kWave + lane] = a[r];
        a_acc[(size_t)j * RS + r * kWave + lane] = 0.0f;
      }
    }

    int wbl = -1;
    if (lane < nwb) wbl = WB[unit * nwb + lane];
    if (wbl >= idlimit) wbl = -1;
    const ColRef pbl = tables.b(wbl, d);
    const float sbl = pbl.flags != 0 ? scale_of(wbl, vexp, smode) : 0.0f;

    for (int kb = 0; kb < nwb; kb += MAXB) {
      float b[MAXB][R];
      float dbb[MAXB][R];
      float* bcol[MAXB];
      int fb[MAXB];
#pragma unroll
      for (int k = 0; k < MAXB; ++k) {
        fb[k] = 0;
        bcol[k] = nullptr;
        if (kb + k < nwb) {
          fb[k] = read_lane(pbl.flags, kb + k);
          if (fb[k] != 0) {
            bcol[k] = tables.b(read_lane(wbl, kb + k), d).col;
            load_col_any_fresh<R>(b[k], bcol[k], lane, d);
          }
        }
        zero_col<R>(dbb[k]);
      }
      for (int j = 0; j < nwa; ++j) {
        const int w = a_id[j];
        if (w < 0) continue;
        const int fa = tables.a(w, d).flags;
        const float as = scale_of(w, vexp, smode);
        float a[R];
#pragma unroll
        for (int r = 0; r < R; ++r) a[r] = a_old[(size_t)j * RS + r * kWave + lane];
        float pre = 0.0f;
#pragma unroll
        for (int k = 0; k < MAXB; ++k) {
          if (fb[k] != 0 && tables.trained(fa, fb[k])) {
            const float s = wave_sum(dot_partial<R>(a, b[k]));
            pre = (lane == k) ? s : pre;
          }
        }
        const float gl = -lrate * sat_sigmoid(pre);
        float daa[R];
        zero_col<R>(daa);
#pragma unroll
        for (int k = 0; k < MAXB; ++k) {
          if (fb[k] != 0 && tables.trained(fa, fb[k])) {
            const float g = read_lane(gl, k);
            const float bs = read_lane(sbl, kb + k);
            axpy<R>(dbb[k], bs * g, a);
            axpy<R>(daa, as * g, b[k]);
          }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) a_acc[(size_t)j * RS + r * kWave + lane] += daa[r];
      }
#pragma unroll
      for (int k = 0; k < MAXB; ++k)
        if (fb[k] != 0 && tables.written(fb[k])) atomic_add_col<R>(bcol[k], dbb[k], lane, d);
    }

    for (int j = 0; j < nwa; ++j) {
      const int w = a_id[j];
      if (w < 0) continue;
      const ColRef ra = tables.a(w, d);
      if (!tables.written(ra.flags)) continue;
      float daa[R];
#pragma unroll
      for (int r = 0; r < R; ++r) daa[r] = a_acc[(size_t)j * RS + r * kWave + lane];
      atomic_add_col<R>(ra.col, daa, lane, d);
    }
  }
}

constexpr int64_t kWideMinGroupsPerWg = 64;
// workgroups (of one wave) that run an ordered launch whose shape the row-by-row kernel has no
// instance for: the group-at-a-time order needs 32 or fewer workers for 1 % of held-out loss
constexpr int64_t kWideOrderedWorkers = 32;

template <int R, typename Tables>
hipError_t launch_wide_r(hipStream_t stream, int d, int ngroups, int idlimit, int nwa, int nwb,
                         const int* WA, const int* WB, const Tables& tables, float lrate,
                         float vexp, Shadow shadow) {
  constexpr int MAXB = R <= 8 ? 8 : 4;
  auto kern = neg_wide_kernel<R, MAXB, Tables>;
  const size_t lds = ((size_t)2 * nwa * R * kWave + nwa) * sizeof(float);
  if (lds > kWideMaxLds) return hipErrorInvalidValue;   // no kernel for this shape
  hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (err != hipSuccess) return err;
  int64_t nwg = 0;
  err = persistent_grid(reinterpret_cast<const void*>(kern), kWave, lds, ngroups,
                        kWideMinGroupsPerWg, &nwg);
  if (err != hipSuccess) return err;
  const int64_t per_wg = ((int64_t)ngroups + nwg - 1) / nwg;
  nwg = ((int64_t)ngroups + per_wg - 1) / per_wg;
  // Only the count of the launch's frequent words is wanted of `shadow` (this kernel uses no
  // shadow copies): the launch is ordered or not, and the row-by-row kernel takes it if it is and
  // has an instance for the shape.
  if constexpr (Tables::kSliced)
    err = prepare_hot_mode_sliced(stream, WB, (int64_t)ngroups * nwb, WA, (int64_t)ngroups * nwa,
                                  tables.m, d, nwg, 1, &shadow);
  else
    err = prepare_hot_mode(stream, WB, (int64_t)ngroups * nwb, WA, (int64_t)ngroups * nwa, nullptr,
                           nullptr, d, nwg, 1, &shadow);
  if (err != hipSuccess) return err;
  const bool rows = shadow.ordered != 0 && neg_rows_available(d, nwa);
  int64_t per_wg_ordered = 0;
  if (shadow.ordered != 0 && !rows) {
    const int64_t wgs = nwg < kWideOrderedWorkers ? nwg : kWideOrderedWorkers;
    per_wg_ordered = ((int64_t)ngroups + wgs - 1) / wgs;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kWave), lds, stream, d, ngroups, idlimit,
                     nwa, nwb, per_wg, per_wg_ordered, WA, WB, tables, lrate, vexp,
                     scale_mode(vexp), shadow);
  err = hipGetLastError();
  if (err != hipSuccess || !rows) return err;
  if constexpr (Tables::kSliced)
    return launch_slice_neg_rows(stream, d, ngroups, nwa, nwb, WA, WB, tables.m, lrate, vexp,
                                 ordered_neg_chains(kWavesPerBlock, kNegRowWorkers), shadow);
  else
    return launch_neg_rows(stream, d, ngroups, idlimit, nwa, nwb, WA, WB, tables.A, tables.B, lrate,
                           vexp, ordered_neg_chains(kWavesPerBlock, kNegRowWorkers), shadow);
}

template <typename Tables>
hipError_t launch_wide(hipStream_t stream, int d, int ngroups, int idlimit, int nwa, int nwb,
                       const int* WA, const int* WB, const Tables& tables, float lrate,
                       float vexp, const Shadow& shadow) {
  const int rounds = (d + kWave - 1) / kWave;
#define CALL(R) \
  return launch_wide_r<R>(stream, d, ngroups, idlimit, nwa, nwb, WA, WB, tables, lrate, vexp, shadow)
  if (rounds <= 2) CALL(2);
  if (rounds <= 5) CALL(5);
  if (rounds <= 8) CALL(8);
  if (rounds <= 12) CALL(12);
  if (rounds <= kMaxRounds) CALL(kMaxRounds);
#undef CALL
  return hipErrorInvalidValue;
}

}  // namespace

bool neg_wide_fits(int nrows, int nwa) {
  const int rounds = (nrows + kWave - 1) / kWave;
  const int R = rounds <= 2 ? 2 : rounds <= 5 ? 5 : rounds <= 8 ? 8 : rounds <= 12 ? 12 : kMaxRounds;
  return rounds <= kMaxRounds && ((size_t)2 * nwa * R * kWave + nwa) * sizeof(float) <= kWideMaxLds;
}

hipError_t launch_neg_wide(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                           const int* WA, const int* WB, float* A, float* B, float lrate,
                           float vexp, const Shadow& shadow) {
  return launch_wide(stream, nrows, ncols, idlimit, nwa, nwb, WA, WB, PlainTables{A, B}, lrate,
                     vexp, shadow);
}

hipError_t launch_slice_neg_wide(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                 const int* WA, const int* WB, const SliceMap& m, float lrate,
                                 float vexp, const Shadow& shadow) {
  return launch_wide(stream, nrows, ncols, 0x7FFFFFFF, nwa, nwb, WA, WB, SlicedTables{m}, lrate,
                     vexp, shadow);
}

}  // namespace w2v
