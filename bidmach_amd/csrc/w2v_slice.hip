// Skip-gram negative-sampling passes over a sliced, multi-part model.
//
// Semantics follow the reference's CPU-only functions word2vecPosSlice / word2vecNegSlice,
// jni/src/BIDMach_CPUMACH.c:80-184 and :267-366, and the forward-only Scala twins
// evalPosCPUslice / evalNegCPUslice, src/main/scala/BIDMach/networks/Word2Vec.scala:1007-1069
// and :1134-1200.  The vocabulary is split over nslices workers: ids below nhead ("head") are
// resident on every worker, an id >= nhead ("tail") on worker id % nslices only.  A worker packs
// its resident words densely (head, then its tail words in id order: packed column
// nhead + (id - nhead) / nslices) and cuts the packed table into parts of maxcols columns, each
// part a separate allocation; part m has its B table at MM[2m] and its A table at MM[2m+1].
//
// Rules of the update (:137-157, :315-349):
//   a pair (a, b) is trained iff both words are resident and at least one of them is the
//   worker's own tail word, or both are head words and doHead > 1;
//   a column is written iff it is the worker's own tail word, or a head word and doHead > 0
//   (so head columns can be trained by one designated worker, or by all of them and averaged).
// Rule of the forward pass: a pair is scored iff both words are resident.
//
// The positive update runs through the tiled kernel of the single-table pass (w2v_pos.hip), which
// takes the model as a policy; the kernels here are the negative update, the forward-only twins,
// and the per-centre positive update used when no tile fits in LDS.  All are wave-per-unit
// (columns in registers, one column of line-aligned float atomics per written column) and
// persistent over contiguous ranges of work units, so the work in flight is bounded the same
// way as in the single-table passes.  The atomics for the first kHotWords packed columns of part 0
// (the most frequent head words) go through their shadow copies.
#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

__device__ __forceinline__ float* read_lane_ptr(float* p, int lane) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
  return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ ColRef read_lane_ref(const ColRef& r, int lane) {
  return ColRef{read_lane_ptr(r.col, lane), read_lane(r.hot, lane), read_lane(r.flags, lane)};
}

template <int R, int CH, bool TRAIN>
__global__ void __launch_bounds__(kBlock)
slice_pos_kernel(int d, int ncols, int64_t units_per_wg, const int* __restrict__ W,
                 const int* __restrict__ LB, const int* __restrict__ UB, SlicedTables tables,
                 float lrate, float vexp, int smode, double floorv, double* __restrict__ partials,
                 Shadow shadow_arg) {
  const Shadow shadow = TRAIN ? resolve_hot_mode(shadow_arg) : shadow_arg;
  if (TRAIN && launch_is_ordered(shadow_arg, shadow)) return;   // pos_chain_kernel does this launch
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slot = blockIdx.x;
  const int64_t u_begin = (int64_t)blockIdx.x * units_per_wg;
  const int64_t u_end = min(u_begin + units_per_wg, (int64_t)ncols);
  double lsum = 0.0;

  for (int64_t unit = u_begin + wave; unit < u_end; unit += kWavesPerBlock) {
    const int i = (int)unit;
    const int wi = __builtin_amdgcn_readfirstlane(W[i]);
    const ColRef pa = tables.a(wi, d);
    if (pa.flags == 0) continue;
    const int jlo = max(LB[i], -i);
    const int jhi = min(UB[i], ncols - 1 - i);
    float a[R];
    load_col_ref<R>(a, pa, shadow, 1, lane, d);
    float daa[R];
    zero_col<R>(daa);
    const float ascale = TRAIN ? scale_of(wi, vexp, smode) : 1.0f;
    bool touched = false;

    for (int base = jlo; base <= jhi; base += kWave) {
      const int j = base + lane;
      int wl = -1;
      if (j <= jhi && j != 0) wl = W[i + j];
      const ColRef pb = tables.b(wl, d);
      bool ok = pb.flags != 0;
      if (TRAIN) ok = ok && tables.trained(pa.flags, pb.flags);
      const float sl = (TRAIN && ok) ? scale_of(wl, vexp, smode) : 0.0f;
      unsigned long long mask = __ballot(ok);
      const unsigned long long wmask = __ballot(ok && tables.written(pb.flags));

      while (mask != 0ull) {
        int src[CH];
        int n = 0;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (mask != 0ull) {
            src[c] = __builtin_ctzll(mask);
            mask &= mask - 1ull;
            n = c + 1;
          } else {
            src[c] = -1;
          }
        }
        float b[CH][R];
        ColRef rb[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (c < n) {
            rb[c] = read_lane_ref(pb, src[c]);
            load_col_ref<R>(b[c], rb[c], shadow, 0, lane, d);
          }
        }
        float pre = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (c < n) {
            const float s = wave_sum(dot_partial<R>(a, b[c]));
            pre = (lane == c) ? s : pre;
          }
        }
        const float sg = sat_sigmoid(pre);
        if (TRAIN) {
          const float gl = lrate * (1.0f - sg);
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (c < n) {
              const float g = read_lane(gl, c);
              const float bs = read_lane(sl, src[c]);
              axpy<R>(daa, ascale * g, b[c]);
              if ((wmask >> src[c]) & 1ull)
                scatter_axpy_ref<R>(rb[c], shadow, 0, slot, bs * g, a, lane, d);
            }
          }
          touched = true;
        } else {
          if (lane < n) lsum += log(fmax((double)sg, floorv));
        }
      }
    }
    if (TRAIN && touched && tables.written(pa.flags))
      scatter_add_ref<R>(pa, shadow, 1, slot, daa, lane, d);
  }

  if (!TRAIN) block_store_partial(wave_sum_f64(lsum), partials);
}

template <int R, int MAXB, int CHA, bool TRAIN>
__global__ void __launch_bounds__(kBlock, 3)
slice_neg_kernel(int d, int ngroups, int nwa, int nwb, int64_t units_per_wg_all,
                 int64_t units_per_wg_ordered, const int* __restrict__ WA, const int* __restrict__ WB, SlicedTables tables,
                 float lrate, float vexp, int smode, double floorv, double* __restrict__ partials,
                 Shadow shadow_arg) {
  static_assert(MAXB * CHA <= kWave, "one lane per pre-activation of a chunk");
  const Shadow shadow = TRAIN ? resolve_hot_mode(shadow_arg) : shadow_arg;
  int64_t units_per_wg = units_per_wg_all;
  if (TRAIN && launch_is_ordered(shadow_arg, shadow)) {
    if (units_per_wg_ordered == 0) return;    // neg_rows_kernel does this launch
    units_per_wg = units_per_wg_ordered;      // no ordered instance for this shape: few workers
  }
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slot = blockIdx.x;
  const int64_t u_begin = (int64_t)blockIdx.x * units_per_wg;
  const int64_t u_end = min(u_begin + units_per_wg, (int64_t)ngroups);
  double lsum = 0.0;

  for (int64_t unit = u_begin + wave; unit < u_end; unit += kWavesPerBlock) {
    int wbl = -1;
    if (lane < nwb) wbl = WB[unit * nwb + lane];
    const ColRef pbl = tables.b(wbl, d);
    const float sbl = (TRAIN && pbl.flags != 0) ? scale_of(wbl, vexp, smode) : 0.0f;
    // words updated without atomics: rare in this launch, written, and only once in the group
    uint64_t rare_b = 0;
    if (TRAIN && shadow.rare_max > 0) {
      bool lone = true;
      for (int k = 0; k < nwb; ++k)
        if (k != lane && read_lane(wbl, k) == wbl) lone = false;
      rare_b = __ballot(lone && pbl.hot < 0 && tables.written(pbl.flags) && is_rare(shadow, wbl));
    }
    // tickets for the writes to hot B columns at the end of the group, taken now
    const unsigned tkb =
        (TRAIN && tables.written(pbl.flags)) ? hot_ticket(shadow, 0, slot, pbl.hot) : 0u;

    // MAXB columns of B at a time: several trips only in the forward-only instance (training
    // groups with nwb > MAXB go to the kernel of w2v_neg_wide.hip, which keeps the reference's
    // rule that every dot of a group sees the A columns as they were when the group started)
    for (int kb = 0; kb < nwb; kb += MAXB) {
    float b[MAXB][R];
    float dbb[MAXB][R];
    ColRef rb[MAXB];
    int fb[MAXB];
#pragma unroll
    for (int k = 0; k < MAXB; ++k) {
      fb[k] = 0;
      rb[k] = ColRef{nullptr, -1, 0};
      if (kb + k < nwb) {
        rb[k] = read_lane_ref(pbl, kb + k);
        fb[k] = rb[k].flags;
        if (fb[k] != 0) {
          if ((rare_b >> (kb + k)) & 1)
            load_col_fresh<R>(b[k], rb[k].col, lane, d);
          else
            load_col_ref<R>(b[k], rb[k], shadow, 0, lane, d);
        }
        zero_col<R>(dbb[k]);
      }
    }

    for (int jbase = 0; jbase < nwa; jbase += kWave) {
      int wal = -1;
      if (jbase + lane < nwa) wal = WA[unit * nwa + jbase + lane];
      const ColRef pal = tables.a(wal, d);
      const float sal = (TRAIN && pal.flags != 0) ? scale_of(wal, vexp, smode) : 0.0f;
      const unsigned tka =
          (TRAIN && tables.written(pal.flags)) ? hot_ticket(shadow, 1, slot, pal.hot) : 0u;
      const int jend = min(nwa - jbase, kWave);
      uint64_t rare_a = 0;
      if (TRAIN && shadow.rare_max > 0) {
        bool lone = true;
        for (int j = 0; j < jend; ++j)
          if (j != lane && read_lane(wal, j) == wal) lone = false;
        rare_a = __ballot(lone && nwb <= MAXB && pal.hot < 0 && tables.written(pal.flags) &&
                          is_rare_a(shadow, wal));
      }

      for (int j0 = 0; j0 < jend; j0 += CHA) {
        float a[CHA][R];
        ColRef ra[CHA];
        int fa[CHA];
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          fa[c] = 0;
          ra[c] = ColRef{nullptr, -1, 0};
          if (j0 + c < jend) {
            ra[c] = read_lane_ref(pal, j0 + c);
            fa[c] = ra[c].flags;
            if (fa[c] != 0) {
              if ((rare_a >> (j0 + c)) & 1)
                load_col_fresh<R>(a[c], ra[c].col, lane, d);
              else
                load_col_ref<R>(a[c], ra[c], shadow, 1, lane, d);
            }
          }
        }
        float pre = 0.0f;
        bool live = false;
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          if (fa[c] != 0) {
#pragma unroll
            for (int k = 0; k < MAXB; ++k) {
              if (fb[k] != 0 && (!TRAIN || tables.trained(fa[c], fb[k]))) {
                const float s = wave_sum(dot_partial<R>(a[c], b[k]));
                const bool here = lane == c * MAXB + k;
                pre = here ? s : pre;
                live = here ? true : live;
              }
            }
          }
        }
        if (TRAIN) {
          const float gl = -lrate * sat_sigmoid(pre);
#pragma unroll
          for (int c = 0; c < CHA; ++c) {
            if (fa[c] != 0) {
              const float as = read_lane(sal, j0 + c);
              float daa[R];
              zero_col<R>(daa);
#pragma unroll
              for (int k = 0; k < MAXB; ++k) {
                if (fb[k] != 0 && tables.trained(fa[c], fb[k])) {
                  const float g = read_lane(gl, c * MAXB + k);
                  const float bs = read_lane(sbl, kb + k);
                  axpy<R>(dbb[k], bs * g, a[c]);
                  axpy<R>(daa, as * g, b[k]);
                }
              }
              if ((rare_a >> (j0 + c)) & 1)
                store_sum_col<R>(ra[c].col, a[c], daa, lane, d);
              else if (tables.written(fa[c]))
                scatter_add_ref<R>(ra[c], shadow, 1, slot, daa, lane, d, read_lane(tka, j0 + c));
            }
          }
        } else {
          if (live) lsum += log(fmax(1.0 - (double)sat_sigmoid(pre), floorv));
        }
      }
    }

    if (TRAIN) {
      // a rare B column is read again just before its plain store (see neg_train_kernel)
#pragma unroll
      for (int k = 0; k < MAXB; ++k) {
        if (kb + k < nwb && ((rare_b >> (kb + k)) & 1))
          load_col_fresh<R>(b[k], rb[k].col, lane, d);
      }
#pragma unroll
      for (int k = 0; k < MAXB; ++k) {
        if (kb + k < nwb && ((rare_b >> (kb + k)) & 1))
          store_sum_col<R>(rb[k].col, b[k], dbb[k], lane, d);
        else if (fb[k] != 0 && tables.written(fb[k]))
          scatter_add_ref<R>(rb[k], shadow, 0, slot, dbb[k], lane, d, read_lane(tkb, kb + k));
      }
    }
    }
  }

  if (!TRAIN) block_store_partial(wave_sum_f64(lsum), partials);
}

constexpr int64_t kSliceMinUnitsPerWg = 256;
constexpr int64_t kSliceMaxGrid = 8192;

int max_slice_parts() { return kMaxSliceParts; }
int64_t slice_eval_partials_needed() { return kSliceMaxGrid; }

// Context columns per chunk of the positive kernel / A columns per chunk of the negative one,
// sized for about a hundred registers of column data per lane.
template <int R>
struct SlicePosChunk {
  static constexpr int value = R <= 4 ? 12 : R <= 6 ? 10 : R <= 8 ? 8 : R <= 12 ? 5 : 3;
};
template <int R, int MAXB>
struct SliceNegChunk {
  static constexpr int budget = (100 - 2 * MAXB * R) / R;
  static constexpr int capped = budget > 5 ? 5 : budget;
  static constexpr int value = capped < 1 ? 1 : capped;
};

static hipError_t slice_grid(const void* kernel, int64_t units, int64_t* nwg, int64_t* per_wg) {
  hipError_t err = persistent_grid(kernel, kBlock, 0, units, kSliceMinUnitsPerWg, nwg);
  if (err != hipSuccess) return err;
  if (*nwg > kSliceMaxGrid) *nwg = kSliceMaxGrid;
  *per_wg = (units + *nwg - 1) / *nwg;
  *nwg = (units + *per_wg - 1) / *per_wg;
  return hipSuccess;
}

template <int R, bool TRAIN>
static hipError_t launch_slice_pos_r(hipStream_t stream, int d, int ncols, int shift, const int* W,
                                     const int* LB, const int* UB, const SliceMap& m, float lrate,
                                     float vexp, double floorv, double* partials, int64_t* nparts,
                                     Shadow shadow) {
  auto kern = slice_pos_kernel<R, SlicePosChunk<R>::value, TRAIN>;
  int64_t nwg = 0, per_wg = 0;
  hipError_t err = slice_grid(reinterpret_cast<const void*>(kern), ncols, &nwg, &per_wg);
  if (err != hipSuccess) return err;
  if (TRAIN) {
    err = prepare_hot_mode_sliced(stream, W, ncols, nullptr, 0, m, d, nwg, kWavesPerBlock, &shadow);
    if (err != hipSuccess) return err;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, ncols, per_wg, W, LB,
                     UB, SlicedTables{m}, lrate, vexp, scale_mode(vexp), floorv, partials, shadow);
  *nparts = nwg;
  err = hipGetLastError();
  if (TRAIN && err == hipSuccess && shadow.ordered != 0)
    err = launch_slice_pos_chain(stream, d, ncols, shift, W, LB, UB, m, lrate, vexp, shadow);
  return err;
}

template <int R, int MAXB, bool TRAIN>
static hipError_t launch_slice_neg_rb(hipStream_t stream, int d, int ngroups, int nwa, int nwb,
                                      const int* WA, const int* WB, const SliceMap& m, float lrate,
                                      float vexp, double floorv, double* partials,
                                      int64_t* nparts, Shadow shadow) {
  auto kern = slice_neg_kernel<R, MAXB, SliceNegChunk<R, MAXB>::value, TRAIN>;
  int64_t nwg = 0, per_wg = 0;
  hipError_t err = slice_grid(reinterpret_cast<const void*>(kern), ngroups, &nwg, &per_wg);
  if (err != hipSuccess) return err;
  if (TRAIN) {
    err = prepare_hot_mode_sliced(stream, WB, (int64_t)ngroups * nwb, WA, (int64_t)ngroups * nwa, m,
                                  d, nwg, kWavesPerBlock, &shadow);
    if (err != hipSuccess) return err;
    err = prepare_rare_words(stream, WA, (int64_t)ngroups * nwa, WB, (int64_t)ngroups * nwb,
                             0x7fffffff, ngroups, nwg * kWavesPerBlock, &shadow);
    if (err != hipSuccess) return err;
  }
  // ordered launches go to the row-by-row kernel where it has an instance for the shape, else
  // this kernel runs them on a few workgroups (8 x 4 waves, as the single-table operator does)
  const bool rows = TRAIN && shadow.ordered != 0 && neg_rows_available(d, nwa);
  int64_t per_wg_ordered = 0;
  if (TRAIN && shadow.ordered != 0 && !rows) {
    const int64_t wgs = nwg < 8 ? nwg : 8;
    per_wg_ordered = ((int64_t)ngroups + wgs - 1) / wgs;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, ngroups, nwa, nwb,
                     per_wg, per_wg_ordered, WA, WB, SlicedTables{m}, lrate, vexp, scale_mode(vexp),
                     floorv, partials, shadow);
  *nparts = nwg;
  err = hipGetLastError();
  if (err == hipSuccess && rows)
    err = launch_slice_neg_rows(stream, d, ngroups, nwa, nwb, WA, WB, m, lrate, vexp,
                                ordered_neg_chains(kWavesPerBlock, kNegRowWorkers), shadow);
  return err;
}

template <int R, bool TRAIN>
static hipError_t launch_slice_neg_r(hipStream_t stream, int d, int ngroups, int nwa, int nwb,
                                     const int* WA, const int* WB, const SliceMap& m, float lrate,
                                     float vexp, double floorv, double* partials, int64_t* nparts,
                                     Shadow shadow) {
  if (nwb <= 5)
    return launch_slice_neg_rb<R, 5, TRAIN>(stream, d, ngroups, nwa, nwb, WA, WB, m, lrate, vexp,
                                            floorv, partials, nparts, shadow);
  if (nwb <= max_nwb())
    return launch_slice_neg_rb<R, 8, TRAIN>(stream, d, ngroups, nwa, nwb, WA, WB, m, lrate, vexp,
                                            floorv, partials, nparts, shadow);
  return hipErrorInvalidValue;
}

hipError_t launch_slice_pos(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                            const int* LB, const int* UB, const SliceMap& m, float lrate,
                            float vexp, Shadow shadow) {
  bool launched = false;
  hipError_t err = launch_slice_pos_tiled(stream, nrows, ncols, shift, W, LB, UB, m, lrate, vexp,
                                          shadow, &launched);
  if (err != hipSuccess || launched) return err;
  const int rounds = (nrows + kWave - 1) / kWave;
  int64_t unused = 0;
#define CALL(R)                                                                               \
  err = launch_slice_pos_r<R, true>(stream, nrows, ncols, shift, W, LB, UB, m, lrate, vexp, 0.0,   \
                                    nullptr, &unused, shadow);                                \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_fold(stream, m.mats[1], m.mats[0], shadow, nrows);
}

hipError_t launch_slice_neg(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                            const int* WA, const int* WB, const SliceMap& m, float lrate,
                            float vexp, Shadow shadow) {
  if (nwb > 8)
    return launch_slice_neg_wide(stream, nrows, ncols, nwa, nwb, WA, WB, m, lrate, vexp, shadow);
  const int rounds = (nrows + kWave - 1) / kWave;
  int64_t unused = 0;
  hipError_t err = hipSuccess;
#define CALL(R)                                                                                \
  err = launch_slice_neg_r<R, true>(stream, nrows, ncols, nwa, nwb, WA, WB, m, lrate, vexp, 0.0, \
                                    nullptr, &unused, shadow);                                 \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_fold(stream, m.mats[1], m.mats[0], shadow, nrows);
}

hipError_t launch_slice_eval_pos(hipStream_t stream, int nrows, int ncols, const int* W,
                                 const int* LB, const int* UB, const SliceMap& m, double floorv,
                                 double* partials, float* Retval32, double* Retval64) {
  const int rounds = (nrows + kWave - 1) / kWave;
  hipError_t err = hipSuccess;
  int64_t nparts = 0;
#define CALL(R)                                                                                   \
  err = launch_slice_pos_r<R, false>(stream, nrows, ncols, 0, W, LB, UB, m, 0.0f, 0.0f, floorv,   \
                                     partials, &nparts, no_shadow());                             \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, nparts, Retval32, Retval64);
}

hipError_t launch_slice_eval_neg(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                 const int* WA, const int* WB, const SliceMap& m, double floorv,
                                 double* partials, float* Retval32, double* Retval64) {
  const int rounds = (nrows + kWave - 1) / kWave;
  hipError_t err = hipSuccess;
  int64_t nparts = 0;
#define CALL(R)                                                                                   \
  err = launch_slice_neg_r<R, false>(stream, nrows, ncols, nwa, nwb, WA, WB, m, 0.0f, 0.0f,       \
                                     floorv, partials, &nparts, no_shadow());                        \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, nparts, Retval32, Retval64);
}

}  // namespace w2v
