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
// With a model of several hundred gigabytes in mind the kernels are the plain wave-per-unit
// forms (one wavefront per centre token / per group, columns in registers, one column of line-
// aligned float atomics per written column), persistent over contiguous ranges of work units so
// that the work in flight is bounded the same way as in the single-table passes.
#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

constexpr int kMine = 1;  // the worker's own tail word
constexpr int kHead = 2;  // head word, resident on every worker

struct Placed {
  float* col;  // start of the word's column, null if the word is not resident
  int flags;   // 0 (not resident), kMine or kHead
};

// which: 0 = B table of the part, 1 = A table.
__device__ __forceinline__ Placed place(const SliceMap& m, int w, int which, int d) {
  Placed p{nullptr, 0};
  if (w < 0) return p;
  const bool head = w < m.nhead;
  const bool mine = !head && (w % m.nslices == m.islice);
  if (!head && !mine) return p;
  const int packed = head ? w : (w - m.nhead) / m.nslices + m.nhead;
  const int part = packed / m.maxcols;
  if (part >= m.nparts) return p;
  p.col = m.mats[2 * part + which] + (int64_t)(packed - part * m.maxcols) * d;
  p.flags = head ? kHead : kMine;
  return p;
}

__device__ __forceinline__ float* read_lane_ptr(float* p, int lane) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
  return reinterpret_cast<float*>(((uint64_t)hi << 32) | lo);
}

// Both flags non-zero (both words resident) is tested by the callers.
__device__ __forceinline__ bool pair_trained(int fa, int fb, int dohead) {
  return (((fa | fb) & kMine) != 0) || dohead > 1;
}

__device__ __forceinline__ bool col_written(int f, int dohead) {
  return f == kMine || (f == kHead && dohead > 0);
}

template <int R, int CH, bool TRAIN>
__global__ void __launch_bounds__(kBlock)
slice_pos_kernel(int d, int ncols, int64_t units_per_wg, const int* __restrict__ W,
                 const int* __restrict__ LB, const int* __restrict__ UB, SliceMap m, float lrate,
                 float vexp, int smode, double floorv, double* __restrict__ partials) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t u_begin = (int64_t)blockIdx.x * units_per_wg;
  const int64_t u_end = min(u_begin + units_per_wg, (int64_t)ncols);
  double lsum = 0.0;

  for (int64_t unit = u_begin + wave; unit < u_end; unit += kWavesPerBlock) {
    const int i = (int)unit;
    const int wi = __builtin_amdgcn_readfirstlane(W[i]);
    const Placed pa = place(m, wi, 1, d);
    if (pa.flags == 0) continue;
    const int jlo = max(LB[i], -i);
    const int jhi = min(UB[i], ncols - 1 - i);
    float a[R];
    load_col<R>(a, pa.col, lane, d);
    float daa[R];
    zero_col<R>(daa);
    const float ascale = TRAIN ? scale_of(wi, vexp, smode) : 1.0f;
    bool touched = false;

    for (int base = jlo; base <= jhi; base += kWave) {
      const int j = base + lane;
      int wl = -1;
      if (j <= jhi && j != 0) wl = W[i + j];
      const Placed pb = place(m, wl, 0, d);
      bool ok = pb.flags != 0;
      if (TRAIN) ok = ok && pair_trained(pa.flags, pb.flags, m.dohead);
      const float sl = (TRAIN && ok) ? scale_of(wl, vexp, smode) : 0.0f;
      unsigned long long mask = __ballot(ok);
      const unsigned long long wmask = __ballot(ok && col_written(pb.flags, m.dohead));

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
        float* bcol[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (c < n) {
            bcol[c] = read_lane_ptr(pb.col, src[c]);
            load_col<R>(b[c], bcol[c], lane, d);
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
              if ((wmask >> src[c]) & 1ull) atomic_axpy_col<R>(bcol[c], bs * g, a, lane, d);
            }
          }
          touched = true;
        } else {
          if (lane < n) lsum += log(fmax((double)sg, floorv));
        }
      }
    }
    if (TRAIN && touched && col_written(pa.flags, m.dohead))
      atomic_add_col<R>(pa.col, daa, lane, d);
  }

  if (!TRAIN) block_store_partial(wave_sum_f64(lsum), partials);
}

template <int R, int MAXB, int CHA, bool TRAIN>
__global__ void __launch_bounds__(kBlock)
slice_neg_kernel(int d, int ngroups, int nwa, int nwb, int64_t units_per_wg,
                 const int* __restrict__ WA, const int* __restrict__ WB, SliceMap m, float lrate,
                 float vexp, int smode, double floorv, double* __restrict__ partials) {
  static_assert(MAXB * CHA <= kWave, "one lane per pre-activation of a chunk");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t u_begin = (int64_t)blockIdx.x * units_per_wg;
  const int64_t u_end = min(u_begin + units_per_wg, (int64_t)ngroups);
  double lsum = 0.0;

  for (int64_t unit = u_begin + wave; unit < u_end; unit += kWavesPerBlock) {
    int wbl = -1;
    if (lane < nwb) wbl = WB[unit * nwb + lane];
    const Placed pbl = place(m, wbl, 0, d);
    const float sbl = (TRAIN && pbl.flags != 0) ? scale_of(wbl, vexp, smode) : 0.0f;

    float b[MAXB][R];
    float dbb[MAXB][R];
    float* bcol[MAXB];
    int fb[MAXB];
#pragma unroll
    for (int k = 0; k < MAXB; ++k) {
      fb[k] = 0;
      bcol[k] = nullptr;
      if (k < nwb) {
        fb[k] = read_lane(pbl.flags, k);
        bcol[k] = read_lane_ptr(pbl.col, k);
        if (fb[k] != 0) load_col<R>(b[k], bcol[k], lane, d);
        zero_col<R>(dbb[k]);
      }
    }

    for (int jbase = 0; jbase < nwa; jbase += kWave) {
      int wal = -1;
      if (jbase + lane < nwa) wal = WA[unit * nwa + jbase + lane];
      const Placed pal = place(m, wal, 1, d);
      const float sal = (TRAIN && pal.flags != 0) ? scale_of(wal, vexp, smode) : 0.0f;
      const int jend = min(nwa - jbase, kWave);

      for (int j0 = 0; j0 < jend; j0 += CHA) {
        float a[CHA][R];
        float* acol[CHA];
        int fa[CHA];
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          fa[c] = 0;
          acol[c] = nullptr;
          if (j0 + c < jend) {
            fa[c] = read_lane(pal.flags, j0 + c);
            acol[c] = read_lane_ptr(pal.col, j0 + c);
            if (fa[c] != 0) load_col<R>(a[c], acol[c], lane, d);
          }
        }
        float pre = 0.0f;
        bool live = false;
#pragma unroll
        for (int c = 0; c < CHA; ++c) {
          if (fa[c] != 0) {
#pragma unroll
            for (int k = 0; k < MAXB; ++k) {
              if (fb[k] != 0 && (!TRAIN || pair_trained(fa[c], fb[k], m.dohead))) {
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
                if (fb[k] != 0 && pair_trained(fa[c], fb[k], m.dohead)) {
                  const float g = read_lane(gl, c * MAXB + k);
                  const float bs = read_lane(sbl, k);
                  axpy<R>(dbb[k], bs * g, a[c]);
                  axpy<R>(daa, as * g, b[k]);
                }
              }
              if (col_written(fa[c], m.dohead)) atomic_add_col<R>(acol[c], daa, lane, d);
            }
          }
        } else {
          if (live) lsum += log(fmax(1.0 - (double)sat_sigmoid(pre), floorv));
        }
      }
    }

    if (TRAIN) {
#pragma unroll
      for (int k = 0; k < MAXB; ++k) {
        if (fb[k] != 0 && col_written(fb[k], m.dohead))
          atomic_add_col<R>(bcol[k], dbb[k], lane, d);
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
static hipError_t launch_slice_pos_r(hipStream_t stream, int d, int ncols, const int* W,
                                     const int* LB, const int* UB, const SliceMap& m, float lrate,
                                     float vexp, double floorv, double* partials, int64_t* nparts) {
  auto kern = slice_pos_kernel<R, SlicePosChunk<R>::value, TRAIN>;
  int64_t nwg = 0, per_wg = 0;
  hipError_t err = slice_grid(reinterpret_cast<const void*>(kern), ncols, &nwg, &per_wg);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, ncols, per_wg, W, LB,
                     UB, m, lrate, vexp, scale_mode(vexp), floorv, partials);
  *nparts = nwg;
  return hipGetLastError();
}

template <int R, int MAXB, bool TRAIN>
static hipError_t launch_slice_neg_rb(hipStream_t stream, int d, int ngroups, int nwa, int nwb,
                                      const int* WA, const int* WB, const SliceMap& m, float lrate,
                                      float vexp, double floorv, double* partials,
                                      int64_t* nparts) {
  auto kern = slice_neg_kernel<R, MAXB, SliceNegChunk<R, MAXB>::value, TRAIN>;
  int64_t nwg = 0, per_wg = 0;
  hipError_t err = slice_grid(reinterpret_cast<const void*>(kern), ngroups, &nwg, &per_wg);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, ngroups, nwa, nwb,
                     per_wg, WA, WB, m, lrate, vexp, scale_mode(vexp), floorv, partials);
  *nparts = nwg;
  return hipGetLastError();
}

template <int R, bool TRAIN>
static hipError_t launch_slice_neg_r(hipStream_t stream, int d, int ngroups, int nwa, int nwb,
                                     const int* WA, const int* WB, const SliceMap& m, float lrate,
                                     float vexp, double floorv, double* partials, int64_t* nparts) {
  if (nwb <= 5)
    return launch_slice_neg_rb<R, 5, TRAIN>(stream, d, ngroups, nwa, nwb, WA, WB, m, lrate, vexp,
                                            floorv, partials, nparts);
  if (nwb <= 8)
    return launch_slice_neg_rb<R, 8, TRAIN>(stream, d, ngroups, nwa, nwb, WA, WB, m, lrate, vexp,
                                            floorv, partials, nparts);
  return hipErrorInvalidValue;
}

hipError_t launch_slice_pos(hipStream_t stream, int nrows, int ncols, const int* W, const int* LB,
                            const int* UB, const SliceMap& m, float lrate, float vexp) {
  const int rounds = (nrows + kWave - 1) / kWave;
  int64_t unused = 0;
#define CALL(R)                                                                                 \
  return launch_slice_pos_r<R, true>(stream, nrows, ncols, W, LB, UB, m, lrate, vexp, 0.0, nullptr, \
                                     &unused)
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
}

hipError_t launch_slice_neg(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                            const int* WA, const int* WB, const SliceMap& m, float lrate,
                            float vexp) {
  const int rounds = (nrows + kWave - 1) / kWave;
  int64_t unused = 0;
#define CALL(R)                                                                               \
  return launch_slice_neg_r<R, true>(stream, nrows, ncols, nwa, nwb, WA, WB, m, lrate, vexp, 0.0, \
                                     nullptr, &unused)
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
}

hipError_t launch_slice_eval_pos(hipStream_t stream, int nrows, int ncols, const int* W,
                                 const int* LB, const int* UB, const SliceMap& m, double floorv,
                                 double* partials, float* Retval32, double* Retval64) {
  const int rounds = (nrows + kWave - 1) / kWave;
  hipError_t err = hipSuccess;
  int64_t nparts = 0;
#define CALL(R)                                                                                   \
  err = launch_slice_pos_r<R, false>(stream, nrows, ncols, W, LB, UB, m, 0.0f, 0.0f, floorv,      \
                                     partials, &nparts);                                          \
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
                                     floorv, partials, &nparts);                                  \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, nparts, Retval32, Retval64);
}

}  // namespace w2v
