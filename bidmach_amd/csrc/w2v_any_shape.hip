// The four operators for shapes the tuned kernels have no instance for: columns longer than a
// wave holds in registers (nrows > 1280), groups with more than 64 B words, and wide groups whose
// A columns do not fit in LDS.  The reference's CPU path takes any nrows, nwa and nwb
// (jni/src/BIDMach_CPUMACH.c:37,206,212); its GPU launcher stops at nrows 1280 and a handful of
// (nwa, nwb) pairs (jni/src/DNN127.cu:1393-1412,1434).
//
// One wavefront per work unit (a centre token, a group), columns walked in chunks of 256 elements
// (four registers per lane), nothing tuned: a unit is done in two passes.  Pass 1 forms every dot
// product of the unit from the columns as they are (each dot walks its two columns chunk by
// chunk) and turns it into the pair's step g (or its log-likelihood term); pass 2 walks the
// chunks once more and, for each, accumulates the deltas of every column of the unit and adds
// them with float atomics.  All dots of a unit therefore see the columns as they were when the
// unit started, which on minibatches without repeated words is the reference's result
// (BIDMach_CPUMACH.c:57-67, :239-254).  The per-pair steps wait in LDS between the passes.
#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

namespace {

constexpr int kAnyRegs = 4;                    // registers per lane per chunk
constexpr int kAnyChunk = kAnyRegs * kWave;    // elements per chunk

// Sum over the chunks of x . y for two columns of d floats, the same value in every lane.
__device__ __forceinline__ float dot_any(const float* __restrict__ x, const float* __restrict__ y,
                                         int d, int lane) {
  float part = 0.0f;
  for (int c0 = 0; c0 < d; c0 += kAnyChunk) {
#pragma unroll
    for (int r = 0; r < kAnyRegs; ++r) {
      const int e = c0 + r * kWave + lane;
      if (e < d) part = fmaf(x[e], y[e], part);
    }
  }
  return wave_sum(part);
}

// Positive pass.  The window is walked in slabs of 64 offsets (lane l looks at offset base + l);
// the steps of the window's pairs wait in LDS between the passes, so that the centre's column is
// added to once, after the whole window, as the reference does (BIDMach_CPUMACH.c:65-67).  (A
// window of more than kAnyMaxWin offsets is done in stretches of that many, each with an add of
// its own.)
constexpr int kAnyMaxWin = 2048;

template <bool TRAIN>
__global__ void __launch_bounds__(kBlock)
pos_any_kernel(int d, int ncols, const int* __restrict__ W, const int* __restrict__ LB,
               const int* __restrict__ UB, float* A, float* B, float lrate, float vexp, int smode,
               double floorv, double* __restrict__ partials) {
  __shared__ float s_step[TRAIN ? kWavesPerBlock : 1][TRAIN ? kAnyMaxWin : 1];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  double lsum = 0.0;
  for (int64_t unit = (int64_t)blockIdx.x * kWavesPerBlock + wave; unit < ncols;
       unit += (int64_t)gridDim.x * kWavesPerBlock) {
    const int i = (int)unit;
    const int wi = W[i];
    if (wi < 0) continue;
    float* const acol = A + (int64_t)wi * d;
    const float ascale = TRAIN ? scale_of(wi, vexp, smode) : 1.0f;
    const int jlo = max(LB[i], -i), jhi = min(UB[i], ncols - 1 - i);
    for (int lo = jlo; lo <= jhi; lo += kAnyMaxWin) {
      const int hi = min(jhi, lo + kAnyMaxWin - 1);
      // pass 1: the step of every pair of the stretch
      bool any = false;
      for (int base = lo; base <= hi; base += kWave) {
        const int j = base + lane;
        int wl = -1;
        if (j <= hi && j != 0) wl = W[i + j];
        const unsigned long long valid = __ballot(wl >= 0);
        float pre = 0.0f;
        for (unsigned long long m = valid; m != 0ull; m &= m - 1ull) {
          const int l = __builtin_ctzll(m);
          const float s = dot_any(acol, B + (int64_t)read_lane(wl, l) * d, d, lane);
          pre = (lane == l) ? s : pre;
        }
        const float sg = sat_sigmoid(pre);
        if (!TRAIN) {
          if (wl >= 0) lsum += log(fmax((double)sg, floorv));
        } else if (j <= hi) {
          s_step[wave][j - lo] = wl >= 0 ? lrate * (1.0f - sg) : 0.0f;
        }
        any = any || valid != 0ull;
      }
      if (!TRAIN || !any) continue;
      // pass 2: chunk by chunk, the B columns' deltas at once, the centre's after the stretch
      for (int c0 = 0; c0 < d; c0 += kAnyChunk) {
        float a[kAnyRegs], daa[kAnyRegs];
#pragma unroll
        for (int r = 0; r < kAnyRegs; ++r) {
          const int e = c0 + r * kWave + lane;
          a[r] = e < d ? acol[e] : 0.0f;
          daa[r] = 0.0f;
        }
        for (int base = lo; base <= hi; base += kWave) {
          const int j = base + lane;
          int wl = -1;
          if (j <= hi && j != 0) wl = W[i + j];
          const float gl = j <= hi ? s_step[wave][j - lo] : 0.0f;
          const float sl = wl >= 0 ? scale_of(wl, vexp, smode) : 0.0f;
          for (unsigned long long m = __ballot(wl >= 0); m != 0ull; m &= m - 1ull) {
            const int l = __builtin_ctzll(m);
            float* const bcol = B + (int64_t)read_lane(wl, l) * d;
            const float g = read_lane(gl, l);
            const float gb = read_lane(sl, l) * g, ga = ascale * g;
#pragma unroll
            for (int r = 0; r < kAnyRegs; ++r) {
              const int e = c0 + r * kWave + lane;
              if (e < d) {
                daa[r] = fmaf(ga, bcol[e], daa[r]);
                unsafeAtomicAdd(bcol + e, gb * a[r]);
              }
            }
          }
        }
#pragma unroll
        for (int r = 0; r < kAnyRegs; ++r) {
          const int e = c0 + r * kWave + lane;
          if (e < d) unsafeAtomicAdd(acol + e, daa[r]);
        }
      }
    }
  }
  if (!TRAIN) block_store_partial(wave_sum_f64(lsum), partials);
}

// Negative pass: one wave per workgroup; the nwa x nwb steps of the group wait in LDS, and so do,
// chunk by chunk, the A columns' deltas: within a chunk the A deltas are formed first (from the B
// chunk as it is), then the B deltas are formed from the A chunk as it is and added, and only
// then are the A deltas added, so both sides are computed from unchanged columns.
template <bool TRAIN>
__global__ void __launch_bounds__(kWave)
neg_any_kernel(int d, int ngroups, int idlimit, int nwa, int nwb, const int* __restrict__ WA,
               const int* __restrict__ WB, float* A, float* B, float lrate, float vexp, int smode,
               double floorv, double* __restrict__ partials) {
  extern __shared__ float s_g[];   // [nwa][nwb] steps, then [nwa][kAnyChunk] parked A deltas
  const int lane = threadIdx.x;
  double lsum = 0.0;
  auto word = [&](const int* ids, int64_t at) {
    const int w = ids[at];
    return (w >= 0 && w < idlimit) ? w : -1;
  };
  for (int64_t unit = blockIdx.x; unit < ngroups; unit += gridDim.x) {
    const int* const wa = WA + unit * nwa;
    const int* const wb = WB + unit * nwb;
    __syncthreads();   // the last group's readers of s_g are done
    for (int j = 0; j < nwa; ++j) {
      const int w = word(wa, j);
      for (int k = 0; k < nwb; ++k) {
        const int x = word(wb, k);
        float g = 0.0f;
        if (w >= 0 && x >= 0) {
          const float sg = sat_sigmoid(dot_any(A + (int64_t)w * d, B + (int64_t)x * d, d, lane));
          if (TRAIN) {
            g = -lrate * sg;
          } else if (lane == 0) {
            lsum += log(fmax(1.0 - (double)sg, floorv));
          }
        }
        if (TRAIN && lane == 0) s_g[j * nwb + k] = g;
      }
    }
    if (!TRAIN) continue;
    __syncthreads();
    for (int c0 = 0; c0 < d; c0 += kAnyChunk) {
      // the A columns' deltas of this chunk, then the B columns'
      for (int j = 0; j < nwa; ++j) {
        const int w = word(wa, j);
        if (w < 0) continue;
        const float as = scale_of(w, vexp, smode);
        float daa[kAnyRegs] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int k = 0; k < nwb; ++k) {
          const int x = word(wb, k);
          if (x < 0) continue;
          const float ga = as * s_g[j * nwb + k];
          const float* const bcol = B + (int64_t)x * d;
#pragma unroll
          for (int r = 0; r < kAnyRegs; ++r) {
            const int e = c0 + r * kWave + lane;
            if (e < d) daa[r] = fmaf(ga, bcol[e], daa[r]);
          }
        }
#pragma unroll
        for (int r = 0; r < kAnyRegs; ++r) s_g[nwa * nwb + (j * kAnyRegs + r) * kWave + lane] = daa[r];
      }
      for (int k = 0; k < nwb; ++k) {
        const int x = word(wb, k);
        if (x < 0) continue;
        const float bs = scale_of(x, vexp, smode);
        float dbb[kAnyRegs] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int j = 0; j < nwa; ++j) {
          const int w = word(wa, j);
          if (w < 0) continue;
          const float gb = bs * s_g[j * nwb + k];
          const float* const acol = A + (int64_t)w * d;
#pragma unroll
          for (int r = 0; r < kAnyRegs; ++r) {
            const int e = c0 + r * kWave + lane;
            if (e < d) dbb[r] = fmaf(gb, acol[e], dbb[r]);
          }
        }
        float* const bcol = B + (int64_t)x * d;
#pragma unroll
        for (int r = 0; r < kAnyRegs; ++r) {
          const int e = c0 + r * kWave + lane;
          if (e < d) unsafeAtomicAdd(bcol + e, dbb[r]);
        }
      }
      for (int j = 0; j < nwa; ++j) {
        const int w = word(wa, j);
        if (w < 0) continue;
        float* const acol = A + (int64_t)w * d;
#pragma unroll
        for (int r = 0; r < kAnyRegs; ++r) {
          const int e = c0 + r * kWave + lane;
          if (e < d) unsafeAtomicAdd(acol + e, s_g[nwa * nwb + (j * kAnyRegs + r) * kWave + lane]);
        }
      }
    }
  }
  if (!TRAIN) {
    const double total = __shfl(lsum, 0, kWave);
    if (lane == 0) partials[blockIdx.x] = total;
  }
}

constexpr size_t kAnyMaxLds = 64 * 1024;

size_t neg_any_lds(int nwa, int nwb) {
  return ((size_t)nwa * nwb + (size_t)nwa * kAnyChunk) * sizeof(float);
}

}  // namespace

// Waves a launch of the any-shape kernels keeps in flight at most (they make no distinction
// between launches with and without frequent words: a bounded number, like a large host).
constexpr int64_t kAnyMaxWaves = 1024;

bool neg_any_fits(int nwa, int nwb) { return neg_any_lds(nwa, nwb) <= kAnyMaxLds; }

hipError_t launch_pos_any(hipStream_t stream, int nrows, int ncols, const int* W, const int* LB,
                          const int* UB, float* A, float* B, float lrate, float vexp) {
  int64_t blocks = ((int64_t)ncols + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > kAnyMaxWaves / kWavesPerBlock) blocks = kAnyMaxWaves / kWavesPerBlock;
  hipLaunchKernelGGL(pos_any_kernel<true>, dim3((unsigned)blocks), dim3(kBlock), 0, stream, nrows,
                     ncols, W, LB, UB, A, B, lrate, vexp, scale_mode(vexp), 0.0, nullptr);
  return hipGetLastError();
}

hipError_t launch_eval_pos_any(hipStream_t stream, int nrows, int ncols, const int* W,
                               const int* LB, const int* UB, const float* A, const float* B,
                               double floorv, double* partials, float* Retval32,
                               double* Retval64) {
  // one partial per block: within what eval_partials_needed(ncols) promises the caller's buffer
  int64_t blocks = ((int64_t)ncols + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > kAnyMaxWaves / kWavesPerBlock) blocks = kAnyMaxWaves / kWavesPerBlock;
  hipLaunchKernelGGL(pos_any_kernel<false>, dim3((unsigned)blocks), dim3(kBlock), 0, stream, nrows,
                     ncols, W, LB, UB, const_cast<float*>(A), const_cast<float*>(B), 0.0f, 0.0f, 0,
                     floorv, partials);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, blocks, Retval32, Retval64);
}

hipError_t launch_neg_any(hipStream_t stream, int nrows, int ncols, int idlimit, int nwa, int nwb,
                          const int* WA, const int* WB, float* A, float* B, float lrate,
                          float vexp) {
  const size_t lds = neg_any_lds(nwa, nwb);
  if (lds > kAnyMaxLds) return hipErrorInvalidValue;
  auto kern = neg_any_kernel<true>;
  if (lds > 48 * 1024) {
    const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return err;
  }
  const int64_t blocks = ncols < kAnyMaxWaves ? ncols : kAnyMaxWaves;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kWave), lds, stream, nrows, ncols, idlimit,
                     nwa, nwb, WA, WB, A, B, lrate, vexp, scale_mode(vexp), 0.0, nullptr);
  return hipGetLastError();
}

hipError_t launch_eval_neg_any(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                               const int* WA, const int* WB, const float* A, const float* B,
                               double floorv, double* partials, float* Retval32, double* Retval64,
                               int64_t partials_capacity) {
  int64_t blocks = ncols < kAnyMaxWaves ? ncols : kAnyMaxWaves;
  if (partials_capacity > 0 && blocks > partials_capacity) blocks = partials_capacity;
  hipLaunchKernelGGL(neg_any_kernel<false>, dim3((unsigned)blocks), dim3(kWave), sizeof(float),
                     stream, nrows, ncols, 0x7fffffff, nwa, nwb, WA, WB, const_cast<float*>(A),
                     const_cast<float*>(B), 0.0f, 0.0f, 0, floorv, partials);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, blocks, Retval32, Retval64);
}

}  // namespace w2v
