// Positive (centre, context) pass of skip-gram negative sampling, and its forward-only twin.
//
// Semantics follow the reference CPU path, jni/src/BIDMach_CPUMACH.c:10-78 (word2vecPos) and
// :368-427 (word2vecEvalPos): for each centre token i with W[i] >= 0 and each offset
// j in [LB[i], UB[i]], j != 0, 0 <= i+j < ncols, W[i+j] >= 0:
//   s = A[:,W[i]] . B[:,W[i+j]];  g = lrate * (1 - sigmoid(s))
//   B[:,W[i+j]] += bscale * g * A[:,W[i]]      (scattered at once)
//   A[:,W[i]]   += ascale * g * B[:,W[i+j]]    (accumulated over the window, scattered once)
//
// One wavefront owns one centre token.  Its A column stays in registers for the whole window;
// context columns are gathered CH at a time (all loads of a chunk are issued before the first
// dot product, so a wave keeps CH columns in flight), dot products are reduced with DPP row
// rotations, the CH pre-activations are parked in lanes 0..CH-1 so that the sigmoid (a double
// exp) is evaluated once per chunk instead of once per pair, and the updates leave as float
// atomics.  A chunk reads its context columns before it updates any of them, so a word that
// occurs twice inside one chunk sees the pre-chunk value (Hogwild staleness, as between waves).
#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

template <int R, int CH, bool TRAIN>
__global__ void __launch_bounds__(kBlock)
pos_kernel(int d, int ncols, int64_t per_xcd, const int* __restrict__ W,
           const int* __restrict__ LB, const int* __restrict__ UB, float* A, float* B, float lrate,
           float vexp, int smode, double floorv, double* __restrict__ partials) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t unit = xcd_contiguous_block(per_xcd) * kWavesPerBlock + wave;
  double lsum = 0.0;

  if (unit < ncols) {
    const int i = (int)unit;
    const int wi = W[i];
    if (wi >= 0) {
      const int jlo = max(LB[i], -i);
      const int jhi = min(UB[i], ncols - 1 - i);
      float* const acol = A + (int64_t)wi * d;
      float a[R];
      load_col<R>(a, acol, lane, d);
      float daa[R];
      zero_col<R>(daa);
      const float ascale = TRAIN ? scale_of(wi, vexp, smode) : 1.0f;
      bool touched = false;

      for (int base = jlo; base <= jhi; base += kWave) {
        // Lane l looks at window offset base+l: word id, validity, and its step scale.
        const int j = base + lane;
        int wl = -1;
        if (j <= jhi && j != 0) wl = W[i + j];
        const bool ok = wl >= 0;
        const float sl = (TRAIN && ok) ? scale_of(wl, vexp, smode) : 0.0f;
        unsigned long long mask = __ballot(ok);

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
          int wb[CH];
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (c < n) {
              wb[c] = read_lane(wl, src[c]);
              load_col<R>(b[c], B + (int64_t)wb[c] * d, lane, d);
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
                atomic_axpy_col<R>(B + (int64_t)wb[c] * d, bs * g, a, lane, d);
              }
            }
            touched = true;
          } else {
            if (lane < n) lsum += log(fmax((double)sg, floorv));
          }
        }
      }
      if (TRAIN && touched) atomic_add_col<R>(acol, daa, lane, d);
    }
  }

  if (!TRAIN) {
    const double wsum = wave_sum_f64(lsum);
    block_store_partial(wsum, partials);
  }
}

// Folds the per-block partial sums in a fixed order (thread t takes t, t+256, ...; then a
// fixed LDS tree), so the result does not depend on block scheduling.
__global__ void __launch_bounds__(kBlock)
finalize_kernel(const double* __restrict__ partials, int64_t n, float* Retval32, double* Retval64) {
  __shared__ double s[kBlock];
  double t = 0.0;
  for (int64_t k = threadIdx.x; k < n; k += kBlock) t += partials[k];
  s[threadIdx.x] = t;
  __syncthreads();
  for (int w = kBlock / 2; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) s[threadIdx.x] += s[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if (Retval32 != nullptr) Retval32[0] += (float)s[0];
    if (Retval64 != nullptr) Retval64[0] += s[0];
  }
}

int max_rows() { return kMaxRounds * kWave; }

int64_t eval_partials_needed(int64_t units) { return blocks_per_xcd(units) * kXcds; }

// Context columns gathered per chunk: as many as fit in roughly 64 registers per lane.
template <int R>
struct PosChunk {
  static constexpr int value = R <= 4 ? 12 : R <= 6 ? 10 : R <= 8 ? 8 : R <= 12 ? 5 : 3;
};

template <int R, bool TRAIN>
static hipError_t launch_pos_r(hipStream_t stream, int d, int ncols, const int* W, const int* LB,
                               const int* UB, float* A, float* B, float lrate, float vexp,
                               double floorv, double* partials) {
  const int64_t per_xcd = blocks_per_xcd(ncols);
  const dim3 grid((unsigned)(per_xcd * kXcds));
  hipLaunchKernelGGL((pos_kernel<R, PosChunk<R>::value, TRAIN>), grid, dim3(kBlock), 0, stream, d,
                     ncols, per_xcd, W, LB, UB, A, B, lrate, vexp, scale_mode(vexp), floorv,
                     partials);
  return hipGetLastError();
}

hipError_t launch_pos(hipStream_t stream, int nrows, int ncols, const int* W, const int* LB,
                      const int* UB, float* A, float* B, float lrate, float vexp) {
  const int rounds = (nrows + kWave - 1) / kWave;
#define CALL(R) \
  return launch_pos_r<R, true>(stream, nrows, ncols, W, LB, UB, A, B, lrate, vexp, 0.0, nullptr)
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
}

hipError_t launch_finalize(hipStream_t stream, const double* partials, int64_t n, float* Retval32,
                           double* Retval64) {
  hipLaunchKernelGGL(finalize_kernel, dim3(1), dim3(kBlock), 0, stream, partials, n, Retval32,
                     Retval64);
  return hipGetLastError();
}

hipError_t launch_eval_pos(hipStream_t stream, int nrows, int ncols, const int* W, const int* LB,
                           const int* UB, const float* A, const float* B, double floorv,
                           double* partials, float* Retval32, double* Retval64) {
  const int rounds = (nrows + kWave - 1) / kWave;
  hipError_t err = hipSuccess;
#define CALL(R)                                                                                  \
  err = launch_pos_r<R, false>(stream, nrows, ncols, W, LB, UB, const_cast<float*>(A),           \
                               const_cast<float*>(B), 0.0f, 0.0f, floorv, partials);             \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, eval_partials_needed(ncols), Retval32, Retval64);
}

}  // namespace w2v
