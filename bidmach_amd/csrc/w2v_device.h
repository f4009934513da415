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

// Hogwild scatter: col[e] += alpha * x[e] with one hardware float atomic per lane and round
// (global_atomic_add_f32, no return value, no compare-and-swap loop).
template <int R>
__device__ __forceinline__ void atomic_axpy_col(float* __restrict__ col, float alpha,
                                                const float (&x)[R], int lane, int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    if (r < R - 1 || e < d) unsafeAtomicAdd(col + e, alpha * x[r]);
  }
}

template <int R>
__device__ __forceinline__ void atomic_add_col(float* __restrict__ col, const float (&x)[R],
                                               int lane, int d) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int e = r * kWave + lane;
    if (r < R - 1 || e < d) unsafeAtomicAdd(col + e, x[r]);
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
