// Positive pass and its forward twin on bfloat16 tables (gfx950, wave64).
//
// One wavefront owns one centre token.  It widens the centre's A column into registers, walks
// the window, and for every valid context widens the B column, reduces the dot over the wave,
// forms the fused sigmoid gradient, accumulates the centre's delta in fp32 registers and writes
// the context column back at once, narrowed with stochastic rounding; the centre column is
// written after the window.  That is the order of the reference's CPU loop
// (jni/src/BIDMach_CPUMACH.c:29-67: B inside the window loop, A after it).  A write-back adds
// the wave's delta to the column as it is at that moment (compare-and-swap per 4-byte word), so
// concurrent updates of one column by several waves are all kept.
//
// Every wave is persistent and walks a contiguous range of tokens in order, as a thread of the
// reference's CPU path does (:21-24): the overlapping windows of neighbouring tokens, which
// rewrite the same context columns ten times over, are then handled by one wave one after the
// other instead of by several waves at once, so those updates are not lost, and the re-read
// columns are still in cache.
#include "w2v_bf16.h"
#include "w2v_internal.h"

namespace w2v {

namespace {

constexpr int64_t kMinTokensPerWave = 16;

// A launch that the device-side count finds full of frequent words is done by
// pos_chain_bf16_kernel below, and this kernel returns at once (launch_is_ordered, w2v_device.h).
template <int RP, bool ALIGNED, bool EVAL>
__global__ void __launch_bounds__(kBlock)
pos_bf16_kernel(int d, int n, int64_t per_wave, const int* __restrict__ W,
                const int* __restrict__ LB, const int* __restrict__ UB, uint16_t* A, uint16_t* B,
                float lrate, float vexp, int smode, uint64_t seed, double floorv,
                double* __restrict__ Retval, HotCols hot, Shadow shadow_arg) {
  if (!EVAL) {
    const Shadow shadow = resolve_hot_mode(shadow_arg);
    if (launch_is_ordered(shadow_arg, shadow)) return;
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int copy = (blockIdx.x * kWavesPerBlock + wave) & (kTopCopies - 1);
  const int64_t first = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * per_wave;
  int64_t last = first + per_wave;
  if (last > n) last = n;
  double lsum = 0.0;
  for (int64_t i = first; i < last; ++i) {
    const int w = __builtin_amdgcn_readfirstlane(W[i]);
    if (w < 0) continue;
    const int lb = __builtin_amdgcn_readfirstlane(LB[i]);
    const int ub = __builtin_amdgcn_readfirstlane(UB[i]);
    uint16_t* acol = A + (int64_t)w * d;
    float a[2 * RP], daa[2 * RP];
    const bool ahot = !EVAL && w < hot.n;
    load_col16<RP, ALIGNED>(a, acol, lane, d);
    if (ahot) read_side<RP>(a, hot.sa, hot.n, w, lane, d);
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) daa[r] = 0.0f;
    const float ascale = EVAL ? 1.0f : scale_of(w, vexp, smode);
    // window clipped to the minibatch, so that the scan below stays inside W
    const int lo = lb < -i ? (int)-i : lb;
    const int hi = ub > n - 1 - i ? (int)(n - 1 - i) : ub;
    // next valid context at or after offset j0 (hi + 1 if none); its word id goes to `word`
    auto next_context = [&](int j0, int& word) {
      for (int j = j0; j <= hi; ++j) {
        if (j == 0) continue;
        const int x = __builtin_amdgcn_readfirstlane(W[i + j]);
        if (x >= 0) {
          word = x;
          return j;
        }
      }
      return hi + 1;
    };
    auto load_b = [&](float (&x)[2 * RP], int word) {
      load_col16<RP, ALIGNED>(x, B + (int64_t)word * d, lane, d);
      if (!EVAL && word < hot.n) read_side<RP>(x, hot.sb, hot.n, word, lane, d);
    };
    int wb = 0;
    int j = next_context(lo, wb);
    float b[2 * RP], bnext[2 * RP];
    if (j <= hi) load_b(b, wb);
    while (j <= hi) {
      // the next context's column is requested before this one is written back, so its gather
      // overlaps the exchange -- unless it is the same word again, which has to see this update.
      // (A frequent word's side column waits in registers of its own until the column becomes
      // the current one: added at once, it would be waited for before this column's dot; a word
      // with several side columns keeps the plain way.)
      int wbnext = 0;
      const int jnext = next_context(j + 1, wbnext);
      const bool ahead = jnext <= hi && wbnext != wb;
      float bnext_side[2 * RP];
      bool side_pending = false;
      if (ahead) {
        if (!EVAL && wbnext < hot.n && !(wbnext < kTopWords && hot.n >= kTopWords)) {
          load_col16<RP, ALIGNED>(bnext, B + (int64_t)wbnext * d, lane, d);
          side_col_request<RP>(bnext_side, hot.sb + (int64_t)wbnext * side_stride(d), lane, d);
          side_pending = true;
        } else {
          load_b(bnext, wbnext);
        }
      }
      uint16_t* bcol = B + (int64_t)wb * d;
      const bool bhot = !EVAL && wb < hot.n;
      float part = 0.0f;
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) part = fmaf(a[r], b[r], part);
      const float sg = sat_sigmoid(wave_sum(part));
      if (EVAL) {
        lsum += log(fmax((double)sg, floorv));
      } else {
        const float g = lrate * (1.0f - sg);
        const float ga = ascale * g;
        const float gb = scale_of(wb, vexp, smode) * g;
        float db[2 * RP];
#pragma unroll
        for (int r = 0; r < 2 * RP; ++r) {
          daa[r] = fmaf(ga, b[r], daa[r]);
          db[r] = gb * a[r];
        }
        if (bhot)
          write_side<RP>(hot.sb, hot.n, wb, copy, db, lane, d);
        else
          add_col16<RP, ALIGNED>(bcol, b, db, lane, d, sr_key(seed, (uint32_t)i, (uint32_t)j));
      }
      if (jnext <= hi && !ahead) load_b(bnext, wbnext);
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) b[r] = bnext[r];
      if (side_pending) side_col_add<RP>(b, bnext_side);
      j = jnext;
      wb = wbnext;
    }
    if (!EVAL) {
      if (ahot)
        write_side<RP>(hot.sa, hot.n, w, copy, daa, lane, d);
      else
        add_col16<RP, ALIGNED>(acol, a, daa, lane, d, sr_key(seed, (uint32_t)i, 0U));
    }
  }
  if (EVAL) {
    // lsum is wave-uniform; one double atomic per wave
    if (lane == 0 && lsum != 0.0) atomicAdd(Retval, lsum);
  }
}

template <int RP, bool ALIGNED, bool EVAL>
hipError_t launch(hipStream_t stream, int d, int n, int shift, const int* W, const int* LB,
                  const int* UB, uint16_t* A, uint16_t* B, float lrate, float vexp, uint64_t seed,
                  double floorv, double* Retval, HotCols hot, Shadow shadow) {
  auto kern = pos_bf16_kernel<RP, ALIGNED, EVAL>;
  int64_t nwg = 0;
  hipError_t err = persistent_grid(reinterpret_cast<const void*>(kern), kBlock, 0, n,
                                   kMinTokensPerWave * kWavesPerBlock, &nwg);
  if (err != hipSuccess) return err;
  const int64_t per_wave = ((int64_t)n + nwg * kWavesPerBlock - 1) / (nwg * kWavesPerBlock);
  nwg = ((int64_t)n + per_wave * kWavesPerBlock - 1) / (per_wave * kWavesPerBlock);
  if (!EVAL) {
    err = prepare_hot_mode(stream, W, n, nullptr, 0, nullptr, nullptr, d, nwg, kWavesPerBlock,
                           &shadow);
    if (err != hipSuccess) return err;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, n, per_wave, W, LB, UB,
                     A, B, lrate, vexp, scale_mode(vexp), seed, floorv, Retval, hot, shadow);
  hipError_t lerr = hipGetLastError();
  if (lerr != hipSuccess || EVAL) return lerr;
  if (shadow.ordered != 0) {
    lerr = launch_pos_chain_bf16(stream, d, n, shift, W, LB, UB, A, B, lrate, vexp, seed, hot,
                                 shadow, ALIGNED);
    if (lerr != hipSuccess) return lerr;
  }
  if (hot.n == 0) return hipSuccess;
  return launch_fold_bf16(stream, d, A, B, seed, hot, shadow, false);
}

// One workgroup per frequent word and table: table column = narrow(widen(column) + side buffer),
// side buffer = 0.  Elements whose side buffer is zero are left alone, so a word the call did not
// update keeps its bits (and a word id beyond the vocabulary is never touched).  The extra side
// columns of the most frequent words are copies to be summed - unless the launch was run by an
// ordered kernel, which uses them as delta slots with twins (side_request_ordered, w2v_bf16.h):
// then the odd slots repeat the even ones and only the even ones count.
__global__ void __launch_bounds__(kBlock)
fold_bf16_kernel(int d, uint16_t* A, uint16_t* B, uint64_t seed, HotCols hot, Shadow shadow_arg,
                 int slots_if_ordered) {
  bool twins = false;
  if (slots_if_ordered) twins = launch_is_ordered(shadow_arg, resolve_hot_mode(shadow_arg));
  const int w = blockIdx.x >> 1;
  const int table_b = blockIdx.x & 1;
  uint16_t* col = (table_b ? B : A) + (int64_t)w * d;
  float* base = table_b ? hot.sb : hot.sa;
  const int64_t stride = side_stride(d);
  const int copies = (w < kTopWords && hot.n >= kTopWords) ? kTopCopies : 1;
  const uint32_t key = sr_key(seed, 0xFFFFFFFFU, fold_slot(table_b, w));
  for (int p = threadIdx.x; p < stride; p += kBlock) {
    const int e = (p >> 7) * 128 + 2 * (p & 63) + ((p >> 6) & 1);   // the element stored at p
    if (e >= d) continue;
    float v = base[(int64_t)w * stride + p];
    bool any = v != 0.0f;
    for (int c = 1; c < copies; ++c) {
      const float u = base[((int64_t)hot.n + (c - 1) * kTopWords + w) * stride + p];
      any = any || u != 0.0f;
      if (!(twins && (c & 1))) v += u;
    }
    if (any) {
      const float x = __builtin_bit_cast(float, (uint32_t)col[e] << 16) + v;
      col[e] = (uint16_t)sr_narrow(x, key, (uint32_t)e);
      base[(int64_t)w * stride + p] = 0.0f;
      for (int c = 1; c < copies; ++c)
        base[((int64_t)hot.n + (c - 1) * kTopWords + w) * stride + p] = 0.0f;
    }
  }
}

__global__ void __launch_bounds__(kBlock)
f32_to_bf16_kernel(size_t n, const float* __restrict__ src, uint16_t* __restrict__ dst) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const uint32_t u = __builtin_bit_cast(uint32_t, src[i]);
    uint32_t h;
    if ((u & 0x7F800000U) == 0x7F800000U)
      h = (u >> 16) | ((u & 0x007FFFFFU) ? 0x40U : 0U);
    else
      h = (u + 0x7FFFU + ((u >> 16) & 1U)) >> 16;
    dst[i] = (uint16_t)h;
  }
}

__global__ void __launch_bounds__(kBlock)
bf16_to_f32_kernel(size_t n, const uint16_t* __restrict__ src, float* __restrict__ dst) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
    dst[i] = __builtin_bit_cast(float, (uint32_t)src[i] << 16);
}

unsigned convert_grid(size_t n) {
  size_t blocks = (n + kBlock - 1) / kBlock;
  if (blocks > 16384) blocks = 16384;
  return (unsigned)blocks;
}

bool pair_aligned(int d, const void* A, const void* B) {
  return (d & 1) == 0 && (reinterpret_cast<uintptr_t>(A) & 3) == 0 &&
         (reinterpret_cast<uintptr_t>(B) & 3) == 0;
}

}  // namespace

hipError_t launch_f32_to_bf16(hipStream_t stream, size_t n, const float* src, uint16_t* dst) {
  hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(convert_grid(n)), dim3(kBlock), 0, stream, n, src,
                     dst);
  return hipGetLastError();
}

hipError_t launch_bf16_to_f32(hipStream_t stream, size_t n, const uint16_t* src, float* dst) {
  hipLaunchKernelGGL(bf16_to_f32_kernel, dim3(convert_grid(n)), dim3(kBlock), 0, stream, n, src,
                     dst);
  return hipGetLastError();
}

hipError_t launch_fold_bf16(hipStream_t stream, int nrows, uint16_t* A, uint16_t* B, uint64_t seed,
                            HotCols hot, const Shadow& shadow, bool slots_if_ordered) {
  if (hot.n <= 0) return hipSuccess;
  hipLaunchKernelGGL(fold_bf16_kernel, dim3(2u * (unsigned)hot.n), dim3(kBlock), 0, stream, nrows,
                     A, B, seed, hot, shadow, slots_if_ordered ? 1 : 0);
  return hipGetLastError();
}

hipError_t launch_pos_bf16(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                           const int* LB, const int* UB, uint16_t* A, uint16_t* B, float lrate,
                           float vexp, uint64_t seed, HotCols hot, Shadow shadow) {
  const int rp = (nrows + 127) / 128;
  if (pair_aligned(nrows, A, B)) {
#define W2V_CALL(RP_)                                                                       \
  return launch<RP_, true, false>(stream, nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, \
                                  seed, 0.0, nullptr, hot, shadow)
    W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
  }
#define W2V_CALL(RP_)                                                                        \
  return launch<RP_, false, false>(stream, nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, \
                                   seed, 0.0, nullptr, hot, shadow)
  W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
}

hipError_t launch_eval_pos_bf16(hipStream_t stream, int nrows, int ncols, const int* W,
                                const int* LB, const int* UB, const uint16_t* A,
                                const uint16_t* B, double floorv, double* Retval) {
  const int rp = (nrows + 127) / 128;
  uint16_t* a = const_cast<uint16_t*>(A);  // the forward instance never stores
  uint16_t* b = const_cast<uint16_t*>(B);
  if (pair_aligned(nrows, A, B)) {
#define W2V_CALL(RP_)                                                                        \
  return launch<RP_, true, true>(stream, nrows, ncols, 0, W, LB, UB, a, b, 0.0f, 0.0f, 0, floorv, \
                                 Retval, HotCols{}, Shadow{})
    W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
  }
#define W2V_CALL(RP_)                                                                         \
  return launch<RP_, false, true>(stream, nrows, ncols, 0, W, LB, UB, a, b, 0.0f, 0.0f, 0, floorv, \
                                  Retval, HotCols{}, Shadow{})
  W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
}

}  // namespace w2v
