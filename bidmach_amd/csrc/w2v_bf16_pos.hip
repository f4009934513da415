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
      // overlaps the exchange -- unless it is the same word again, which has to see this update
      int wbnext = 0;
      const int jnext = next_context(j + 1, wbnext);
      const bool ahead = jnext <= hi && wbnext != wb;
      if (ahead) load_b(bnext, wbnext);
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

// Ordered form of the update (launch_is_ordered, w2v_device.h): the token-by-token order of the
// reference's CPU loop (BIDMach_CPUMACH.c:26-68) on a bounded number of workers, as
// pos_chain_kernel (w2v_pos.hip) has it for fp32 tables.  A wave walks a contiguous range of
// centre tokens one after the other; per token it reads the centre's A column and the window's B
// columns with device-scope loads (table column plus the side buffer of a frequent word), writes
// every B delta back at once - float atomics on the side buffer of a frequent word, else a
// compare-and-swap with stochastic rounding, the exchanges of a chunk of columns in flight
// together - and the A delta after the window, and waits for all of it before the next token's
// reads.  A word that stands at several offsets of one window is worked on in rounds, occurrence
// r after the writes of occurrence r - 1.  Every write uses the key of pos_bf16_kernel, so on a
// minibatch without repeated words both kernels store the same bits.
template <int RP>
struct PosChunk16 {
  // (larger chunks cost more registers than a wave has, and a spilled exchange result is waited
  // for at once: 8 columns at dim 300 are slower than 4, 165 against 145 ms per 1M tokens)
  static constexpr int value = RP <= 2 ? 8 : RP <= 6 ? 4 : 3;
};

template <int RP, bool ALIGNED, int CH>
__global__ void __launch_bounds__(kBlock, 1)
pos_chain_bf16_kernel(int d, int n, int64_t per_chain, const int* __restrict__ W,
                      const int* __restrict__ LB, const int* __restrict__ UB, uint16_t* A,
                      uint16_t* B, float lrate, float vexp, int smode, uint64_t seed, HotCols hot,
                      Shadow shadow_arg) {
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  if (!launch_is_ordered(shadow_arg, shadow)) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t chain = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t i_begin = chain * per_chain;
  const int64_t i_end = min(i_begin + per_chain, (int64_t)n);

  // the ids of the next token and of its window (offsets -32..31) are fetched while the current
  // token is worked on
  constexpr int kLook = 32;
  int lb = 0, ub = 0, wnear = -1;
  auto fetch = [&](int64_t t) {
    lb = ub = 0;
    wnear = -1;
    if (t < i_end) {
      lb = LB[t];
      ub = UB[t];
      const int64_t p = t + lane - kLook;
      if (p >= 0 && p < n) wnear = W[p];
    }
  };
  fetch(i_begin);
  for (int64_t unit = i_begin; unit < i_end; ++unit) {
    const int i = (int)unit;
    const int wi = read_lane(wnear, kLook);
    const int jlo = max(__builtin_amdgcn_readfirstlane(lb), -i);
    const int jhi = min(__builtin_amdgcn_readfirstlane(ub), n - 1 - i);
    const int wnear_now = wnear;
    fetch(unit + 1);
    if (wi < 0) continue;
    uint16_t* const acol = A + (int64_t)wi * d;
    float a[2 * RP], daa[2 * RP];
    load_col16_fresh<RP, ALIGNED>(a, acol, lane, d);
    if (wi < hot.n) read_side_main<RP>(a, hot.sa, wi, lane, d);
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) daa[r] = 0.0f;
    const float ascale = scale_of(wi, vexp, smode);
    bool touched = false, a_written = false;
    const uint32_t akey = sr_key(seed, (uint32_t)i, 0U);
    const bool a_rare = wi >= hot.n && is_rare(shadow, wi);

    const int base0 = min(jlo, -kLook);
    for (int base = base0; base <= jhi; base += kWave) {
      // lane l looks at window offset base + l; the offsets -32..31 were fetched beforehand (a
      // window wider than 64 offsets is worked on in slabs, each after the writes of the last)
      if (base != base0) wait_for_own_writes();
      const int j = base + lane;
      int wl = -1;
      if (j >= jlo && j <= jhi && j != 0) wl = base == -kLook ? wnear_now : W[i + j];
      const bool ok = wl >= 0;
      const float sl = ok ? scale_of(wl, vexp, smode) : 0.0f;
      const unsigned long long valid = __ballot(ok);
      int occ = 0;
      {
        unsigned long long m = valid;
        while (m != 0ull) {
          const int l = __builtin_ctzll(m);
          m &= m - 1ull;
          if (l < lane && read_lane(wl, l) == wl) ++occ;
        }
      }
      for (int round = 0;; ++round) {
        unsigned long long mask = __ballot(ok && occ == round);
        if (mask == 0ull) break;
        if (round > 0) wait_for_own_writes();
        while (mask != 0ull) {
          int src[CH];
          int nc = 0;
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (mask != 0ull) {
              src[c] = __builtin_ctzll(mask);
              mask &= mask - 1ull;
              nc = c + 1;
            } else {
              src[c] = -1;
            }
          }
          float b[CH][2 * RP];
          float gbs[CH];
          uint32_t guess[CH][RP], found[CH][RP];
          int wb[CH];
          bool cas[CH];
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            wb[c] = -1;
            cas[c] = false;
            if (c < nc) {
              wb[c] = read_lane(wl, src[c]);
              load_col16_fresh<RP, ALIGNED>(b[c], B + (int64_t)wb[c] * d, lane, d);
              if (wb[c] < hot.n) read_side_main<RP>(b[c], hot.sb, wb[c], lane, d);
            }
          }
          // lane c forms the sigmoid of the dot with context c: one evaluation per chunk
          float pre = 0.0f;
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (c < nc) {
              float part = 0.0f;
#pragma unroll
              for (int r = 0; r < 2 * RP; ++r) part = fmaf(a[r], b[c][r], part);
              const float sum = wave_sum(part);
              pre = (lane == c) ? sum : pre;
            }
          }
          const float gl = lrate * (1.0f - sat_sigmoid(pre));
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (c < nc) {
              const float g = read_lane(gl, c);
              const float ga = ascale * g;
              const float gb = read_lane(sl, src[c]) * g;
              gbs[c] = gb;
              float db[2 * RP];
#pragma unroll
              for (int r = 0; r < 2 * RP; ++r) {
                daa[r] = fmaf(ga, b[c][r], daa[r]);
                db[r] = gb * a[r];
              }
              uint16_t* const bcol = B + (int64_t)wb[c] * d;
              const uint32_t key = sr_key(seed, (uint32_t)i, (uint32_t)(base + src[c]));
              cas[c] = false;
              if (wb[c] < hot.n) {
                write_side_main<RP>(hot.sb, wb[c], db, lane, d);
              } else if (is_rare(shadow, wb[c])) {
                // rare within the launch: a plain store, nothing to wait for (store_col16)
                store_col16<RP, ALIGNED>(bcol, b[c], db, lane, d, key);
              } else if (ALIGNED) {
                cas[c] = true;
                cas_first<RP>(bcol, b[c], db, lane, d, key, guess[c], found[c]);
              } else {
                add_col16<RP, false>(bcol, b[c], db, lane, d, key);
              }
            }
          }
          touched = true;
          // after the token's last chunk the centre's delta is complete: its exchange joins
          // those of the chunk's columns in flight
          const bool last = mask == 0ull && __ballot(ok && occ == round + 1) == 0ull &&
                            base + kWave > jhi;
          uint32_t aguess[RP], afound[RP];
          bool acas = false;
          if (last) {
            a_written = true;
            if (wi < hot.n) {
              write_side_main<RP>(hot.sa, wi, daa, lane, d);
            } else if (a_rare) {
              store_col16<RP, ALIGNED>(acol, a, daa, lane, d, akey);
            } else if (ALIGNED) {
              acas = true;
              cas_first<RP>(acol, a, daa, lane, d, akey, aguess, afound);
            } else {
              add_col16<RP, false>(acol, a, daa, lane, d, akey);
            }
          }
          if (ALIGNED) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
              if (cas[c])
                cas_rest_axpy<RP>(B + (int64_t)wb[c] * d, gbs[c], a, lane, d,
                                  sr_key(seed, (uint32_t)i, (uint32_t)(base + src[c])), guess[c],
                                  found[c]);
            }
            if (acas) cas_rest<RP>(acol, daa, lane, d, akey, aguess, afound);
          }
        }
      }
    }
    if (touched) {
      if (!a_written) {
        if (wi < hot.n)
          write_side_main<RP>(hot.sa, wi, daa, lane, d);
        else if (a_rare)
          store_col16<RP, ALIGNED>(acol, a, daa, lane, d, akey);
        else
          add_col16<RP, ALIGNED>(acol, a, daa, lane, d, akey);
      }
      // the writes of this token are performed before the next token's columns are read
      wait_for_own_writes();
    }
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
    const int64_t chains = ordered_pos_chains(n, shift, kPosChainsBf16);
    const int64_t per_chain = ((int64_t)n + chains - 1) / chains;   // waves beyond: empty range
    // words that are rare within the launch are written back with plain stores (store_col16)
    lerr = prepare_rare_words(stream, W, n, nullptr, 0, 0x7fffffff, n, chains, &shadow,
                              kRareCapOrderedBf16);
    if (lerr != hipSuccess) return lerr;
    hipLaunchKernelGGL((pos_chain_bf16_kernel<RP, ALIGNED, PosChunk16<RP>::value>),
                       dim3((unsigned)((chains + kWavesPerBlock - 1) / kWavesPerBlock)),
                       dim3(kBlock), 0, stream, d, n, per_chain, W, LB, UB, A, B, lrate, vexp,
                       scale_mode(vexp), seed, hot, shadow);
    lerr = hipGetLastError();
    if (lerr != hipSuccess) return lerr;
  }
  if (hot.n == 0) return hipSuccess;
  return launch_fold_bf16(stream, d, A, B, seed, hot);
}

// One workgroup per frequent word and table: table column = narrow(widen(column) + side buffer),
// side buffer = 0.  Elements whose side buffer is zero are left alone, so a word the call did not
// update keeps its bits (and a word id beyond the vocabulary is never touched).
__global__ void __launch_bounds__(kBlock)
fold_bf16_kernel(int d, uint16_t* A, uint16_t* B, uint64_t seed, HotCols hot) {
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
      v += u;
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
                            HotCols hot) {
  if (hot.n <= 0) return hipSuccess;
  hipLaunchKernelGGL(fold_bf16_kernel, dim3(2u * (unsigned)hot.n), dim3(kBlock), 0, stream, nrows,
                     A, B, seed, hot);
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
