// Negative pass and its forward twin on bfloat16 tables (gfx950, wave64).
//
// One wavefront owns one group of nwa x nwb words.  It widens the group's nwb B columns into
// registers, keeps an fp32 delta for each of them, and streams the nwa A columns through: each A
// column is widened once, dotted with every B column (wave-level reduction), takes its own delta
// from all of them and is written back at once, narrowed with stochastic rounding; the B columns
// are written after the last A column.  All dots of a group therefore see the tables as they
// were when the group started, which is what the reference's CPU loop computes for a group
// without repeated words (jni/src/BIDMach_CPUMACH.c:210-254: A is written after every dot of the
// group, a B column after its own dots).  A write-back adds the wave's delta to the column as
// it is at that moment (compare-and-swap per 4-byte word), so concurrent updates of one column by
// several waves are all kept.
//
// Every wave is persistent and walks a contiguous range of groups in order.
#include "w2v_bf16.h"
#include "w2v_internal.h"

namespace w2v {

namespace {

constexpr int64_t kMinGroupsPerWave = 4;

// A launch that the device-side count finds full of frequent words (launch_is_ordered,
// w2v_device.h) is done by the row-by-row kernel of w2v_bf16_neg_rows.hip, and this kernel returns
// at once (per_wave_ordered == 0); for a shape that kernel has no instance for, this one runs on
// a few waves (ranges of per_wave_ordered groups; waves beyond the last range find it empty).
template <int RP, bool ALIGNED, int MAXB, bool EVAL>
__global__ void __launch_bounds__(kBlock)
neg_bf16_kernel(int d, int n, int64_t per_wave, int64_t per_wave_ordered, int nwa, int nwb,
                const int* __restrict__ WA, const int* __restrict__ WB, uint16_t* A, uint16_t* B,
                float lrate, float vexp, int smode, uint64_t seed, double floorv,
                double* __restrict__ Retval, HotCols hot, Shadow shadow_arg) {
  if (!EVAL) {
    const Shadow shadow = resolve_hot_mode(shadow_arg);
    if (launch_is_ordered(shadow_arg, shadow)) {
      if (per_wave_ordered == 0) return;
      per_wave = per_wave_ordered;
    }
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int copy = (blockIdx.x * kWavesPerBlock + wave) & (kTopCopies - 1);
  const int64_t first = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * per_wave;
  int64_t last = first + per_wave;
  if (last > n) last = n;
  double lsum = 0.0;
  for (int64_t i = first; i < last; ++i) {
    // MAXB columns of B at a time: several trips only in the forward-only instance (an update
    // of a group with more B words goes to the row-by-row kernel, w2v_bf16_neg_rows.h)
    for (int kb = 0; kb < nwb; kb += MAXB) {
    float b[MAXB][2 * RP], dbb[MAXB][2 * RP];
    float bscale[MAXB];
    int wb[MAXB];
#pragma unroll
    for (int k = 0; k < MAXB; ++k) {
      // an id below zero (the positive stream's mark for a dropped word) skips its pairs, as in
      // the fp32 kernels; wb[k] < 0 also stands for kb + k >= nwb from here on
      wb[k] = -1;
      bscale[k] = 0.0f;
      if (kb + k < nwb) wb[k] = __builtin_amdgcn_readfirstlane(WB[i * nwb + kb + k]);
      if (wb[k] >= 0) {
        load_col16<RP, ALIGNED>(b[k], B + (int64_t)wb[k] * d, lane, d);
        if (!EVAL) bscale[k] = scale_of(wb[k], vexp, smode);
      } else {
#pragma unroll
        for (int r = 0; r < 2 * RP; ++r) b[k][r] = 0.0f;
      }
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) dbb[k][r] = 0.0f;
    }
    // (the side columns of the frequent words only now, when every table column has been asked
    // for: read_side uses what it reads at once, so inside the loop above each frequent column
    // would be waited for before the next one is requested)
    if (!EVAL) {
#pragma unroll
      for (int k = 0; k < MAXB; ++k) {
        if (wb[k] >= 0 && wb[k] < hot.n) read_side<RP>(b[k], hot.sb, hot.n, wb[k], lane, d);
      }
    }
    // the next A column is requested before the current one is written back, so its gather
    // overlaps the exchange; a word that occurs twice among a group's A words is then dotted as
    // it was before the first of its two updates, as in the reference, which writes A after
    // every dot of the group
    float a[2 * RP], anext[2 * RP];
    int wa = __builtin_amdgcn_readfirstlane(WA[i * nwa]);
    if (wa >= 0) {
      load_col16<RP, ALIGNED>(a, A + (int64_t)wa * d, lane, d);
      if (!EVAL && wa < hot.n) read_side<RP>(a, hot.sa, hot.n, wa, lane, d);
    }
    for (int j = 0; j < nwa; ++j) {
      uint16_t* acol = A + (int64_t)wa * d;
      const bool ahot = !EVAL && wa < hot.n;
      int wanext = -1;
      // (the next column's side column waits in registers of its own until the column becomes
      // the current one: added here, it would be waited for before this column's dots; a word
      // with several side columns keeps the plain way)
      float anext_side[2 * RP];
      bool side_pending = false;
      if (j + 1 < nwa) {
        wanext = __builtin_amdgcn_readfirstlane(WA[i * nwa + j + 1]);
        if (wanext >= 0) {
          load_col16<RP, ALIGNED>(anext, A + (int64_t)wanext * d, lane, d);
          if (!EVAL && wanext < hot.n) {
            if (wanext < kTopWords && hot.n >= kTopWords) {
              read_side<RP>(anext, hot.sa, hot.n, wanext, lane, d);
            } else {
              side_col_request<RP>(anext_side, hot.sa + (int64_t)wanext * side_stride(d), lane, d);
              side_pending = true;
            }
          }
        }
      }
      float daa[2 * RP];
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) daa[r] = 0.0f;
      const float ascale = (EVAL || wa < 0) ? 1.0f : scale_of(wa, vexp, smode);
      // lane k forms the sigmoid (and, in the forward instance, the log term) of the dot with B
      // column k: one evaluation per A column instead of one per pair
      float pre = 0.0f;
      bool live = false;
#pragma unroll
      for (int k = 0; k < MAXB; ++k) {
        if (wa >= 0 && wb[k] >= 0) {
          float part = 0.0f;
#pragma unroll
          for (int r = 0; r < 2 * RP; ++r) part = fmaf(a[r], b[k][r], part);
          const float sum = wave_sum(part);
          pre = (lane == k) ? sum : pre;
          live = (lane == k) ? true : live;
        }
      }
      const float sgl = sat_sigmoid(pre);
      if (EVAL) {
        if (live) lsum += log(fmax(1.0 - (double)sgl, floorv));
      } else {
#pragma unroll
        for (int k = 0; k < MAXB; ++k) {
          if (wa >= 0 && wb[k] >= 0) {
            const float g = -lrate * read_lane(sgl, k);
            const float ga = ascale * g;
            const float gb = bscale[k] * g;
#pragma unroll
            for (int r = 0; r < 2 * RP; ++r) {
              dbb[k][r] = fmaf(gb, a[r], dbb[k][r]);
              daa[r] = fmaf(ga, b[k][r], daa[r]);
            }
          }
        }
      }
      if (!EVAL && wa >= 0) {
        if (ahot)
          write_side<RP>(hot.sa, hot.n, wa, copy, daa, lane, d);
        else
          add_col16<RP, ALIGNED>(acol, a, daa, lane, d,
                                 sr_key(seed, (uint32_t)i, 0x10000U + (uint32_t)j));
      }
      if (j + 1 < nwa) {
        wa = wanext;
#pragma unroll
        for (int r = 0; r < 2 * RP; ++r) a[r] = anext[r];
        if (side_pending) side_col_add<RP>(a, anext_side);
      }
    }
    if (!EVAL) {
      if (ALIGNED) {
        // the exchanges of all B columns are in flight together before the first result is used
        uint32_t guess[MAXB][RP], found[MAXB][RP];
#pragma unroll
        for (int k = 0; k < MAXB; ++k) {
          if (wb[k] >= 0) {
            if (wb[k] < hot.n)
              write_side<RP>(hot.sb, hot.n, wb[k], copy, dbb[k], lane, d);
            else
              cas_first<RP>(B + (int64_t)wb[k] * d, b[k], dbb[k], lane, d,
                            sr_key(seed, (uint32_t)i, (uint32_t)k), guess[k], found[k]);
          }
        }
#pragma unroll
        for (int k = 0; k < MAXB; ++k) {
          if (wb[k] >= 0 && wb[k] >= hot.n)
            cas_rest<RP>(B + (int64_t)wb[k] * d, dbb[k], lane, d,
                         sr_key(seed, (uint32_t)i, (uint32_t)k), guess[k], found[k]);
        }
      } else {
#pragma unroll
        for (int k = 0; k < MAXB; ++k) {
          if (wb[k] >= 0) {
            if (wb[k] < hot.n)
              write_side<RP>(hot.sb, hot.n, wb[k], copy, dbb[k], lane, d);
            else
              add_col16<RP, false>(B + (int64_t)wb[k] * d, b[k], dbb[k], lane, d,
                                   sr_key(seed, (uint32_t)i, (uint32_t)k));
          }
        }
      }
    }
    }
  }
  if (EVAL) {
    // every lane holds the terms of its B column: one double atomic per wave
    const double total = wave_sum_f64(lsum);
    if (lane == 0 && total != 0.0) atomicAdd(Retval, total);
  }
}

constexpr int kNegFallbackWaves = 32;   // workers of an ordered launch without a rows instance

template <int RP, bool ALIGNED, int MAXB, bool EVAL>
hipError_t launch(hipStream_t stream, int d, int n, int nwa, int nwb, const int* WA,
                  const int* WB, uint16_t* A, uint16_t* B, float lrate, float vexp, uint64_t seed,
                  double floorv, double* Retval, HotCols hot, Shadow shadow) {
  auto kern = neg_bf16_kernel<RP, ALIGNED, MAXB, EVAL>;
  int64_t nwg = 0;
  hipError_t err = persistent_grid(reinterpret_cast<const void*>(kern), kBlock, 0, n,
                                   kMinGroupsPerWave * kWavesPerBlock, &nwg);
  if (err != hipSuccess) return err;
  const int64_t per_wave = ((int64_t)n + nwg * kWavesPerBlock - 1) / (nwg * kWavesPerBlock);
  nwg = ((int64_t)n + per_wave * kWavesPerBlock - 1) / (per_wave * kWavesPerBlock);
  bool rows = false;
  int64_t per_wave_ordered = 0;
  if (!EVAL) {
    err = prepare_hot_mode(stream, WB, (int64_t)n * nwb, WA, (int64_t)n * nwa, nullptr, nullptr, d,
                           nwg, kWavesPerBlock, &shadow);
    if (err != hipSuccess) return err;
    if (nwb > MAXB) {
      // this kernel holds a group's B columns in registers: wider groups go to the row-by-row
      // kernel whatever the launch holds, on the ordered form's number of workers
      if (!neg_rows_bf16_available(d, nwa)) return hipErrorInvalidValue;
      shadow.ordered = 2;
      note_last_launch(shadow);
    }
    rows = shadow.ordered != 0 && neg_rows_bf16_available(d, nwa);
    if (shadow.ordered != 0 && !rows) {
      int64_t waves = kNegFallbackWaves;
      const int limit = get_max_workgroups();
      if (limit > 0 && waves > (int64_t)limit * kWavesPerBlock) waves = (int64_t)limit * kWavesPerBlock;
      if (waves > nwg * kWavesPerBlock) waves = nwg * kWavesPerBlock;   // the grid that is launched
      per_wave_ordered = ((int64_t)n + waves - 1) / waves;
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, n, per_wave,
                     per_wave_ordered, nwa, nwb, WA, WB, A, B, lrate, vexp, scale_mode(vexp), seed,
                     floorv, Retval, hot, shadow);
  hipError_t lerr = hipGetLastError();
  if (lerr != hipSuccess || EVAL) return lerr;
  if (rows) {
    const int64_t chains = ordered_neg_chains(kWavesPerBlock, kNegRowWorkersBf16);
    // words that are rare within the launch are written back with plain stores (store_col16)
    lerr = prepare_rare_words(stream, WA, (int64_t)n * nwa, WB, (int64_t)n * nwb, 0x7fffffff, n,
                              chains, &shadow, kRareCapOrderedBf16);
    if (lerr != hipSuccess) return lerr;
    lerr = launch_neg_rows_bf16(stream, d, n, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, hot,
                                ordered_neg_chains(kWavesPerBlock, kNegRowWorkersBf16), shadow);
    if (lerr != hipSuccess) return lerr;
  }
  if (hot.n == 0) return hipSuccess;
  return launch_fold_bf16(stream, d, A, B, seed, hot, shadow, rows);
}

template <bool ALIGNED, bool EVAL>
hipError_t dispatch(hipStream_t stream, int d, int n, int nwa, int nwb, const int* WA,
                    const int* WB, uint16_t* A, uint16_t* B, float lrate, float vexp,
                    uint64_t seed, double floorv, double* Retval, HotCols hot, Shadow shadow) {
  const int rp = (d + 127) / 128;
  if (nwb <= 5) {
#define W2V_CALL(RP_)                                                                         \
  return launch<RP_, ALIGNED, 5, EVAL>(stream, d, n, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, \
                                       floorv, Retval, hot, shadow)
    W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
  }
#define W2V_CALL(RP_)                                                                         \
  return launch<RP_, ALIGNED, 8, EVAL>(stream, d, n, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, \
                                       floorv, Retval, hot, shadow)
  W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
}

bool pair_aligned(int d, const void* A, const void* B) {
  return (d & 1) == 0 && (reinterpret_cast<uintptr_t>(A) & 3) == 0 &&
         (reinterpret_cast<uintptr_t>(B) & 3) == 0;
}

}  // namespace

hipError_t launch_neg_bf16(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                           const int* WA, const int* WB, uint16_t* A, uint16_t* B, float lrate,
                           float vexp, uint64_t seed, HotCols hot, Shadow shadow) {
  if (nwb < 1 || nwb > kWave) return hipErrorInvalidValue;
  if (pair_aligned(nrows, A, B))
    return dispatch<true, false>(stream, nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed,
                                 0.0, nullptr, hot, shadow);
  return dispatch<false, false>(stream, nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed,
                                0.0, nullptr, hot, shadow);
}

hipError_t launch_eval_neg_bf16(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                const int* WA, const int* WB, const uint16_t* A,
                                const uint16_t* B, double floorv, double* Retval) {
  if (nwb < 1 || nwb > kWave) return hipErrorInvalidValue;
  uint16_t* a = const_cast<uint16_t*>(A);  // the forward instance never stores
  uint16_t* b = const_cast<uint16_t*>(B);
  if (pair_aligned(nrows, A, B))
    return dispatch<true, true>(stream, nrows, ncols, nwa, nwb, WA, WB, a, b, 0.0f, 0.0f, 0,
                                floorv, Retval, HotCols{}, Shadow{});
  return dispatch<false, true>(stream, nrows, ncols, nwa, nwb, WA, WB, a, b, 0.0f, 0.0f, 0, floorv,
                               Retval, HotCols{}, Shadow{});
}

}  // namespace w2v
