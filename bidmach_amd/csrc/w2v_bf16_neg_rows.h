// Ordered form of the negative-sample pass on bfloat16 tables (launch_is_ordered, w2v_device.h):
// the row-by-row order of the reference's CPU loop, jni/src/BIDMach_CPUMACH.c:210-254, as
// w2v_neg_rows.hip has it for fp32 tables.
//
// A wave is one of a few hundred workers and walks a contiguous range of groups, as a thread of
// the reference does (:197-201).  It keeps the group's A columns (widened) and an fp32 delta for
// each in registers and takes the B columns one row at a time: device-scope read (table column,
// plus the side buffer of a frequent word), nwa dots, sigmoid, and the row's delta goes back at
// once (:244-246) - to the side buffer of a frequent word with float atomics, else into the table
// by compare-and-swap with stochastic rounding - before the wave turns to the next B word; the A
// columns are written after the last row (:248-254).  The next row's column is requested while
// the current row is worked on; the exchanges of the A columns are in flight together.  Words
// that are rare within the launch (counted on the device beforehand) are written back with plain
// stores instead of exchanges: nothing to wait for.  (Keeping
// the rows' exchanges in flight as well costs more registers than a wave has: the results spill
// and every spill waits for its exchange, 136 against 122 ms on a 1.2M-group launch.)
// Sums are formed in the order of the group-at-a-time kernel (w2v_bf16_neg.hip) and every write
// uses that kernel's key, so on a minibatch without repeated words both kernels store the same
// bits.
#pragma once
#include "w2v_bf16.h"
#include "w2v_internal.h"

namespace w2v {

namespace rows16 {

template <int RP, bool ALIGNED, int MAXA>
__global__ void __launch_bounds__(kBlock, 1)
neg_rows_bf16_kernel(int d, int n, int64_t per_chain, int nwa, int nwb,
                     const int* __restrict__ WA, const int* __restrict__ WB, uint16_t* A,
                     uint16_t* B, float lrate, float vexp, int smode, uint64_t seed, HotCols hot,
                     Shadow shadow_arg) {
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  if (!launch_is_ordered(shadow_arg, shadow)) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t chain = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t g_begin = chain * per_chain;
  const int64_t g_end = min(g_begin + per_chain, (int64_t)n);

  // A column is requested here and used later: a frequent word's side column goes to registers
  // of its own (`side`) and is added where the column is first used, so that several columns, or
  // a row's column and the arithmetic of the row before it, are in flight together.
  auto request_a = [&](float (&x)[2 * RP], float (&side)[2 * RP], int word) {
    load_col16_fresh<RP, ALIGNED>(x, A + (int64_t)word * d, lane, d);
    if (word < hot.n) side_col_request<RP>(side, hot.sa + (int64_t)word * side_stride(d), lane, d);
  };
  // (table B holds the context words, the frequent ones of a raw stream: its most frequent words'
  // side columns are read and written as delta slots, side_request_ordered)
  auto request_b = [&](float (&x)[2 * RP], float (&side)[2 * RP], float (&side2)[2 * RP],
                       int word) {
    load_col16_fresh<RP, ALIGNED>(x, B + (int64_t)word * d, lane, d);
    if (word < hot.n) side_request_ordered<RP>(side, side2, hot.sb, hot.n, word, chain, lane, d);
  };

  int wal = -1, wbl = -1;
  auto fetch = [&](int64_t g) {
    wal = wbl = -1;
    if (g < g_end) {
      if (lane < nwa) wal = WA[g * nwa + lane];
      if (lane < nwb) wbl = WB[g * nwb + lane];
    }
  };
  fetch(g_begin);
  for (int64_t i = g_begin; i < g_end; ++i) {
    const int wa_l = wal, wb_l = wbl;
    fetch(i + 1);
    const float sal = wa_l >= 0 ? scale_of(wa_l, vexp, smode) : 0.0f;
    const float sbl = wb_l >= 0 ? scale_of(wb_l, vexp, smode) : 0.0f;

    // A word that is neither frequent (side buffer) nor rare within the launch is written back by
    // compare-and-swap; a rare one by a plain store (store_col16).
    // The counters of the group's words that may be rare within the launch are requested first
    // and looked at after the columns have been requested (below): the other way round the
    // columns would wait for the counters, or the counters for the columns.
    const int seen_a = wa_l >= hot.n ? rare_seen(shadow, wa_l) : 0x7fffffff;
    const int seen_b = wb_l >= hot.n ? rare_seen(shadow, wb_l) : 0x7fffffff;

    float a[MAXA][2 * RP], daa[MAXA][2 * RP];
    int wa[MAXA];
#pragma unroll
    for (int j = 0; j < MAXA; ++j) {
      wa[j] = -1;
      if (j < nwa) wa[j] = read_lane(wa_l, j);
      // (the side column of a frequent word waits in the registers of the column's delta, which
      // are not needed before the first row)
      if (wa[j] >= 0) request_a(a[j], daa[j], wa[j]);
    }

    // a B word that was a B word of an earlier row of this group is read only after that row's
    // delta has been added
    bool seen_before = false;
    for (int k = 0; k < nwb; ++k)
      if (k < lane && read_lane(wb_l, k) == wb_l) seen_before = true;
    const unsigned long long repeats = __ballot(seen_before && wb_l >= 0);

    float bn[2 * RP], bnside[2 * RP], bnside2[2 * RP];
    int wbn = read_lane(wb_l, 0);
    if (wbn >= 0) request_b(bn, bnside, bnside2, wbn);
    const unsigned long long rare_a = __ballot(seen_a <= shadow.rare_max);
    const unsigned long long rare_b = __ballot(seen_b <= shadow.rare_max);
    // the A columns have been requested, and the first row's column: now their side columns
#pragma unroll
    for (int j = 0; j < MAXA; ++j) {
      if (wa[j] >= 0 && wa[j] < hot.n) side_col_add<RP>(a[j], daa[j]);
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) daa[j][r] = 0.0f;
    }
    for (int k = 0; k < nwb; ++k) {
      const int wb = wbn;
      float b[2 * RP];
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) b[r] = bn[r];
      if (wb >= 0 && wb < hot.n) side_add_ordered<RP>(b, bnside, bnside2, hot.n, wb);
      bool again = false;
      if (k + 1 < nwb) {
        wbn = read_lane(wb_l, k + 1);
        again = wbn >= 0 && ((repeats >> (k + 1)) & 1ull) != 0;
        if (wbn >= 0 && !again) request_b(bn, bnside, bnside2, wbn);
      }
      if (wb >= 0) {
        const float bs = read_lane(sbl, k);
        float dbb[2 * RP];
#pragma unroll
        for (int r = 0; r < 2 * RP; ++r) dbb[r] = 0.0f;
        // lane j forms the sigmoid of the dot with A column j: one evaluation per row
        float pre = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXA; ++j) {
          if (wa[j] >= 0) {
            float part = 0.0f;
#pragma unroll
            for (int r = 0; r < 2 * RP; ++r) part = fmaf(a[j][r], b[r], part);
            const float sum = wave_sum(part);
            pre = (lane == j) ? sum : pre;
          }
        }
        const float gl = -lrate * sat_sigmoid(pre);
#pragma unroll
        for (int j = 0; j < MAXA; ++j) {
          if (wa[j] >= 0) {
            const float g = read_lane(gl, j);
            const float ga = read_lane(sal, j) * g;
            const float gb = bs * g;
#pragma unroll
            for (int r = 0; r < 2 * RP; ++r) {
              dbb[r] = fmaf(gb, a[j][r], dbb[r]);
              daa[j][r] = fmaf(ga, b[r], daa[j][r]);
            }
          }
        }
        const uint32_t key = sr_key(seed, (uint32_t)i, (uint32_t)k);
        if (wb < hot.n)
          write_side_ordered<RP>(hot.sb, hot.n, wb, chain, dbb, lane, d);
        else if ((rare_b >> k) & 1ull)
          store_col16<RP, ALIGNED>(B + (int64_t)wb * d, b, dbb, lane, d, key);
        else
          add_col16<RP, ALIGNED>(B + (int64_t)wb * d, b, dbb, lane, d, key);
      }
      if (again) {
        wait_for_own_writes();
        request_b(bn, bnside, bnside2, wbn);
      }
    }

    // the A columns, their exchanges in flight together
    {
      uint32_t ga_[MAXA][RP], fa_[MAXA][RP];
      bool cas[MAXA];
#pragma unroll
      for (int j = 0; j < MAXA; ++j) {
        cas[j] = false;
        if (wa[j] >= 0) {
          const uint32_t key = sr_key(seed, (uint32_t)i, 0x10000U + (uint32_t)j);
          // (a word that is an A word of the group twice keeps the exchange: two plain stores
          // of "value read at the start of the group + delta" would keep only the second)
          bool twice = false;
#pragma unroll
          for (int j2 = 0; j2 < MAXA; ++j2) twice = twice || (j2 != j && wa[j2] == wa[j]);
          if (wa[j] < hot.n) {
            write_side_main<RP>(hot.sa, wa[j], daa[j], lane, d);
          } else if (!twice && ((rare_a >> j) & 1ull)) {
            store_col16<RP, ALIGNED>(A + (int64_t)wa[j] * d, a[j], daa[j], lane, d, key);
          } else if (ALIGNED) {
            cas[j] = true;
            cas_first<RP>(A + (int64_t)wa[j] * d, a[j], daa[j], lane, d, key, ga_[j], fa_[j]);
          } else {
            add_col16<RP, false>(A + (int64_t)wa[j] * d, a[j], daa[j], lane, d, key);
          }
        }
      }
      if (ALIGNED) {
#pragma unroll
        for (int j = 0; j < MAXA; ++j) {
          if (cas[j])
            cas_rest<RP>(A + (int64_t)wa[j] * d, daa[j], lane, d,
                         sr_key(seed, (uint32_t)i, 0x10000U + (uint32_t)j), ga_[j], fa_[j]);
        }
      }
    }
    // the adds of this group are performed before the next group's columns are read
    wait_for_own_writes();
  }
}

constexpr int64_t kMinGroupsPerChain = 16;

template <int RP, bool ALIGNED, int MAXA>
hipError_t launch(hipStream_t stream, int d, int n, int nwa, int nwb, const int* WA,
                  const int* WB, uint16_t* A, uint16_t* B, float lrate, float vexp, uint64_t seed,
                  HotCols hot, int64_t chains, const Shadow& shadow) {
  const int64_t by_size = ((int64_t)n + kMinGroupsPerChain - 1) / kMinGroupsPerChain;
  if (chains > by_size) chains = by_size;
  if (chains < 1) chains = 1;
  const int64_t per_chain = ((int64_t)n + chains - 1) / chains;   // waves beyond: empty range
  hipLaunchKernelGGL((neg_rows_bf16_kernel<RP, ALIGNED, MAXA>),
                     dim3((unsigned)((chains + kWavesPerBlock - 1) / kWavesPerBlock)),
                     dim3(kBlock), 0, stream, d, n, per_chain, nwa, nwb, WA, WB, A, B, lrate, vexp,
                     scale_mode(vexp), seed, hot, shadow);
  return hipGetLastError();
}

// Shapes with an instance: up to 5 A columns at any dim, up to 16 at dim <= 512 (the register
// arrays of more or wider columns would spill).
inline bool has_instance(int d, int nwa) {
  const int rp = (d + 127) / 128;
  return nwa <= 5 || (nwa <= 16 && rp <= 4);
}

template <bool ALIGNED>
hipError_t dispatch(hipStream_t stream, int d, int n, int nwa, int nwb, const int* WA,
                    const int* WB, uint16_t* A, uint16_t* B, float lrate, float vexp,
                    uint64_t seed, HotCols hot, int64_t chains, const Shadow& shadow) {
  const int rp = (d + 127) / 128;
  if (nwb < 1 || nwb > kWave || !has_instance(d, nwa)) return hipErrorInvalidValue;
  if (nwa <= 5) {
#define W2V_CALL(RP_)                                                                           \
  return launch<RP_, ALIGNED, 5>(stream, d, n, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, hot, \
                                 chains, shadow)
    W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
  }
  switch (rp) {
#define W2V_CALL(RP_)                                                                            \
  case RP_:                                                                                      \
    return launch<RP_, ALIGNED, 16>(stream, d, n, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, hot, \
                                    chains, shadow)
    W2V_CALL(1); W2V_CALL(2); W2V_CALL(3); W2V_CALL(4);
#undef W2V_CALL
    default: break;
  }
  return hipErrorInvalidValue;
}

}  // namespace rows16

}  // namespace w2v
