// Ordered form of the positive pass on bfloat16 tables (launch_is_ordered, w2v_device.h): the
// token-by-token order of the reference's CPU loop (BIDMach_CPUMACH.c:26-68) on a bounded number
// of workers, as pos_chain_kernel (w2v_pos.hip) has it for fp32 tables.  A worker walks a
// contiguous range of centre tokens one after the other; per token it reads the centre's A column
// and the window's B columns with device-scope loads (table column plus the side buffer of a
// frequent word), writes every B delta back at once - float atomics on the side buffer of a
// frequent word, a plain stochastic-rounded store for a word that is rare within the launch, else
// a compare-and-swap with stochastic rounding, the exchanges of a chunk of columns in flight
// together - and the A delta after the window.  A word that stands at several offsets of one
// window is worked on in rounds, occurrence r after the writes of occurrence r - 1.  Every write
// uses the key of pos_bf16_kernel, so on a minibatch without repeated words both kernels store the
// same bits.
//
// How many workers there may be is set by the held-out loss (every token in flight is a token
// whose updates the others do not see), so what makes the pass faster is the time a worker
// spends on a token.  On 4-byte aligned tables and windows within +-31 a worker is a TEAM of four
// wavefronts (pos_team_bf16_kernel), as in the fp32 kernel: the window's positions are dealt to
// the waves by their place in the token stream, the centre's column is read by one wave and
// handed round in LDS, and the waves' shares of the centre's delta meet in LDS.  Otherwise a
// worker is one wave (pos_chain_bf16_kernel).
#include "w2v_bf16.h"
#include "w2v_internal.h"

namespace w2v {

namespace {

template <int RP>
struct PosChunk16 {
  // (larger chunks cost more registers than a wave has, and a spilled exchange result is waited
  // for at once: 8 columns at dim 300 are slower than 4, 165 against 145 ms per 1M tokens)
  static constexpr int value = RP <= 2 ? 8 : RP <= 6 ? 4 : 3;
};

// Columns a wave of a team gathers at a time: it meets a quarter of the window.
template <int RP>
struct TeamChunk16 {
  static constexpr int value = RP <= 4 ? 3 : 2;
};

// One centre token worked on by one wave alone: window offsets of any reach, in slabs of 64.
// `wnear` holds the word ids at offsets -32..31 of token i (lane l: offset l - 32).
template <int RP, bool ALIGNED, int CH>
__device__ __forceinline__ void chain_token16_solo(int i, int wi, int jlo, int jhi, int wnear,
                                                   int d, const int* __restrict__ W, uint16_t* A,
                                                   uint16_t* B, float lrate, float vexp, int smode,
                                                   uint64_t seed, const HotCols& hot,
                                                   const Shadow& shadow, int lane) {
  uint16_t* const acol = A + (int64_t)wi * d;
  float a[2 * RP], daa[2 * RP];
  load_col16_fresh<RP, ALIGNED>(a, acol, lane, d);
  // (a frequent word's side column is requested here and added once the window's first columns
  // have been requested too: adding it at once would wait for the centre's column first)
  float aside[2 * RP];
  bool aside_pending = wi < hot.n;
  if (aside_pending) side_col_request<RP>(aside, hot.sa + (int64_t)wi * side_stride(d), lane, d);
#pragma unroll
  for (int r = 0; r < 2 * RP; ++r) daa[r] = 0.0f;
  const float ascale = scale_of(wi, vexp, smode);
  bool touched = false, a_written = false;
  const uint32_t akey = sr_key(seed, (uint32_t)i, 0U);
  // (counters of the words that may be rare within the launch are requested where the word is
  // known and looked at where the column is written: looking at once would wait for them before
  // the columns are even asked for)
  const int a_seen = wi >= hot.n ? rare_seen(shadow, wi) : 0x7fffffff;

  const int base0 = min(jlo, -kChainLook);
  for (int base = base0; base <= jhi; base += kWave) {
    // lane l looks at window offset base + l; the offsets -32..31 were fetched beforehand (a
    // window wider than 64 offsets is worked on in slabs, each after the writes of the last)
    if (base != base0) wait_for_own_writes();
    const int j = base + lane;
    int wl = -1;
    if (j >= jlo && j <= jhi && j != 0) wl = base == -kChainLook ? wnear : W[i + j];
    const bool ok = wl >= 0;
    const float sl = ok ? scale_of(wl, vexp, smode) : 0.0f;
    const unsigned long long valid = __ballot(ok);
    const int seen = (ok && wl >= hot.n) ? rare_seen(shadow, wl) : 0x7fffffff;
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
          }
        }
        // the frequent words' side columns: all requested before the first is added
        if (hot.n > 0) {
          float bside[CH][2 * RP];
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (c < nc && wb[c] < hot.n)
              side_col_request<RP>(bside[c], hot.sb + (int64_t)wb[c] * side_stride(d), lane, d);
          }
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            if (c < nc && wb[c] < hot.n) side_col_add<RP>(b[c], bside[c]);
          }
        }
        if (aside_pending) {
          side_col_add<RP>(a, aside);
          aside_pending = false;
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
        // which of the window's words are rare within the launch (plain stores)
        const unsigned long long rare = __ballot(seen <= shadow.rare_max);
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
            } else if ((rare >> src[c]) & 1ull) {
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
          } else if (a_seen <= shadow.rare_max) {
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
      else if (a_seen <= shadow.rare_max)
        store_col16<RP, ALIGNED>(acol, a, daa, lane, d, akey);
      else
        add_col16<RP, ALIGNED>(acol, a, daa, lane, d, akey);
    }
    // the writes of this token are issued before the next token's columns are read
    wait_for_own_writes();
  }
}

// Workers of one wave each, four to a workgroup.
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
  int lb = 0, ub = 0, wnear = -1;
  auto fetch = [&](int64_t t) {
    lb = ub = 0;
    wnear = -1;
    if (t < i_end) {
      lb = LB[t];
      ub = UB[t];
      const int64_t p = t + lane - kChainLook;
      if (p >= 0 && p < n) wnear = W[p];
    }
  };
  fetch(i_begin);
  for (int64_t unit = i_begin; unit < i_end; ++unit) {
    const int i = (int)unit;
    const int wi = read_lane(wnear, kChainLook);
    const int jlo = max(__builtin_amdgcn_readfirstlane(lb), -i);
    const int jhi = min(__builtin_amdgcn_readfirstlane(ub), n - 1 - i);
    const int wnear_now = wnear;
    fetch(unit + 1);
    if (wi < 0) continue;
    chain_token16_solo<RP, ALIGNED, CH>(i, wi, jlo, jhi, wnear_now, d, W, A, B, lrate, vexp, smode,
                                        seed, hot, shadow, lane);
  }
}

// Workers of TW waves each (a workgroup), tables on 4-byte boundaries.
template <int RP, int CH, int TW>
__global__ void __launch_bounds__(TW * kWave)
pos_team_bf16_kernel(int d, int n, int64_t per_chain, const int* __restrict__ W,
                     const int* __restrict__ LB, const int* __restrict__ UB, uint16_t* A,
                     uint16_t* B, float lrate, float vexp, int smode, uint64_t seed, HotCols hot,
                     Shadow shadow_arg) {
  // the centre's column as its owner read it, and each wave's share of the centre's delta
  __shared__ float s_a[2 * RP * kWave];
  __shared__ float s_da[TW][2 * RP * kWave];
  __shared__ int s_hands;   // the team waits for its writes before the next token (see below)
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  if (!launch_is_ordered(shadow_arg, shadow)) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t chain = blockIdx.x;   // a workgroup is a worker
  const int64_t i_begin = chain * per_chain;
  const int64_t i_end = min(i_begin + per_chain, (int64_t)n);

  // Word ids of token t and of its window; the window bounds are requested one token further
  // ahead (those of token t were asked for with token t - 1), so that a token also knows its
  // successor's window without waiting for anything it has just asked for.
  int lb = 0, ub = 0, lbn = 0, ubn = 0, wnear = -1;
  auto fetch = [&](int64_t t) {
    lb = lbn;
    ub = ubn;
    lbn = ubn = 0;
    wnear = -1;
    if (t < i_end) {
      const int64_t p = t + lane - kChainLook;
      if (p >= 0 && p < n) wnear = W[p];
    }
    if (t + 1 < i_end) {
      lbn = LB[t + 1];
      ubn = UB[t + 1];
    }
  };
  if (i_begin < i_end) {
    lbn = LB[i_begin];
    ubn = UB[i_begin];
  }
  fetch(i_begin);
  for (int64_t unit = i_begin; unit < i_end; ++unit) {
    const int i = (int)unit;
    const int wi = read_lane(wnear, kChainLook);
    const int jlo = max(__builtin_amdgcn_readfirstlane(lb), -i);
    const int jhi = min(__builtin_amdgcn_readfirstlane(ub), n - 1 - i);
    const int wnear_now = wnear;
    const int nlb = __builtin_amdgcn_readfirstlane(lbn);   // the next token's bounds
    const int nub = __builtin_amdgcn_readfirstlane(ubn);
    fetch(unit + 1);
    if (wi < 0) continue;
    const int oa = team_wave(wi, TW);
    if (jlo < -kChainLook || jhi >= kChainLook) {
      // a window beyond the offsets a wave's lanes cover: the centre's owner does the token alone
      // and waits for its writes to be performed before the team goes on (the next tokens read
      // the same columns from other waves)
      if (wave == oa) {
        chain_token16_solo<RP, true, CH>(i, wi, jlo, jhi, wnear_now, d, W, A, B, lrate, vexp,
                                         smode, seed, hot, shadow, lane);
        __builtin_amdgcn_s_waitcnt(0);
      }
      __syncthreads();
      continue;
    }
    // lane l looks at window offset l - 32 (every wave computes the same picture of the window)
    const int j = lane - kChainLook;
    int wl = -1;
    if (j >= jlo && j <= jhi && j != 0) wl = wnear_now;
    const bool ok = wl >= 0;
    const unsigned long long valid = __ballot(ok);
    if (valid == 0ull) continue;
    const float sl = ok ? scale_of(wl, vexp, smode) : 0.0f;
    // The counters of the words that may be rare within the launch (plain stores) are requested
    // here and looked at where a column is written: looking at once would wait for them before
    // the columns are even asked for.
    const int seen = (ok && wl >= hot.n) ? rare_seen(shadow, wl) : 0x7fffffff;
    const int a_seen = wi >= hot.n ? rare_seen(shadow, wi) : 0x7fffffff;
    // A window position belongs to the wave that its place in the token stream selects; a word
    // that stands at several positions of the window belongs, with all of them, to the wave of
    // its first position, and occurrence number r of it is worked on in round r.
    int occ = 0, first = lane;
    {
      unsigned long long m = valid;
      while (m != 0ull) {
        const int l = __builtin_ctzll(m);
        m &= m - 1ull;
        if (l < lane && read_lane(wl, l) == wl) {
          if (occ == 0) first = l;
          ++occ;
        }
      }
    }
    const bool mine = ok && ((i + first) & (TW - 1)) == wave;
    const bool repeats = __ballot(ok && occ > 0) != 0ull;
    uint16_t* const acol = A + (int64_t)wi * d;
    float a[2 * RP], daa[2 * RP];
    float aside[2 * RP];
    if (wave == oa) {
      load_col16_fresh<RP, true>(a, acol, lane, d);
      // (a frequent word's side column: requested here, added after this wave's first B columns
      // have been requested too)
      if (wi < hot.n) side_col_request<RP>(aside, hot.sa + (int64_t)wi * side_stride(d), lane, d);
    }
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) daa[r] = 0.0f;
    const float ascale = scale_of(wi, vexp, smode);

    int src[CH], wb[CH];
    int nc = 0;
    float b[CH][2 * RP];
    float bside[CH][2 * RP];   // the side columns of the chunk's frequent words
    auto gather = [&](unsigned long long& mask) {
      nc = 0;
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
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        wb[c] = -1;
        if (c < nc) {
          wb[c] = read_lane(wl, src[c]);
          load_col16_fresh<RP, true>(b[c], B + (int64_t)wb[c] * d, lane, d);
        }
      }
      // the frequent words' side columns: all requested before anything is added (one round
      // trip for the chunk, not one per column)
      if (hot.n > 0) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (c < nc && wb[c] < hot.n)
            side_col_request<RP>(bside[c], hot.sb + (int64_t)wb[c] * side_stride(d), lane, d);
        }
      }
    };
    auto add_sides = [&]() {
      if (hot.n <= 0) return;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (c < nc && wb[c] < hot.n) side_col_add<RP>(b[c], bside[c]);
      }
    };
    auto update = [&]() {
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
      const unsigned long long rare = __ballot(seen <= shadow.rare_max);
      float gbs[CH];
      uint32_t guess[CH][RP], found[CH][RP];
      bool cas[CH];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        cas[c] = false;
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
          const uint32_t key = sr_key(seed, (uint32_t)i, (uint32_t)(src[c] - kChainLook));
          if (wb[c] < hot.n) {
            write_side_main<RP>(hot.sb, wb[c], db, lane, d);
          } else if ((rare >> src[c]) & 1ull) {
            store_col16<RP, true>(bcol, b[c], db, lane, d, key);
          } else {
            cas[c] = true;
            cas_first<RP>(bcol, b[c], db, lane, d, key, guess[c], found[c]);
          }
        }
      }
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (cas[c])
          cas_rest_axpy<RP>(B + (int64_t)wb[c] * d, gbs[c], a, lane, d,
                            sr_key(seed, (uint32_t)i, (uint32_t)(src[c] - kChainLook)), guess[c],
                            found[c]);
      }
    };

    // the first columns of this wave are requested before the centre's column is handed round
    unsigned long long mask = __ballot(mine && occ == 0);
    gather(mask);
    // Whether a column passes to another wave with the next token (window_hands_over): worked
    // out by one wave that is not the centre's, which would otherwise only wait at the barrier
    // for the centre's column, from what the token knew when it began, and handed round in LDS.
    if (wave == ((oa + 1) & (TW - 1))) {
      bool hands = false;
      if (!repeats && unit + 1 < i_end) {
        const int wn = read_lane(wnear_now, kChainLook + 1);
        const int nlo = max(nlb, -(i + 1));
        const int nhi = min(nub, n - 2 - i);
        hands = wn < 0 || nlo < -kChainLook || nhi >= kChainLook - 1 ||
                window_hands_over(wl, wnear_now, lane, nlo, nhi, TW);
      }
      if (lane == 0) s_hands = hands ? 1 : 0;
    }
    if (wave == oa) {
      if (wi < hot.n) side_col_add<RP>(a, aside);
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) s_a[r * kWave + lane] = a[r];
    }
    add_sides();
    __syncthreads();
    if (wave != oa) {
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) a[r] = s_a[r * kWave + lane];
    }
    if (nc > 0) update();
    while (mask != 0ull) {
      gather(mask);
      add_sides();
      update();
    }
    for (int round = 1;; ++round) {
      mask = __ballot(mine && occ == round);
      if (mask == 0ull) break;
      wait_for_own_writes();
      while (mask != 0ull) {
        gather(mask);
        add_sides();
        update();
      }
    }
    // the waves' shares of the centre's delta meet at the centre's owner
#pragma unroll
    for (int r = 0; r < 2 * RP; ++r) s_da[wave][r * kWave + lane] = daa[r];
    // Where the next reader of a column may be another wave (a word at several positions whose
    // first one leaves the window; a word that the next token's window meets again at a new
    // position, window_hands_over; any word after a token that is skipped), this wave's writes
    // have been performed before the team goes on
    if (repeats || s_hands != 0) __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (wave == oa) {
#pragma unroll
      for (int r = 0; r < 2 * RP; ++r) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < TW; ++w) t += s_da[w][r * kWave + lane];
        daa[r] = t;
      }
      const uint32_t akey = sr_key(seed, (uint32_t)i, 0U);
      if (wi < hot.n)
        write_side_main<RP>(hot.sa, wi, daa, lane, d);
      else if (a_seen <= shadow.rare_max)
        store_col16<RP, true>(acol, a, daa, lane, d, akey);
      else
        add_col16<RP, true>(acol, a, daa, lane, d, akey);
    }
  }
}

template <int RP, bool ALIGNED>
hipError_t launch_chain(hipStream_t stream, int d, int n, int shift, const int* W, const int* LB,
                        const int* UB, uint16_t* A, uint16_t* B, float lrate, float vexp,
                        uint64_t seed, HotCols hot, Shadow shadow) {
  const bool team = ALIGNED && shift < kChainLook;
  const int64_t chains = ordered_pos_chains(n, shift, team ? kPosTeamsBf16 : kPosChainsBf16);
  const int64_t per_chain = ((int64_t)n + chains - 1) / chains;   // workers beyond: empty range
  // words that are rare within the launch are written back with plain stores (store_col16)
  hipError_t err = prepare_rare_words(stream, W, n, nullptr, 0, 0x7fffffff, n, chains, &shadow,
                                      kRareCapOrderedBf16);
  if (err != hipSuccess) return err;
  if (team) {
    hipLaunchKernelGGL((pos_team_bf16_kernel<RP, TeamChunk16<RP>::value, kTeamWaves>),
                       dim3((unsigned)chains), dim3(kTeamWaves * kWave), 0, stream, d, n,
                       per_chain, W, LB, UB, A, B, lrate, vexp, scale_mode(vexp), seed, hot,
                       shadow);
  } else {
    hipLaunchKernelGGL((pos_chain_bf16_kernel<RP, ALIGNED, PosChunk16<RP>::value>),
                       dim3((unsigned)((chains + kWavesPerBlock - 1) / kWavesPerBlock)),
                       dim3(kBlock), 0, stream, d, n, per_chain, W, LB, UB, A, B, lrate, vexp,
                       scale_mode(vexp), seed, hot, shadow);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_pos_chain_bf16(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                                 const int* LB, const int* UB, uint16_t* A, uint16_t* B,
                                 float lrate, float vexp, uint64_t seed, HotCols hot,
                                 const Shadow& shadow, bool aligned) {
  const int rp = (nrows + 127) / 128;
  if (aligned) {
#define W2V_CALL(RP_)                                                                          \
  return launch_chain<RP_, true>(stream, nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, seed, \
                                 hot, shadow)
    W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
  }
#define W2V_CALL(RP_)                                                                           \
  return launch_chain<RP_, false>(stream, nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, seed, \
                                  hot, shadow)
  W2V_PAIR_ROUNDS_SWITCH(rp, W2V_CALL);
#undef W2V_CALL
}

}  // namespace w2v
