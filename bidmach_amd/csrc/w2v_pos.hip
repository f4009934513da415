// Positive (centre, context) pass of skip-gram negative sampling, and its forward-only twin.
//
// Semantics follow the reference CPU path, jni/src/BIDMach_CPUMACH.c:10-78 (word2vecPos) and
// :368-427 (word2vecEvalPos): for each centre token i with W[i] >= 0 and each offset
// j in [LB[i], UB[i]], j != 0, 0 <= i+j < ncols, W[i+j] >= 0:
//   s = A[:,W[i]] . B[:,W[i+j]];  g = lrate * (1 - sigmoid(s))
//   B[:,W[i+j]] += bscale * g * A[:,W[i]]
//   A[:,W[i]]   += ascale * g * B[:,W[i+j]]    (accumulated over the window, scattered once)
//
// Three kernels.
//
// pos_kernel (the update when a tile does not fit in LDS) and pos_eval_kernel (forward-only
// scoring): one wavefront owns one centre token.  Its A column stays in registers for the whole
// window; context columns are gathered CH at a time (all loads of a chunk are issued before the
// first dot product, so a wave keeps CH columns in flight), dot products are reduced with DPP row
// rotations, and the CH pre-activations are parked in lanes 0..CH-1 so that the sigmoid (a double
// exp) is evaluated once per chunk instead of once per pair.
//
// pos_tile_kernel (the update): float atomics are the scarce resource on this GPU (the L2
// retires about one dword atomic per clock per channel, roughly 1.1 TB/s of payload for the
// whole chip, whatever the footprint), so the update is organised to issue as few of them as
// the data allows.  A workgroup owns a tile of T consecutive tokens.  It stages the A columns of
// its T centres and the B columns of the T + 2*Sh positions its windows can reach in LDS
// (each column is gathered from HBM once per tile instead of once per pair), then
//   phase 1, one wave per centre: dot products against the staged B columns, sigmoid, the
//     centre's delta accumulated in registers and scattered with one column of atomics; every
//     g is left in an LDS table G[centre][offset];
//   phase 2, one wave per staged position: the sum over the tile's centres of g * A column,
//     scattered with one column of atomics.
// A token therefore costs about (2T + 2Sh)/T columns of atomics instead of 1 + (pairs).
// All dot products of a tile use the columns as staged (a tile is a small synchronous batch);
// between tiles the updates are Hogwild, as between the reference's threads.
#include <algorithm>
#include <cstdlib>
#include <atomic>
#include <type_traits>

#include "w2v_device.h"
#include "w2v_internal.h"

namespace w2v {

template <int R, int CH, bool TRAIN>
__global__ void __launch_bounds__(kBlock)
pos_kernel(int d, int ncols, int64_t per_xcd, const int* __restrict__ W,
           const int* __restrict__ LB, const int* __restrict__ UB, float* A, float* B, float lrate,
           float vexp, int smode, double floorv, double* __restrict__ partials,
           Shadow shadow_arg) {
  // a launch full of frequent words is done by pos_chain_kernel (launch_is_ordered)
  if (TRAIN && shadow_arg.ordered != 0 &&
      launch_is_ordered(shadow_arg, resolve_hot_mode(shadow_arg)))
    return;
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

// Forward-only scoring, persistent form of pos_kernel: workgroup b walks a contiguous range of
// centres (ranges are laid out so that each XCD's workgroups cover one contiguous stretch of the
// minibatch and neighbouring centres' shared context columns meet in one L2), one centre per wave
// at a time, and a wave fetches word id and window bounds of its next centre while it scores the
// current one.
template <int R, int CH>
__global__ void __launch_bounds__(kBlock)
pos_eval_kernel(int d, int ncols, int64_t units_per_wg, const int* __restrict__ W,
                const int* __restrict__ LB, const int* __restrict__ UB,
                const float* __restrict__ A, const float* __restrict__ B, double floorv,
                double* __restrict__ partials) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t per_xcd = gridDim.x / kXcds;   // the grid is a multiple of the XCD count
  const int64_t range = xcd_contiguous_block(per_xcd);
  const int64_t u_begin = range * units_per_wg;
  const int64_t u_end = min(u_begin + units_per_wg, (int64_t)ncols);
  double lsum = 0.0;

  int64_t unit = u_begin + wave;
  int wi = -1, lb = 0, ub = 0;
  if (unit < u_end) {
    wi = W[unit];
    lb = LB[unit];
    ub = UB[unit];
  }
  for (; unit < u_end; unit += kWavesPerBlock) {
    const int i = (int)unit;
    const int wi_now = __builtin_amdgcn_readfirstlane(wi);
    const int jlo = max(__builtin_amdgcn_readfirstlane(lb), -i);
    const int jhi = min(__builtin_amdgcn_readfirstlane(ub), ncols - 1 - i);
    {
      const int64_t next = unit + kWavesPerBlock;
      wi = -1;
      if (next < u_end) {
        wi = W[next];
        lb = LB[next];
        ub = UB[next];
      }
    }
    if (wi_now < 0) continue;
    float a[R];
    load_col<R>(a, A + (int64_t)wi_now * d, lane, d);
    for (int base = jlo; base <= jhi; base += kWave) {
      const int j = base + lane;
      int wl = -1;
      if (j <= jhi && j != 0) wl = W[i + j];
      unsigned long long mask = __ballot(wl >= 0);
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
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (c < n) load_col<R>(b[c], B + (int64_t)read_lane(wl, src[c]) * d, lane, d);
        }
        float pre = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (c < n) {
            const float s = wave_sum(dot_partial<R>(a, b[c]));
            pre = (lane == c) ? s : pre;
          }
        }
        if (lane < n) lsum += log(fmax((double)sat_sigmoid(pre), floorv));
      }
    }
  }
  block_store_partial(wave_sum_f64(lsum), partials);
}

// Ordered form of the update (launch_is_ordered, w2v_device.h): the token-by-token order of the
// reference's CPU loop (BIDMach_CPUMACH.c:26-68).  A worker is one of a few dozen, like a thread
// of the reference (:21-24): it walks a contiguous range of centre tokens one after the other;
// for each it reads the centre's A column and the window's B columns afresh (device-scope loads,
// so neither this CU's L1 nor this XCD's L2 can hand back a value from before another worker's
// update), adds every B delta to the table at once and the A delta after the window, and only
// then reads for the next token, whose window shares all but two positions with this one.  (A
// tile of adjacent tokens that computes from one snapshot of its columns misses exactly those
// updates: 16 tokens per snapshot move the held-out loss of a raw Zipf stream by 5 %, 2 tokens
// by 1.7 %.)
// The ids of the next token and of its window (offsets -32..31) are fetched while the current
// token is worked on.
//
// How many workers there may be is set by the held-out loss (every token in flight is a token
// whose updates the others do not see), so what is left to make the pass faster is the time a
// worker spends on a token: a random 1.2 KB column takes about 2 us to arrive, and a wave issues
// the float atomics of one column in about 0.35 us.  A worker is therefore a TEAM of TW
// wavefronts (a workgroup): the window's positions are dealt to the waves by their place in the
// token stream, each wave gathers, dots and updates the B columns of its positions, the centre's
// column is read by the wave that the centre's word hashes to (team_wave) and handed round in
// LDS, and the waves' shares of the centre's delta meet in LDS and are added by that same wave.
// A position stays with one wave while it moves through consecutive windows, and requests of one
// wave to one address are performed in order (requests of different waves need not be); where a
// column goes from one wave to another (a word at several positions, window_hands_over) the
// team waits for its adds' acknowledgements first, so one team reproduces the sequential result.

// One centre token worked on by one wave alone: window offsets of any reach, in slabs of 64.
// `wnear` holds the word ids at offsets -32..31 of token i (lane l: offset l - 32).
// `tables` places a word's column and, for a sliced model, says which pairs are trained and
// which columns are written (BIDMach_CPUMACH.c:137-157).
template <int R, int CH, class Tables>
__device__ __forceinline__ void chain_token_solo(int i, int wi, int jlo, int jhi, int wnear,
                                                 const ColRef& pa, int d, int ncols,
                                                 const int* __restrict__ W, const Tables& tables,
                                                 float lrate, float vexp, int smode,
                                                 const Shadow& shadow, int64_t chain, int lane) {
  float a[R];
  load_col_ordered<R>(a, pa, shadow, 1, chain, lane, d);
  float daa[R];
  zero_col<R>(daa);
  const float ascale = scale_of(wi, vexp, smode);
  bool touched = false;

  const int base0 = min(jlo, -kChainLook);
  for (int base = base0; base <= jhi; base += kWave) {
    // lane l looks at window offset base + l; the offsets -32..31 were fetched beforehand.
    // (A window wider than 64 offsets is worked on in slabs, each after the adds of the last.)
    if (base != base0) wait_for_own_writes();
    const int j = base + lane;
    int wl = -1;
    if (j >= jlo && j <= jhi && j != 0) wl = base == -kChainLook ? wnear : W[i + j];
    const int fl = tables.b(wl, d).flags;
    const bool ok = fl != 0 && tables.trained(pa.flags, fl);
    const float sl = ok ? scale_of(wl, vexp, smode) : 0.0f;
    const unsigned long long valid = __ballot(ok);
    const unsigned long long wmask = __ballot(ok && tables.written(fl));
    // A word that stands at several offsets of the window is updated once per offset, and the
    // reference reads it again each time (:43-46 after :60): occurrence number r of a word is
    // worked on in round r, after the adds of round r - 1.  Pairs of different words commute, so
    // the rounds change nothing else.
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
            rb[c] = tables.b(read_lane(wl, src[c]), d);
            load_col_ordered<R>(b[c], rb[c], shadow, 0, chain, lane, d);
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
        const float gl = lrate * (1.0f - sat_sigmoid_fast(pre));
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (c < n) {
            const float g = read_lane(gl, c);
            const float bs = read_lane(sl, src[c]);
            axpy<R>(daa, ascale * g, b[c]);
            if ((wmask >> src[c]) & 1ull) {
              float db[R];
#pragma unroll
              for (int r = 0; r < R; ++r) db[r] = (bs * g) * a[r];
              add_col_ordered<R>(rb[c], shadow, 0, chain, db, lane, d);
            }
          }
        }
        touched = true;
      }
    }
  }
  if (touched && tables.written(pa.flags)) add_col_ordered<R>(pa, shadow, 1, chain, daa, lane, d);
}

// Columns a wave of a team gathers at a time: a team's wave meets a fraction of the window.
template <int R>
struct TeamChunk {
  static constexpr int value = R <= 8 ? 6 : R <= 12 ? 4 : 3;
};

template <int R, int CH, int TW, class Tables>
__global__ void __launch_bounds__(TW * kWave)
pos_chain_kernel(int d, int ncols, int64_t per_chain, const int* __restrict__ W,
                 const int* __restrict__ LB, const int* __restrict__ UB, Tables tables,
                 float lrate, float vexp, int smode, Shadow shadow_arg) {
  // the centre's column as its owner read it, and each wave's share of the centre's delta
  __shared__ float s_a[TW > 1 ? R * kWave : 1];
  __shared__ float s_da[TW > 1 ? TW : 1][TW > 1 ? R * kWave : 1];
  __shared__ int s_hands;   // the team waits for its adds before the next token (see below)
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  if (!launch_is_ordered(shadow_arg, shadow)) return;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t chain = blockIdx.x;   // a workgroup is a worker
  const int64_t i_begin = chain * per_chain;
  const int64_t i_end = min(i_begin + per_chain, (int64_t)ncols);

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
      if (p >= 0 && p < ncols) wnear = W[p];
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
    const int jhi = min(__builtin_amdgcn_readfirstlane(ub), ncols - 1 - i);
    const int wnear_now = wnear;
    const int nlb = __builtin_amdgcn_readfirstlane(lbn);   // the next token's bounds
    const int nub = __builtin_amdgcn_readfirstlane(ubn);
    fetch(unit + 1);
    const ColRef pa = tables.a(wi, d);
    if (pa.flags == 0) continue;
    if (TW == 1) {
      chain_token_solo<R, CH, Tables>(i, wi, jlo, jhi, wnear_now, pa, d, ncols, W, tables, lrate,
                                      vexp, smode, shadow, chain, lane);
      continue;
    }
    const int oa = team_wave(wi, TW);
    if (jlo < -kChainLook || jhi >= kChainLook) {
      // a window beyond the offsets a wave's lanes cover: the centre's owner does the token alone
      // and waits for its adds to be performed before the team goes on (the next tokens read the
      // same columns from other waves)
      if (wave == oa) {
        chain_token_solo<R, CH, Tables>(i, wi, jlo, jhi, wnear_now, pa, d, ncols, W, tables, lrate,
                                        vexp, smode, shadow, chain, lane);
        __builtin_amdgcn_s_waitcnt(0);
      }
      __syncthreads();
      continue;
    }
    // lane l looks at window offset l - 32 (every wave computes the same picture of the window)
    const int j = lane - kChainLook;
    int wl = -1;
    if (j >= jlo && j <= jhi && j != 0) wl = wnear_now;
    const int fl = tables.b(wl, d).flags;
    const bool ok = fl != 0 && tables.trained(pa.flags, fl);
    const unsigned long long valid = __ballot(ok);
    if (valid == 0ull) continue;
    const unsigned long long wmask = __ballot(ok && tables.written(fl));
    const float sl = ok ? scale_of(wl, vexp, smode) : 0.0f;
    // A window position belongs to the wave that its place in the token stream selects (so the
    // same position stays with the same wave while it moves through the windows of consecutive
    // tokens); a word that stands at several positions of the window belongs, with all of them,
    // to the wave of its first position, and occurrence number r of it is worked on in round r
    // (see chain_token_solo).
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
    float a[R];
    if (wave == oa) load_col_ordered<R>(a, pa, shadow, 1, chain, lane, d);
    float daa[R];
    zero_col<R>(daa);
    const float ascale = scale_of(wi, vexp, smode);

    int src[CH];
    int n = 0;
    float b[CH][R];
    ColRef rb[CH];
    auto gather = [&](unsigned long long& mask) {
      n = 0;
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
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (c < n) {
          rb[c] = tables.b(read_lane(wl, src[c]), d);
          load_col_ordered<R>(b[c], rb[c], shadow, 0, chain, lane, d);
        }
      }
    };
    auto update = [&]() {
      float pre = 0.0f;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (c < n) {
          const float s = wave_sum(dot_partial<R>(a, b[c]));
          pre = (lane == c) ? s : pre;
        }
      }
      const float gl = lrate * (1.0f - sat_sigmoid_fast(pre));
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (c < n) {
          const float g = read_lane(gl, c);
          const float bs = read_lane(sl, src[c]);
          axpy<R>(daa, ascale * g, b[c]);
          if ((wmask >> src[c]) & 1ull) {
            float db[R];
#pragma unroll
            for (int r = 0; r < R; ++r) db[r] = (bs * g) * a[r];
            add_col_ordered<R>(rb[c], shadow, 0, chain, db, lane, d);
          }
        }
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
        const int nhi = min(nub, ncols - 2 - i);
        hands = tables.a(wn, d).flags == 0 || nlo < -kChainLook || nhi >= kChainLook - 1 ||
                window_hands_over(wl, wnear_now, lane, nlo, nhi, TW);
      }
      if (lane == 0) s_hands = hands ? 1 : 0;
    }
    if (wave == oa) {
#pragma unroll
      for (int r = 0; r < R; ++r) s_a[r * kWave + lane] = a[r];
    }
    __syncthreads();
    if (wave != oa) {
#pragma unroll
      for (int r = 0; r < R; ++r) a[r] = s_a[r * kWave + lane];
    }
    if (n > 0) update();
    while (mask != 0ull) {
      gather(mask);
      update();
    }
    for (int round = 1;; ++round) {
      mask = __ballot(mine && occ == round);
      if (mask == 0ull) break;
      wait_for_own_writes();
      while (mask != 0ull) {
        gather(mask);
        update();
      }
    }
    // the waves' shares of the centre's delta meet at the centre's owner
#pragma unroll
    for (int r = 0; r < R; ++r) s_da[wave][r * kWave + lane] = daa[r];
    // The next reader of a word that stands at several positions may be another wave (when its
    // first position leaves the window), and so may the reader of a word that the next token's
    // window meets again at a new position (window_hands_over), or of any word after a token that
    // is skipped: then this wave's adds have been performed before the team goes on
    if (repeats || s_hands != 0) __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (wave == oa && tables.written(pa.flags)) {
      zero_col<R>(daa);
#pragma unroll
      for (int w = 0; w < TW; ++w) {
#pragma unroll
        for (int r = 0; r < R; ++r) daa[r] += s_da[w][r * kWave + lane];
      }
      add_col_ordered<R>(pa, shadow, 1, chain, daa, lane, d);
    }
  }
}

constexpr int64_t kMinEvalCentresPerWg = 256;

constexpr int kTileWaves = 8;
constexpr int kTileThreads = kTileWaves * kWave;
constexpr int kMaxHalo = 31;       // 2*Sh + 1 window offsets must fit in the 64 lanes of a wave
constexpr int kMinTilesPerWg = 64; // a workgroup walks at least this many consecutive tiles
constexpr int kMinTilesPerWgWide = 4;  // the same for a launch without hot words

// LDS layout of a workgroup:
//   a_t[T][dp] | b_t[T + 2*Sh][dp] | G[T][2*Sh + 1] | wt[T + 2*Sh] | ft[T + 2*Sh]
// with dp = R*64 (columns zero-padded so that LDS reads need no bounds test).  wt holds the word
// id of a staged position (-1 if the word is skipped), ft its residency flags.
__host__ __device__ inline size_t tile_lds_bytes(int R, int T, int Sh) {
  const size_t dp = (size_t)R * kWave;
  return ((size_t)T * dp + (size_t)(T + 2 * Sh) * dp + (size_t)T * (2 * Sh + 1) +
          2 * (size_t)(T + 2 * Sh)) * 4;
}

// Two buffers of 2*Sh columns for the B deltas a tile hands to the next one (see the kernel).
__host__ __device__ inline size_t tile_carry_bytes(int R, int Sh) {
  return (size_t)2 * (2 * Sh) * R * kWave * 4;
}

// `tables` is PlainTables (word2vecPos) or SlicedTables (word2vecPosSlice): it places a word's
// column and says which pairs are trained and which columns are written.
// Up to R = 7 two workgroups fit in a CU's LDS, which needs four waves per SIMD: the register
// budget is held to that.
template <int R, class Tables>
__global__ void __launch_bounds__(kTileThreads, (R <= 7 ? 4 : 2))
pos_tile_kernel(int d, int ncols, int T, int Sh, int carry, int64_t ntiles,
                int64_t tiles_per_wg_hot, int64_t tiles_per_wg_wide,
                const int* __restrict__ W, const int* __restrict__ LB,
                const int* __restrict__ UB, Tables tables, float lrate, float vexp, int smode,
                Shadow shadow_arg) {
  extern __shared__ float lds[];
  const Shadow shadow = resolve_hot_mode(shadow_arg);
  constexpr int dp = R * kWave;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int gw = 2 * Sh + 1;
  float* const a_t = lds;
  float* const b_t = a_t + (size_t)T * dp;
  float* const G = b_t + (size_t)(T + 2 * Sh) * dp;
  int* const wt = reinterpret_cast<int*>(G + (size_t)T * gw);
  int* const ft = wt + (T + 2 * Sh);
  // Consecutive tiles of a workgroup overlap in 2*Sh staged positions (the last Sh centres of a
  // tile and its trailing halo are the leading halo and the first Sh centres of the next).  With
  // `carry` a tile does not scatter the B deltas of those positions but leaves them here, and the
  // next tile adds its own share and scatters once: a position then costs one column of atomics
  // instead of two.  Two buffers, because the waves that read the deltas handed in and the waves
  // that write the deltas handed on run in the same phase.
  float* const pend = reinterpret_cast<float*>(ft + (T + 2 * Sh));
  const int slot = blockIdx.x;  // picks the shadow copy this workgroup writes to

  if (launch_is_ordered(shadow_arg, shadow)) return;   // pos_chain_kernel does this launch
  const bool cold = launch_is_cold(shadow_arg, shadow);
  const int64_t tiles_per_wg = cold ? tiles_per_wg_wide : tiles_per_wg_hot;
  // Measured: handing deltas on pays on launches without hot words (6 % on a subsampled stream),
  // where many staged positions are empty and the atomics saved are a larger part of a tile's
  // work; on a raw stream the longer second phase costs more than the atomics saved (7 %).
  const bool carrying = carry != 0 && cold;
  const int64_t tile_begin = (int64_t)blockIdx.x * tiles_per_wg;
  const int64_t tile_end = min(tile_begin + tiles_per_wg, ntiles);

  for (int64_t tile = tile_begin; tile < tile_end; ++tile) {
    const int lo = (int)(tile * T);
    const int hi = min(lo + T, ncols);          // centres [lo, hi)
    const int hlo = max(lo - Sh, 0);
    const int hhi = min(hi + Sh, ncols);        // staged positions [hlo, hhi)
    const int nh = hhi - hlo;
    const int nc = hi - lo;
    // deltas handed in cover staged positions [0, 2*Sh); deltas handed on cover [c_out, nh)
    const bool carry_in = carrying && tile > tile_begin;
    const bool carry_out = carrying && tile + 1 < tile_end;
    const int c_out = hi - Sh - hlo;
    const float* const pend_in = pend + (size_t)(tile & 1) * (2 * Sh) * dp;
    float* const pend_out = pend + (size_t)((tile + 1) & 1) * (2 * Sh) * dp;

    // ---- stage: word ids, B columns of every staged position, A columns of the centres.
    //      Two columns per wave are in flight at a time.
    for (int c0 = wave; c0 < nh; c0 += 2 * kTileWaves) {
      const int c1 = c0 + kTileWaves;
      const int w0 = W[hlo + c0];
      const int w1 = c1 < nh ? W[hlo + c1] : -1;
      const ColRef r0 = tables.b(w0, d);
      const ColRef r1 = tables.b(w1, d);
      float x0[R], x1[R];
      if (r0.flags != 0) load_col_ref<R>(x0, r0, shadow, 0, lane, d);
      if (r1.flags != 0) load_col_ref<R>(x1, r1, shadow, 0, lane, d);
      if (lane == 0) {
        wt[c0] = r0.flags != 0 ? w0 : -1;
        ft[c0] = r0.flags;
        if (c1 < nh) {
          wt[c1] = r1.flags != 0 ? w1 : -1;
          ft[c1] = r1.flags;
        }
      }
      // what the previous tile computed for this position but has not written to the table yet
      const bool in0 = carry_in && c0 < 2 * Sh && tables.written(r0.flags);
      const bool in1 = carry_in && c1 < 2 * Sh && tables.written(r1.flags);
      if (r0.flags != 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
          b_t[(size_t)c0 * dp + r * kWave + lane] =
              x0[r] + (in0 ? pend_in[(size_t)c0 * dp + r * kWave + lane] : 0.0f);
      }
      if (r1.flags != 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
          b_t[(size_t)c1 * dp + r * kWave + lane] =
              x1[r] + (in1 ? pend_in[(size_t)c1 * dp + r * kWave + lane] : 0.0f);
      }
    }
    for (int c0 = wave; c0 < nc; c0 += 2 * kTileWaves) {
      const int c1 = c0 + kTileWaves;
      const int w0 = W[lo + c0];
      const int w1 = c1 < nc ? W[lo + c1] : -1;
      const ColRef r0 = tables.a(w0, d);
      const ColRef r1 = tables.a(w1, d);
      float x0[R], x1[R];
      if (r0.flags != 0) load_col_ref<R>(x0, r0, shadow, 1, lane, d);
      if (r1.flags != 0) load_col_ref<R>(x1, r1, shadow, 1, lane, d);
      if (r0.flags != 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) a_t[(size_t)c0 * dp + r * kWave + lane] = x0[r];
      }
      if (r1.flags != 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) a_t[(size_t)c1 * dp + r * kWave + lane] = x1[r];
      }
    }
    for (int k = threadIdx.x; k < nc * gw; k += kTileThreads) G[k] = 0.0f;
    __syncthreads();

    // ---- phase 1: one wave per centre ----
    for (int ci = wave; ci < nc; ci += kTileWaves) {
      const int i = lo + ci;
      const int wi = wt[i - hlo];
      if (wi < 0) continue;
      const int fi = Tables::kSliced ? ft[i - hlo] : kMine;
      // ticket for the write to this centre's A column at the end of the iteration, taken now
      const ColRef ra = tables.a(wi, d);
      const unsigned tka = lane == 0 ? hot_ticket(shadow, 1, slot, ra.hot) : 0u;
      const int jlo = max(LB[i], -i);
      const int jhi = min(UB[i], ncols - 1 - i);
      float a[R];
#pragma unroll
      for (int r = 0; r < R; ++r) a[r] = a_t[(size_t)ci * dp + r * kWave + lane];
      float daa[R];
      zero_col<R>(daa);
      const float ascale = scale_of(wi, vexp, smode);
      bool touched = false;

      // Staged part of the window: lane l stands for offset j = l - Sh.
      {
        const int j = lane - Sh;
        int wl = -1;
        if (lane < gw && j != 0 && j >= jlo && j <= jhi) wl = wt[i + j - hlo];
        if (Tables::kSliced) {
          if (wl >= 0 && !tables.trained(fi, ft[i + j - hlo])) wl = -1;
        }
        const unsigned long long valid = __ballot(wl >= 0);
        if (valid != 0ull) {
          float pre = 0.0f;
          unsigned long long mask = valid;
          while (mask != 0ull) {
            const int l = __builtin_ctzll(mask);
            mask &= mask - 1ull;
            const float* bcol = b_t + (size_t)(i + l - Sh - hlo) * dp + lane;
            float s = 0.0f;
#pragma unroll
            for (int r = 0; r < R; ++r) s = fmaf(a[r], bcol[r * kWave], s);
            s = wave_sum(s);
            pre = (lane == l) ? s : pre;
          }
          const float gl = lrate * (1.0f - sat_sigmoid(pre));
          if (wl >= 0) G[ci * gw + lane] = gl;
          mask = valid;
          while (mask != 0ull) {
            const int l = __builtin_ctzll(mask);
            mask &= mask - 1ull;
            const float ag = ascale * read_lane(gl, l);
            const float* bcol = b_t + (size_t)(i + l - Sh - hlo) * dp + lane;
#pragma unroll
            for (int r = 0; r < R; ++r) daa[r] = fmaf(ag, bcol[r * kWave], daa[r]);
          }
          touched = true;
        }
      }

      // Offsets beyond the staged halo (only when LB/UB exceed the caller's `shift`): one
      // context at a time, gathered from memory and scattered at once.
      for (int j = jlo; j <= jhi; ++j) {
        if (j >= -Sh && j <= Sh) {
          j = Sh;  // skip the staged range
          continue;
        }
        const int wb = W[i + j];
        const ColRef rb = tables.b(wb, d);
        if (rb.flags == 0 || !tables.trained(fi, rb.flags)) continue;
        float b[R];
        load_col_ref<R>(b, rb, shadow, 0, lane, d);
        const float s = wave_sum(dot_partial<R>(a, b));
        const float g = lrate * (1.0f - sat_sigmoid(s));
        axpy<R>(daa, ascale * g, b);
        if (tables.written(rb.flags))
          scatter_axpy_ref<R>(rb, shadow, 0, slot, scale_of(wb, vexp, smode) * g, a,
                              lane, d);
        touched = true;
      }
      if (touched && tables.written(fi))
        scatter_add_ref<R>(ra, shadow, 1, slot, daa, lane, d,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)tka));
    }
    __syncthreads();

    // ---- phase 2: one wave per staged position ----
    for (int c = wave; c < nh; c += kTileWaves) {
      const int wp = wt[c];
      if (wp < 0) continue;
      if (Tables::kSliced) {
        if (!tables.written(ft[c])) continue;
      }
      const int p = hlo + c;
      const bool handed_in = carry_in && c < 2 * Sh;
      const bool hand_on = carry_out && c >= c_out;
      // lane l looks at centre i = p - Sh + l; its g for this position sits at offset p - i
      const int i = p - Sh + lane;
      float gl = 0.0f;
      if (lane < gw && i >= lo && i < hi && i != p) gl = G[(i - lo) * gw + (p - i + Sh)];
      unsigned long long mask = __ballot(gl != 0.0f);
      if (mask == 0ull && !handed_in && !hand_on) continue;
      const ColRef rp = tables.b(wp, d);
      const unsigned tkb = (lane == 0 && !hand_on) ? hot_ticket(shadow, 0, slot, rp.hot) : 0u;
      float dbb[R];
      zero_col<R>(dbb);
      while (mask != 0ull) {
        const int l = __builtin_ctzll(mask);
        mask &= mask - 1ull;
        const float g = read_lane(gl, l);
        const float* acol = a_t + (size_t)(p - Sh + l - lo) * dp + lane;
#pragma unroll
        for (int r = 0; r < R; ++r) dbb[r] = fmaf(g, acol[r * kWave], dbb[r]);
      }
      const float bs = scale_of(wp, vexp, smode);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        dbb[r] *= bs;
        if (handed_in) dbb[r] += pend_in[(size_t)c * dp + r * kWave + lane];
      }
      if (hand_on) {
#pragma unroll
        for (int r = 0; r < R; ++r) pend_out[(size_t)(c - c_out) * dp + r * kWave + lane] = dbb[r];
      } else {
        scatter_add_ref<R>(rp, shadow, 0, slot, dbb, lane, d,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)tkb));
      }
    }
    __syncthreads();
  }
}

// Adds the shadow copies of hot column w of table t (blockIdx.y) into the table and zeroes them.
// A column no wave touched has all-zero shadows and is left alone, so the vocabulary may be
// smaller than kHotWords.
__global__ void __launch_bounds__(kBlock)
fold_kernel(float* A, float* B, Shadow shadow, int d) {
  const int w = blockIdx.x;
  float* const table = blockIdx.y == 0 ? A : B;
  float* const sh = blockIdx.y == 0 ? shadow.a : shadow.b;
  for (int e = threadIdx.x; e < d; e += kBlock) {
    float v[kShadows];
#pragma unroll
    for (int s = 0; s < kShadows; ++s) v[s] = sh[((int64_t)s * kHotWords + w) * d + e];  // all in flight
    float sum = 0.0f;
    bool any = false;
#pragma unroll
    for (int s = 0; s < kShadows; ++s) {
      if (v[s] != 0.0f) {
        any = true;
        sum += v[s];
        sh[((int64_t)s * kHotWords + w) * d + e] = 0.0f;
      }
    }
    if (any) table[(int64_t)w * d + e] += sum;
  }
}

// How full of frequent words a launch is, whatever the numbering of the vocabulary: a sample of
// at most kHeavySamples ids of `ids` (the words read from table B) is counted into a hashed
// histogram in LDS, and the sum of its kHeavyTop largest bins and its largest bin, scaled up to
// the n ids of the launch, are left where the update kernels look for "the ids among the 16 most
// frequent words" and "the most frequent word" (Shadow::hot_seen: four arrays of kHotCountSlots
// partial counts; the values go to slot 0, the other slots are zeroed); the same for `ids2` (the
// words read from table A; null: not counted).  The words that are not frequent add about four
// ids to every bin (0.4 % of the sample over the kHeavyTop bins, enough to tip a stream that is
// just below the line): the mean of the other bins is taken off each of the largest.  Two
// frequent words that share a bin only make the largest bin larger, which errs towards
// "frequent".  The sample's own noise is 0.18 % of the ids at a share of 6 %.  One workgroup.
constexpr int kHeavyThreads = 1024;
constexpr int kHeavyWaves = kHeavyThreads / kWave;
constexpr int kHeavySamples = 16384;
constexpr int kHeavyPerThread = kHeavySamples / kHeavyThreads;
constexpr int kHeavyBins = 4096;
constexpr int kHeavyPerLane = kHeavyBins / kHeavyThreads;   // bins a lane looks after
constexpr int kHeavyTop = kHotWords;
static_assert(kHeavyWaves * kHeavyTop == kWave * kHeavyPerLane, "second stage: one wave, same shape");

// Maximum over the 64 lanes, the same value in every lane: four DPP row rotations inside each
// 16-lane row, then the four row maxima are read out (as wave_sum does for sums).
__device__ __forceinline__ int wave_max(int x) {
  auto rot = [](int v, auto ctrl) {
    return __builtin_amdgcn_update_dpp(0, v, decltype(ctrl)::value, 0xf, 0xf, false);
  };
  x = max(x, rot(x, std::integral_constant<int, 0x128>{}));
  x = max(x, rot(x, std::integral_constant<int, 0x124>{}));
  x = max(x, rot(x, std::integral_constant<int, 0x122>{}));
  x = max(x, rot(x, std::integral_constant<int, 0x121>{}));
  return max(max(read_lane(x, 0), read_lane(x, 16)), max(read_lane(x, 32), read_lane(x, 48)));
}

// The kHeavyTop largest of the kWave * kHeavyPerLane counts a wave holds (v[k] of every lane,
// each below 2^22), largest first: out[r] is valid in every lane.  A count travels with its place
// (lane, k) in its low 8 bits, so every key is unique and the winner knows itself.  Wave-level
// only: no barrier, no LDS.
__device__ __forceinline__ void wave_top(int (&v)[kHeavyPerLane], int (&out)[kHeavyTop]) {
  static_assert(kHeavyPerLane <= 4, "two bits for the place inside a lane");
  const int lane = threadIdx.x & 63;
  int key[kHeavyPerLane];
#pragma unroll
  for (int k = 0; k < kHeavyPerLane; ++k) key[k] = v[k] < 0 ? -1 : (v[k] << 8) | (lane << 2) | k;
#pragma unroll
  for (int r = 0; r < kHeavyTop; ++r) {
    int best = -1;
#pragma unroll
    for (int k = 0; k < kHeavyPerLane; ++k) best = max(best, key[k]);
    const int top = wave_max(best);
    out[r] = top < 0 ? 0 : top >> 8;
#pragma unroll
    for (int k = 0; k < kHeavyPerLane; ++k)
      if (key[k] == top) key[k] = -1;
  }
}

__global__ void __launch_bounds__(kHeavyThreads)
count_heavy_kernel(const int* __restrict__ ids, int64_t n, const int* __restrict__ ids2, int64_t n2,
                   int* __restrict__ out) {
  __shared__ int s_bins[kHeavyBins];
  __shared__ int s_cand[kHeavyWaves * kHeavyTop];
  __shared__ long long s_result[2];
  __shared__ int s_binned;
  const int tid = threadIdx.x;
  for (int which = 0; which < 2; ++which) {
    const int* const p = which ? ids2 : ids;
    const int64_t len = which ? n2 : n;
    if (tid < 2) s_result[tid] = 0;
    if (tid == 0) s_binned = 0;
    if (p != nullptr && len > 0) {
      for (int k = tid; k < kHeavyBins; k += kHeavyThreads) s_bins[k] = 0;
      __syncthreads();
      const int64_t stride = (len + kHeavySamples - 1) / kHeavySamples;
      const int64_t nsamp = (len + stride - 1) / stride;
      int w[kHeavyPerThread];
#pragma unroll
      for (int k = 0; k < kHeavyPerThread; ++k) {   // all loads in flight together
        const int64_t at = (int64_t)k * kHeavyThreads + tid;
        w[k] = at < nsamp ? p[at * stride] : -1;
      }
      int binned = 0;
#pragma unroll
      for (int k = 0; k < kHeavyPerThread; ++k) {
        if (w[k] >= 0) {
          atomicAdd(&s_bins[((unsigned)w[k] * 2654435761u) >> 20], 1);
          ++binned;
        }
      }
      // (one LDS atomic per wave, not per thread: a thousand adds to one address take longer than
      // the histogram)
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) binned += __shfl_xor(binned, m, kWave);
      if ((tid & 63) == 0 && binned > 0) atomicAdd(&s_binned, binned);
      __syncthreads();
      // every wave picks the largest of its 256 bins, then the first wave the largest of those
      int v[kHeavyPerLane], top[kHeavyTop];
#pragma unroll
      for (int k = 0; k < kHeavyPerLane; ++k) v[k] = s_bins[k * kHeavyThreads + tid];
      wave_top(v, top);
      if ((tid & 63) == 0) {
#pragma unroll
        for (int r = 0; r < kHeavyTop; ++r) s_cand[(tid >> 6) * kHeavyTop + r] = top[r];
      }
      __syncthreads();
      if (tid < kWave) {
#pragma unroll
        for (int k = 0; k < kHeavyPerLane; ++k) v[k] = s_cand[k * kWave + tid];
        wave_top(v, top);
        if (tid == 0) {
          long long sum = 0;
#pragma unroll
          for (int r = 0; r < kHeavyTop; ++r) sum += top[r] > 0 ? top[r] : 0;
          // what the words that are not frequent leave in a bin: the mean of the other bins
          const double rest = (double)(s_binned - sum) / (double)(kHeavyBins - kHeavyTop);
          const double top_sum = fmax((double)sum - kHeavyTop * rest, 0.0);
          const double top_one = fmax((double)(top[0] > 0 ? top[0] : 0) - rest, 0.0);
          // sampled counts scaled up to the whole array (dropped words, id < 0, stay in the total)
          s_result[0] = (long long)(top_sum * (double)len / (double)nsamp);
          s_result[1] = (long long)(top_one * (double)len / (double)nsamp);
        }
      }
    }
    __syncthreads();
    const long long top_sum = s_result[0], top_one = s_result[1];
    for (int k = tid; k < kHotCountSlots; k += kHeavyThreads) {
      out[(2 * which) * kHotCountSlots + k] = k == 0 ? (int)min(top_sum, (long long)0x7fffffff) : 0;
      out[(2 * which + 1) * kHotCountSlots + k] = k == 0 ? (int)min(top_one, (long long)0x7fffffff) : 0;
    }
    __syncthreads();
  }
}

// Leaves, in mask[b] and mask[kHotCountSlots + b] (kHotCountSlots blocks), bit masks of the ids
// below kHotWords that block b saw in `ids` (the words read from table B) and in `ids2` (those
// read from table A; null: the same as `ids`): the columns that may have shadow copies, read
// copies or delta slots in this launch.  There a word counts under the index of its shadow
// copies (ColRef::hot), which for a sliced model is its packed column and not its id.  Every slot
// is written on every launch, so nothing needs clearing.
template <class Tables>
__global__ void __launch_bounds__(kBlock)
count_hot_kernel(const int* __restrict__ ids, int64_t n, const int* __restrict__ ids2, int64_t n2,
                 Tables tables, int* __restrict__ mask) {
  __shared__ int s_mask[kWavesPerBlock], s_mask2[kWavesPerBlock];
  int seen = 0, seen2 = 0;
  auto scan = [&](const int* p, int64_t len, int& bits, bool of_a) {
    auto bit = [&](int w) {
      if (Tables::kSliced) {
        const int h = w >= 0 ? (of_a ? tables.a(w, 0).hot : tables.b(w, 0).hot) : -1;
        return h >= 0 ? (1 << h) : 0;
      }
      return (w >= 0 && w < kHotWords) ? (1 << w) : 0;
    };
    const int64_t len4 = len / 4;
    const int4* p4 = reinterpret_cast<const int4*>(p);   // device allocations are 16-byte aligned
    const bool aligned = (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
    if (aligned) {
      for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < len4;
           i += (int64_t)gridDim.x * kBlock) {
        const int4 v = p4[i];
        bits |= bit(v.x) | bit(v.y) | bit(v.z) | bit(v.w);
      }
    }
    for (int64_t i = (aligned ? len4 * 4 : 0) + (int64_t)blockIdx.x * kBlock + threadIdx.x;
         i < len; i += (int64_t)gridDim.x * kBlock)
      bits |= bit(p[i]);
  };
  scan(ids, n, seen, false);
  if (ids2 != nullptr || Tables::kSliced) {
    scan(ids2 != nullptr ? ids2 : ids, ids2 != nullptr ? n2 : n, seen2, true);
  } else {
    seen2 = seen;
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    seen |= __shfl_xor(seen, m, kWave);
    seen2 |= __shfl_xor(seen2, m, kWave);
  }
  if ((threadIdx.x & 63) == 0) {
    s_mask[threadIdx.x >> 6] = seen;
    s_mask2[threadIdx.x >> 6] = seen2;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int m1 = 0, m2 = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) {
      m1 |= s_mask[w];
      m2 |= s_mask2[w];
    }
    mask[blockIdx.x] = m1;
    mask[kHotCountSlots + blockIdx.x] = m2;
  }
}

// Fills the per-XCD read copies of the hot columns the launch holds (block (w, t): word w of
// table t, 0 = B, 1 = A) from the tables.  Words the launch does not hold are skipped, so the
// vocabulary may be smaller than kHotWords.
__global__ void __launch_bounds__(kBlock)
publish_kernel(const float* __restrict__ A, const float* __restrict__ B, Shadow shadow, int d) {
  __shared__ int s_mask;
  const int w = blockIdx.x, which = blockIdx.y;
  if (threadIdx.x == 0) s_mask = 0;
  __syncthreads();
  int m = 0;
  for (int k = threadIdx.x; k < kHotCountSlots; k += kBlock)
    m |= shadow.hot_mask[which * kHotCountSlots + k];
  if (m != 0) atomicOr(&s_mask, m);
  __syncthreads();
  if (((s_mask >> w) & 1) == 0) return;
  const float* const col = (which ? A : B) + (int64_t)w * d;
  float* const pub = which ? shadow.pub_a : shadow.pub_b;
  for (int e = threadIdx.x; e < d; e += kBlock) {
    const float v = col[e];
#pragma unroll
    for (int x = 0; x < kXcds; ++x) pub[((int64_t)x * kHotWords + w) * d + e] = v;
  }
}

size_t shadow_bytes() { return (size_t)kShadows * kHotWords * kMaxRounds * kWave * sizeof(float); }
size_t shadow_counter_bytes() {
  return (size_t)2 * kShadows * kHotWords * kCounterStride * sizeof(unsigned) +
         (size_t)6 * kHotCountSlots * sizeof(int);   // four hot-word counts and the two id masks
}
size_t read_copy_bytes() { return (size_t)kXcds * kHotWords * kMaxRounds * kWave * sizeof(float); }

size_t occurs_bytes() { return (size_t)kOccurSlots * sizeof(int); }

hipError_t launch_fold(hipStream_t stream, float* A, float* B, Shadow shadow, int d) {
  hipLaunchKernelGGL(fold_kernel, dim3(kHotWords, 2), dim3(kBlock), 0, stream, A, B, shadow, d);
  return hipGetLastError();
}

static std::atomic<int> g_max_workgroups{0};
void set_max_workgroups(int n) { g_max_workgroups.store(n < 0 ? 0 : n); }
int get_max_workgroups() { return g_max_workgroups.load(); }

static std::atomic<int> g_ordered_mode{-1};
void set_ordered_mode(int mode) { g_ordered_mode.store(mode == 0 || mode == 1 ? mode : -1); }
int get_ordered_mode() { return g_ordered_mode.load(); }
int ordered_flag(bool forced_hot_mode) {
  const int mode = g_ordered_mode.load();
  if (mode == 1) return 2;
  if (mode == 0 || forced_hot_mode) return 0;   // a forced hot-word mode asks for that mode
  return 1;
}

static std::atomic<int> g_ordered_pos_workers{0}, g_ordered_neg_workers{0};
void set_ordered_workers(int pos, int neg) {
  g_ordered_pos_workers.store(pos > 0 ? pos : 0);
  g_ordered_neg_workers.store(neg > 0 ? neg : 0);
}
int ordered_pos_workers() { return g_ordered_pos_workers.load(); }
int ordered_neg_workers() { return g_ordered_neg_workers.load(); }

// Delta slots of the frequent columns in the ordered kernels: copies x twins.
static std::atomic<int> g_ordered_copies{2}, g_ordered_twins{2};
void set_ordered_copies(int copies, int twins) {
  if (copies < 0 || copies > kGridMaxC || twins < 1 || copies * twins > kShadows) return;
  g_ordered_copies.store(copies);
  g_ordered_twins.store(twins);
}
void get_ordered_copies(int* copies, int* twins) {
  *copies = g_ordered_copies.load();
  *twins = g_ordered_twins.load();
}

static std::atomic<int> g_hot_update_mode{-1};
void set_hot_update_mode(int mode) { g_hot_update_mode.store(mode >= 0 && mode <= 2 ? mode : -1); }
int get_hot_update_mode() { return g_hot_update_mode.load(); }

// Chooses how a launch of nwg workgroups treats the hot words (Shadow::combine and the hot-word
// count the kernels consult).  The combining mode parks up to kFoldEvery - 1 updates in each shadow
// copy, a couple of hundred for the most frequent word.  A launch of W waves keeps W work units in flight whose updates are
// invisible to each other anyway; with the Zipf share of the top word that is several hundred
// invisible updates of that word per 2048 waves.  Below that size the exact mode is used.
constexpr int64_t kCombineMinWaves = 2048;

static thread_local Shadow t_last_launch{};
static thread_local bool t_last_launch_set = false;
const Shadow* last_launch_shadow() { return t_last_launch_set ? &t_last_launch : nullptr; }
void note_last_launch(const Shadow& shadow) {
  t_last_launch = shadow;
  t_last_launch_set = true;
}

template <class Tables>
static hipError_t prepare_hot_mode_for(hipStream_t stream, const int* ids, int64_t n,
                                       const int* ids2, int64_t n2, const Tables& tables,
                                       const float* A, const float* B, int d, int64_t nwg,
                                       int waves_per_wg, Shadow* shadow) {
  const int mode = g_hot_update_mode.load();
  shadow->hot_total = 0;
  shadow->hot_total_a = 0;
  if (A == nullptr || B == nullptr) shadow->pub_a = shadow->pub_b = nullptr;
  const bool forced = mode == kHotExact || mode == kHotCombining || mode == kHotOff;
  if (forced)
    shadow->combine = mode;
  else
    shadow->combine = nwg * waves_per_wg >= kCombineMinWaves ? kHotCombining : kHotExact;
  shadow->combine_a = shadow->combine;
  shadow->ordered = ordered_flag(forced);
  shadow->grid_c = g_ordered_copies.load();
  shadow->grid_r = g_ordered_twins.load();
  if (shadow->combine != kHotCombining) shadow->pub_a = shadow->pub_b = nullptr;
  if (n <= 0 || (forced && shadow->pub_a == nullptr)) {
    note_last_launch(*shadow);
    return hipSuccess;
  }
  // Shadow copies pay only if the launch really holds hot words: count them first (the kernels
  // read the count from memory, the host does not wait for it).  The same pass notes which hot
  // ids occur at all, for the read copies.
  hipLaunchKernelGGL(count_hot_kernel<Tables>, dim3(kHotCountSlots), dim3(kBlock), 0, stream, ids,
                     n, ids2, n2, tables, shadow->hot_mask);
  hipLaunchKernelGGL(count_heavy_kernel, dim3(1), dim3(kHeavyThreads), 0, stream, ids, n, ids2, n2,
                     shadow->hot_seen);
  if (!forced) {
    shadow->hot_total = n;
    shadow->hot_total_a = ids2 != nullptr ? n2 : 0;
  }
  if (shadow->pub_a != nullptr)
    hipLaunchKernelGGL(publish_kernel, dim3(kHotWords, 2), dim3(kBlock), 0, stream, A, B, *shadow,
                       d);
  note_last_launch(*shadow);
  return hipGetLastError();
}

hipError_t prepare_hot_mode(hipStream_t stream, const int* ids, int64_t n, const int* ids2,
                            int64_t n2, const float* A, const float* B, int d, int64_t nwg,
                            int waves_per_wg, Shadow* shadow) {
  return prepare_hot_mode_for(stream, ids, n, ids2, n2, PlainTables{nullptr, nullptr}, A, B, d, nwg,
                              waves_per_wg, shadow);
}

hipError_t prepare_hot_mode_sliced(hipStream_t stream, const int* ids, int64_t n, const int* ids2,
                                   int64_t n2, const SliceMap& m, int d, int64_t nwg,
                                   int waves_per_wg, Shadow* shadow) {
  // the shadowed columns are the first columns of part 0
  return prepare_hot_mode_for(stream, ids, n, ids2, n2, SlicedTables{m}, m.mats[1], m.mats[0], d,
                              nwg, waves_per_wg, shadow);
}

hipError_t persistent_grid(const void* kernel, int threads, size_t lds_bytes, int64_t units,
                           int64_t min_units_per_wg, int64_t* nwg) {
  int dev = 0, cus = 0, per_cu = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (err != hipSuccess) return err;
  err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, lds_bytes);
  if (err != hipSuccess) return err;
  if (per_cu < 1) per_cu = 1;
  int64_t n = (int64_t)cus * per_cu;
  const int64_t by_units = (units + min_units_per_wg - 1) / min_units_per_wg;
  if (n > by_units) n = by_units;
  const int limit = g_max_workgroups.load();
  if (limit > 0 && n > limit) n = limit;
  if (n < 1) n = 1;
  *nwg = n;
  return hipSuccess;
}

// Two ways of cutting `units` over a persistent grid.  `bounded` gives every workgroup at least
// min_units consecutive units, which keeps the number of units in flight (whose updates do not see
// each other) small against a launch that is full of frequent words; `wide` fills the device as
// soon as every workgroup has min_units_wide units.  The kernel is launched with the wide grid and
// picks one of the two once it knows whether the launch holds hot words.
hipError_t split_grid(const void* kernel, int threads, size_t lds_bytes, int64_t units,
                      int64_t min_units, int64_t min_units_wide, GridSplit* out) {
  int64_t nwg = 0;
  hipError_t err = persistent_grid(kernel, threads, lds_bytes, units, min_units, &nwg);
  if (err != hipSuccess) return err;
  out->per_wg = (units + nwg - 1) / nwg;
  if (out->per_wg < 1) out->per_wg = 1;
  out->nwg = (units + out->per_wg - 1) / out->per_wg;
  if (out->nwg < 1) out->nwg = 1;
  err = persistent_grid(kernel, threads, lds_bytes, units, min_units_wide, &nwg);
  if (err != hipSuccess) return err;
  out->per_wg_wide = (units + nwg - 1) / nwg;
  if (out->per_wg_wide < 1) out->per_wg_wide = 1;
  out->nwg_wide = (units + out->per_wg_wide - 1) / out->per_wg_wide;
  if (out->nwg_wide < out->nwg) {
    out->nwg_wide = out->nwg;
    out->per_wg_wide = out->per_wg;
  }
  return hipSuccess;
}

// Sum of the block's 256 per-thread values by a fixed LDS tree; the result is valid in thread 0.
__device__ __forceinline__ double block_tree_sum(double t, double* s) {
  s[threadIdx.x] = t;
  __syncthreads();
  for (int w = kBlock / 2; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) s[threadIdx.x] += s[threadIdx.x + w];
    __syncthreads();
  }
  return s[0];
}

// First stage of the fold for long partial arrays: block b sums its slice [b*len, (b+1)*len) in a
// fixed order and leaves the sum in the slice's first element (it has read the whole slice before
// it writes, and no other block touches the slice).
__global__ void __launch_bounds__(kBlock)
finalize_slices_kernel(double* __restrict__ partials, int64_t n, int64_t len) {
  __shared__ double s[kBlock];
  const int64_t base = (int64_t)blockIdx.x * len;
  const int64_t end = base + len < n ? base + len : n;
  double t = 0.0;
  for (int64_t k = base + threadIdx.x; k < end; k += kBlock) t += partials[k];
  const double total = block_tree_sum(t, s);
  if (threadIdx.x == 0) partials[base] = total;
}

// Folds partials[0], partials[stride], ... (n of them) in a fixed order (thread t takes t, t+256,
// ...; then a fixed LDS tree), so the result does not depend on block scheduling.
__global__ void __launch_bounds__(kBlock)
finalize_kernel(const double* __restrict__ partials, int64_t n, int64_t stride, float* Retval32,
                double* Retval64) {
  __shared__ double s[kBlock];
  double t = 0.0;
  for (int64_t k = threadIdx.x; k < n; k += kBlock) t += partials[k * stride];
  const double total = block_tree_sum(t, s);
  if (threadIdx.x == 0) {
    if (Retval32 != nullptr) Retval32[0] += (float)total;
    if (Retval64 != nullptr) Retval64[0] += total;
  }
}

int max_rows() { return kMaxRounds * kWave; }

int64_t eval_partials_needed(int64_t units) { return blocks_per_xcd(units) * kXcds; }

// Context columns gathered per chunk: as many as fit in roughly 64 registers per lane.
template <int R>
struct PosChunk {
  static constexpr int value = R <= 4 ? 12 : R <= 6 ? 10 : R <= 8 ? 8 : R <= 12 ? 5 : 3;
};


// Workers of the ordered form, and no fewer than 64 tokens per worker.  What the held-out loss
// bounds is the tokens that are between their reads and their adds at any time.  Held-out loss of
// the 10k-vocabulary configuration on a raw stream against the sequential oracle, teams of four
// waves, 576 negative workers: 96: -0.07 %, 128: -0.06 %, 192: -0.25 %, 256: -0.67 %, 384: -3.1 %;
// headline shape (8 minibatches, sequential oracle 9.8094): 128: -0.3 %, 192: -0.9 %, 256: -1.7 %.
constexpr int64_t kMinTokensPerChain = 64;

int64_t ordered_pos_chains(int ncols, int shift, int builtin_workers) {
  int64_t chains = ((int64_t)ncols + kMinTokensPerChain - 1) / kMinTokensPerChain;
  // what is bounded is the pairs in flight: a token of a window of half-width 10 has twice the
  // pairs of one of half-width 5, so half the workers
  int64_t builtin = builtin_workers;
  if (shift > 5) builtin = std::max<int64_t>(32, builtin * 6 / (shift + 1));
  const int64_t most = ordered_pos_workers() > 0 ? ordered_pos_workers() : builtin;
  if (chains > most) chains = most;
  const int limit = g_max_workgroups.load();
  if (limit > 0 && chains > (int64_t)limit * kWavesPerBlock) chains = (int64_t)limit * kWavesPerBlock;
  return chains < 1 ? 1 : chains;
}

template <int R, int TW, class Tables>
static hipError_t launch_pos_chain_tw(hipStream_t stream, int d, int ncols, int64_t chains,
                                      const int* W, const int* LB, const int* UB,
                                      const Tables& tables, float lrate, float vexp,
                                      const Shadow& shadow) {
  const int64_t per_chain = ((int64_t)ncols + chains - 1) / chains;   // teams beyond: empty range
  constexpr int CH = TW == 1 ? PosChunk<R>::value : TeamChunk<R>::value;
  hipLaunchKernelGGL((pos_chain_kernel<R, CH, TW, Tables>), dim3((unsigned)chains),
                     dim3(kWave * TW), 0, stream, d, ncols, per_chain, W, LB, UB, tables, lrate,
                     vexp, scale_mode(vexp), shadow);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  return launch_grid_fold(stream, tables, shadow, d);
}

template <int R, class Tables>
static hipError_t launch_pos_chain(hipStream_t stream, int d, int ncols, int shift, const int* W,
                                   const int* LB, const int* UB, const Tables& tables, float lrate,
                                   float vexp, const Shadow& shadow) {
  const int64_t chains = ordered_pos_chains(ncols, shift, kPosTeams);
  // a window that the 64 lanes of a wave cannot cover is walked by single waves
  if (shift < kChainLook)
    return launch_pos_chain_tw<R, kTeamWaves>(stream, d, ncols, chains, W, LB, UB, tables, lrate,
                                              vexp, shadow);
  return launch_pos_chain_tw<R, 1>(stream, d, ncols, chains, W, LB, UB, tables, lrate, vexp, shadow);
}

// Tile size: 16 tokens, or 8 if that is what lets two workgroups share a CU's LDS; if even 8
// tokens do not fit in one CU's LDS the per-centre kernel is used instead.  A tile is a small
// synchronous batch (all its dot products use the staged columns), so larger tiles would trade
// fewer atomics for staler updates of the frequent words.
static int pick_tile(int R, int Sh) {
  constexpr size_t kShare = 80 * 1024, kLimit = 160 * 1024;
  int T = 16;
  while (T > 8 && tile_lds_bytes(R, T, Sh) > kShare) T >>= 1;
  if (tile_lds_bytes(R, T, Sh) > kLimit) return 0;
  return T;
}

// Launches the tiled pass and the fold of the shadow copies into fold_a / fold_b (the tables that
// hold the shadowed columns).  *launched is false, and nothing is enqueued, if no tile fits.
template <int R, class Tables>
static hipError_t launch_pos_tile_r(hipStream_t stream, int d, int ncols, int shift, const int* W,
                                    const int* LB, const int* UB, const Tables& tables,
                                    float* fold_a, float* fold_b, float lrate, float vexp,
                                    Shadow shadow, bool* launched) {
  const int Sh = shift < 0 ? 0 : (shift > kMaxHalo ? kMaxHalo : shift);
  const int T = Sh > 0 ? pick_tile(R, Sh) : 0;
  *launched = T != 0;
  if (T == 0) return hipSuccess;
  // Deltas are carried between tiles when the overlaps of consecutive tiles do not overlap each
  // other and the extra LDS does not cost a workgroup per CU.
  constexpr size_t kShareLds = 80 * 1024, kLimitLds = 160 * 1024;
  const size_t base = tile_lds_bytes(R, T, Sh), with = base + tile_carry_bytes(R, Sh);
  const int carry = (T >= 2 * Sh && with <= (base <= kShareLds ? kShareLds : kLimitLds)) ? 1 : 0;
  const size_t lds = carry ? with : base;
  auto kern = pos_tile_kernel<R, Tables>;
  hipError_t err = hipSuccess;
  if (lds > 48 * 1024) {
    err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return err;
  }
  const int64_t ntiles = ((int64_t)ncols + T - 1) / T;
  GridSplit g;
  err = split_grid(reinterpret_cast<const void*>(kern), kTileThreads, lds, ntiles, kMinTilesPerWg,
                   kMinTilesPerWgWide, &g);
  if (err != hipSuccess) return err;
  if constexpr (Tables::kSliced)
    err = prepare_hot_mode_sliced(stream, W, ncols, nullptr, 0, tables.m, d, g.nwg, kTileWaves,
                                  &shadow);
  else
    err = prepare_hot_mode(stream, W, ncols, nullptr, 0, fold_a, fold_b, d, g.nwg, kTileWaves,
                           &shadow);
  if (err != hipSuccess) return err;
  // only a launch that counts its hot words can turn out cold
  const int64_t nwg = shadow.hot_total > 0 ? g.nwg_wide : g.nwg;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kTileThreads), lds, stream, d, ncols, T, Sh,
                     carry, ntiles, g.per_wg, g.per_wg_wide, W, LB, UB, tables, lrate, vexp,
                     scale_mode(vexp), shadow);
  err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (shadow.ordered != 0) {
    err = launch_pos_chain<R>(stream, d, ncols, shift, W, LB, UB, tables, lrate, vexp, shadow);
    if (err != hipSuccess) return err;
  }
  return launch_fold(stream, fold_a, fold_b, shadow, d);
}

template <int R>
static hipError_t launch_pos_plain_r(hipStream_t stream, int d, int ncols, int shift, const int* W,
                                     const int* LB, const int* UB, float* A, float* B, float lrate,
                                     float vexp, Shadow shadow) {
  bool launched = false;
  hipError_t err = launch_pos_tile_r<R>(stream, d, ncols, shift, W, LB, UB, PlainTables{A, B}, A, B,
                                        lrate, vexp, shadow, &launched);
  if (err != hipSuccess || launched) return err;
  // no tile fits in LDS: one wave per centre, or the ordered kernel if the launch's count of
  // frequent words says so (no shadow copies here, only the count)
  const int64_t per_xcd = blocks_per_xcd(ncols);
  err = prepare_hot_mode(stream, W, ncols, nullptr, 0, nullptr, nullptr, d, per_xcd * kXcds,
                         kWavesPerBlock, &shadow);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL((pos_kernel<R, PosChunk<R>::value, true>), dim3((unsigned)(per_xcd * kXcds)),
                     dim3(kBlock), 0, stream, d, ncols, per_xcd, W, LB, UB, A, B, lrate, vexp,
                     scale_mode(vexp), 0.0, nullptr, shadow);
  err = hipGetLastError();
  if (err != hipSuccess || shadow.ordered == 0) return err;
  return launch_pos_chain<R>(stream, d, ncols, shift, W, LB, UB, PlainTables{A, B}, lrate, vexp,
                             shadow);
}

hipError_t launch_pos(hipStream_t stream, int nrows, int ncols, int shift, const int* W,
                      const int* LB, const int* UB, float* A, float* B, float lrate, float vexp,
                      Shadow shadow) {
  const int rounds = (nrows + kWave - 1) / kWave;
#define CALL(R) \
  return launch_pos_plain_r<R>(stream, nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, shadow)
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
}

hipError_t launch_slice_pos_chain(hipStream_t stream, int nrows, int ncols, int shift,
                                  const int* W, const int* LB, const int* UB, const SliceMap& m,
                                  float lrate, float vexp, const Shadow& shadow) {
  const int rounds = (nrows + kWave - 1) / kWave;
#define CALL(R)                                                                               \
  return launch_pos_chain<R>(stream, nrows, ncols, shift, W, LB, UB, SlicedTables{m}, lrate, vexp, \
                             shadow)
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
}

hipError_t launch_slice_pos_tiled(hipStream_t stream, int nrows, int ncols, int shift,
                                  const int* W, const int* LB, const int* UB, const SliceMap& m,
                                  float lrate, float vexp, Shadow shadow, bool* launched) {
  const int rounds = (nrows + kWave - 1) / kWave;
#define CALL(R)                                                                                 \
  return launch_pos_tile_r<R>(stream, nrows, ncols, shift, W, LB, UB, SlicedTables{m}, m.mats[1], \
                              m.mats[0], lrate, vexp, shadow, launched)
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
}

hipError_t launch_finalize(hipStream_t stream, double* partials, int64_t n, float* Retval32,
                           double* Retval64) {
  // Long arrays are first cut into at most 1024 slices summed by one block each.
  constexpr int64_t kSliceMin = 256;
  int64_t stride = 1;
  if (n > 4 * kSliceMin) {
    int64_t len = (n + 1023) / 1024;
    if (len < kSliceMin) len = kSliceMin;
    const int64_t slices = (n + len - 1) / len;
    hipLaunchKernelGGL(finalize_slices_kernel, dim3((unsigned)slices), dim3(kBlock), 0, stream,
                       partials, n, len);
    stride = len;
    n = slices;
  }
  hipLaunchKernelGGL(finalize_kernel, dim3(1), dim3(kBlock), 0, stream, partials, n, stride,
                     Retval32, Retval64);
  return hipGetLastError();
}

template <int R>
static hipError_t launch_pos_eval_r(hipStream_t stream, int d, int ncols, const int* W,
                                    const int* LB, const int* UB, const float* A, const float* B,
                                    double floorv, double* partials, int64_t* nparts) {
  auto kern = pos_eval_kernel<R, PosChunk<R>::value>;
  int64_t nwg = 0;
  hipError_t err = persistent_grid(reinterpret_cast<const void*>(kern), kBlock, 0, ncols,
                                   kMinEvalCentresPerWg, &nwg);
  if (err != hipSuccess) return err;
  const int64_t cap = eval_partials_needed(ncols);   // what the caller's buffer holds
  if (nwg > cap) nwg = cap;
  nwg = (nwg + kXcds - 1) / kXcds * kXcds;           // whole XCD rows; empty ranges write 0
  const int64_t units_per_wg = ((int64_t)ncols + nwg - 1) / nwg;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(kBlock), 0, stream, d, ncols, units_per_wg, W,
                     LB, UB, A, B, floorv, partials);
  *nparts = nwg;
  return hipGetLastError();
}

hipError_t launch_eval_pos(hipStream_t stream, int nrows, int ncols, const int* W, const int* LB,
                           const int* UB, const float* A, const float* B, double floorv,
                           double* partials, float* Retval32, double* Retval64) {
  const int rounds = (nrows + kWave - 1) / kWave;
  hipError_t err = hipSuccess;
  int64_t nparts = 0;
#define CALL(R)                                                                              \
  err = launch_pos_eval_r<R>(stream, nrows, ncols, W, LB, UB, A, B, floorv, partials, &nparts); \
  break
  W2V_ROUNDS_SWITCH(rounds, CALL)
#undef CALL
  if (err != hipSuccess) return err;
  return launch_finalize(stream, partials, nparts, Retval32, Retval64);
}

}  // namespace w2v
