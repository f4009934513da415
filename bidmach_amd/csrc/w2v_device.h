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

// Hogwild scatter of a column held in the dword-strided register layout: col[e] += x[e] with
// hardware float atomics (global_atomic_add_f32, no return value, no compare-and-swap loop).
//
// The L2 retires atomics per 128-byte line request, and a column starts wherever w*d*4 falls,
// so a wave instruction that covers elements [64r, 64r+64) of the column straddles three lines.
// The lanes are therefore rotated by the column's misalignment (ds_bpermute) so that every
// instruction covers exactly two whole lines: lane l of round r' handles element
// 64*r' + l - mis, where mis = (column start / 4) mod 32.  One extra, mostly empty, round pays
// for roughly a third fewer line requests.
template <int R>
__device__ __forceinline__ void atomic_add_col(float* __restrict__ col, const float (&x)[R],
                                               int lane, int d) {
  const int mis = (int)((reinterpret_cast<uintptr_t>(col) >> 2) & 31u);
  const int src = (lane - mis) & (kWave - 1);
  float prev = 0.0f;
#pragma unroll
  for (int r = 0; r <= R; ++r) {
    float cur = 0.0f;
    if (r < R) cur = __shfl(x[r], src, kWave);
    const float v = (lane >= mis) ? cur : prev;
    const int e = r * kWave + lane - mis;
    if (e >= 0 && e < d) unsafeAtomicAdd(col + e, v);
    prev = cur;
  }
}

template <int R>
__device__ __forceinline__ void atomic_axpy_col(float* __restrict__ col, float alpha,
                                                const float (&x)[R], int lane, int d) {
  float y[R];
#pragma unroll
  for (int r = 0; r < R; ++r) y[r] = alpha * x[r];
  atomic_add_col<R>(col, y, lane, d);
}

// Shadow copies of the hottest columns.
//
// Word ids are frequency ranks, so under a Zipf law ids 0..7 each receive hundreds of thousands
// of column updates per call.  Atomics to one cache line retire one after the other in L2
// (about 36 ns each), which would make those few columns the critical path of the whole pass.
// While a pass runs, the value of a hot column w < kHotWords is therefore represented as
//     table[w] + sum over s < kShadows of shadow[s][w]
// with the shadows in a scratch buffer that is zero between calls: a reader sums all copies, a
// writer adds into the one copy chosen by its workgroup index, so the same-line queue is spread
// over several lines and no update is delayed or dropped.  A small kernel folds the shadows
// back into the table (and zeroes them) at the end of the call.  The number of copies follows
// the Zipf law: 16 for word 0, 8 for words 1-2, 4 for words 3-6, 2 for word 7, so every hot
// line sees about the same queue and readers do not sum more copies than needed.
constexpr int kHotWords = 8;
constexpr int kShadows = 16;

__device__ __forceinline__ int shadow_copies(int w) {
  return kShadows >> (31 - __builtin_clz(w + 1));
}

struct Shadow {
  float* a;  // [kShadows][kHotWords][d] for table A
  float* b;  // same for table B
};

// ---- where a word's column lives -------------------------------------------------------------
//
// The kernels that serve both the single-table model and the sliced, multi-part model see the
// model through a small policy object: it turns a word id into a ColRef and answers the two
// questions the sliced model adds (is this pair trained? may this column be written?).

constexpr int kMine = 1;  // sliced model: a tail word this worker owns; single table: any word
constexpr int kHead = 2;  // sliced model: a head word, resident on every worker

struct ColRef {
  float* col;  // start of the column
  int hot;     // index of its shadow copies, or -1 if the column has none
  int flags;   // 0: not resident (skip the word), else kMine or kHead
};

template <int R>
__device__ __forceinline__ void load_col_ref(float (&x)[R], const ColRef& ref, const float* shadow,
                                             int lane, int d) {
  load_col<R>(x, ref.col, lane, d);
  if (ref.hot >= 0) {
    const int copies = shadow_copies(ref.hot);
#pragma unroll 1
    for (int s = 0; s < copies; s += 2) {
      float y0[R], y1[R];
      load_col<R>(y0, shadow + ((int64_t)s * kHotWords + ref.hot) * d, lane, d);
      load_col<R>(y1, shadow + ((int64_t)(s + 1) * kHotWords + ref.hot) * d, lane, d);
#pragma unroll
      for (int r = 0; r < R; ++r) x[r] += y0[r] + y1[r];
    }
  }
}

// Column that receives the atomics for `ref` from workgroup number `wg`.
__device__ __forceinline__ float* scatter_ref(const ColRef& ref, float* shadow, int wg, int d) {
  if (ref.hot < 0) return ref.col;
  const int slot = wg & (shadow_copies(ref.hot) - 1);
  return shadow + ((int64_t)slot * kHotWords + ref.hot) * d;
}

// A table-relative form of the two helpers above, for kernels that address one pair of tables by
// word id: column w of `table`, shadowed iff w < kHotWords.
template <int R>
__device__ __forceinline__ void load_col_hot(float (&x)[R], const float* table,
                                             const float* shadow, int w, int lane, int d) {
  const ColRef ref{const_cast<float*>(table) + (int64_t)w * d, w < kHotWords ? w : -1, kMine};
  load_col_ref<R>(x, ref, shadow, lane, d);
}

// Column that receives the atomics for word w from workgroup number `wg`.
__device__ __forceinline__ float* scatter_target(float* table, float* shadow, int w, int wg,
                                                 int d) {
  const ColRef ref{table + (int64_t)w * d, w < kHotWords ? w : -1, kMine};
  return scatter_ref(ref, shadow, wg, d);
}

// One pair of tables: word w is column w of A / of B; every pair is trained, every column written.
struct PlainTables {
  float* A;
  float* B;
  static constexpr bool kSliced = false;
  __device__ __forceinline__ ColRef a(int w, int d) const {
    return ColRef{A + (int64_t)w * d, w < kHotWords ? w : -1, w >= 0 ? kMine : 0};
  }
  __device__ __forceinline__ ColRef b(int w, int d) const {
    return ColRef{B + (int64_t)w * d, w < kHotWords ? w : -1, w >= 0 ? kMine : 0};
  }
  __device__ __forceinline__ bool trained(int, int) const { return true; }
  __device__ __forceinline__ bool written(int) const { return true; }
};

// A sliced, multi-part model (jni/src/BIDMach_CPUMACH.c:80-88 of the reference).  The vocabulary
// is split over nslices workers: ids below nhead ("head") are resident on every worker, an id
// >= nhead ("tail") on worker id % nslices only.  A worker packs its resident words densely
// (head, then its tail words in id order: packed column nhead + (id - nhead) / nslices) and cuts
// the packed table into parts of maxcols columns, each part a separate allocation; part m has
// its B table at mats[2m] and its A table at mats[2m+1].  Passed to kernels by value.
constexpr int kMaxSliceParts = 32;
struct SliceMap {
  float* mats[2 * kMaxSliceParts];
  int nparts;   // parts present; a word whose packed column falls beyond them is skipped
  int islice;   // this worker
  int nslices;  // workers the tail of the vocabulary is dealt to
  int nhead;    // ids below this are resident on every worker
  int maxcols;  // columns per part
  int dohead;   // 0: head columns read-only, 1: written, 2: written and head-head pairs trained
};

struct SlicedTables {
  SliceMap m;
  static constexpr bool kSliced = true;
  // which: 0 = B table of the part, 1 = A table
  __device__ __forceinline__ ColRef place(int w, int which, int d) const {
    ColRef r{nullptr, -1, 0};
    if (w < 0) return r;
    const bool head = w < m.nhead;
    const bool mine = !head && (w % m.nslices == m.islice);
    if (!head && !mine) return r;
    const int packed = head ? w : (w - m.nhead) / m.nslices + m.nhead;
    const int part = packed / m.maxcols;
    if (part >= m.nparts) return r;
    r.col = m.mats[2 * part + which] + (int64_t)(packed - part * m.maxcols) * d;
    r.hot = (part == 0 && packed < kHotWords) ? packed : -1;  // the first columns of part 0
    r.flags = head ? kHead : kMine;
    return r;
  }
  __device__ __forceinline__ ColRef a(int w, int d) const { return place(w, 1, d); }
  __device__ __forceinline__ ColRef b(int w, int d) const { return place(w, 0, d); }
  // Rules of the reference (:137-157, :315-349); both words are resident when these are asked.
  __device__ __forceinline__ bool trained(int fa, int fb) const {
    return (((fa | fb) & kMine) != 0) || m.dohead > 1;
  }
  __device__ __forceinline__ bool written(int f) const {
    return f == kMine || (f == kHead && m.dohead > 0);
  }
};

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
