// Minibatch preprocessing on the device: what BIDMach.networks.Word2Vec.wordMats does before the
// operators run (src/main/scala/BIDMach/networks/Word2Vec.scala:214-364 of the reference).
//
//   words   out-of-vocabulary and subsampled tokens become -1 (:218-225)
//   lb, ub  random window bounds, ub = min(nskip, floor(u*nskip)+1), lb = -ub, clipped so that a
//           window never leaves its sentence or the minibatch (:228-237)
//   ctx     the context word of every valid (centre, context) pair, compacted in centre-major
//           order (:283-330), then randomly permuted (:334-346; here, as in the reference's GPU
//           branch :250-256, by sorting on random keys)
//   negs    G*nneg draws min(V-1, floor(V * u**expt)), G = floor(#pairs / nreuse) (:349-358)
//
// Random numbers come from a counter-based generator (Philox4x32-10) keyed by (seed, call
// counter, stream, element index), so a run is reproducible and a host twin can regenerate the
// same draws.  The reference draws from BIDMat's generators, which are not part of its tree.
#include <hipcub/hipcub.hpp>

#include "../../include/bidmach_w2v.h"
#include "w2v_device.h"

namespace w2v {

__host__ __device__ inline unsigned philox_word0(unsigned long long index, unsigned stream,
                                                 unsigned call, unsigned long long seed) {
  unsigned c0 = (unsigned)index, c1 = (unsigned)(index >> 32), c2 = stream, c3 = call;
  unsigned k0 = (unsigned)seed, k1 = (unsigned)(seed >> 32);
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const unsigned long long p0 = (unsigned long long)0xD2511F53u * c0;
    const unsigned long long p1 = (unsigned long long)0xCD9E8D57u * c2;
    const unsigned n0 = (unsigned)(p1 >> 32) ^ c1 ^ k0;
    const unsigned n1 = (unsigned)p1;
    const unsigned n2 = (unsigned)(p0 >> 32) ^ c3 ^ k1;
    const unsigned n3 = (unsigned)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

__device__ __forceinline__ float uniform01(unsigned x) { return (float)(x >> 8) * (1.0f / 16777216.0f); }

enum Stream : unsigned { kSubsample = 0, kWindow = 1, kPermute = 2, kNegative = 3 };

// mats is the reference's 2 x n IMat, column-major: mats[2*i + wrow] is the word of token i and
// mats[2*i + 1 - wrow] its sentence id (wrow = 1 when iflip).
__global__ void __launch_bounds__(kBlock)
wm_words_kernel(int n, const int* __restrict__ mats, int wrow, int vocab, float salpha,
                unsigned call, unsigned long long seed, int* __restrict__ words) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const int w = mats[2 * i + wrow];
  bool good = w >= 0 && w < vocab;
  float wrat = (float)(w + 1) * salpha;
  wrat = sqrtf(wrat) + wrat;
  good = good && uniform01(philox_word0(i, kSubsample, call, seed)) < wrat;
  words[i] = good ? w : -1;
}

__global__ void __launch_bounds__(kBlock)
wm_bounds_kernel(int n, const int* __restrict__ mats, int wrow, const int* __restrict__ words,
                 int nskip, unsigned call, unsigned long long seed, int* __restrict__ lb,
                 int* __restrict__ ub, int* __restrict__ npairs) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const float u = uniform01(philox_word0(i, kWindow, call, seed));
  int hi = min(nskip, (int)(u * (float)nskip) + 1);
  int lo = -hi;
  const int s = mats[2 * i + 1 - wrow];
  // nearest sentence boundary within reach of the window
  for (int j = 1; j <= hi; ++j) {
    if (i + j >= n || mats[2 * (i + j) + 1 - wrow] != s) { hi = j - 1; break; }
  }
  for (int j = 1; j <= -lo; ++j) {
    if (i - j < 0 || mats[2 * (i - j) + 1 - wrow] != s) { lo = -(j - 1); break; }
  }
  lb[i] = lo;
  ub[i] = hi;
  int cnt = 0;
  if (words[i] >= 0) {
    for (int j = lo; j <= hi; ++j) cnt += (j != 0 && words[i + j] >= 0) ? 1 : 0;
  }
  npairs[i] = cnt;
}

__global__ void __launch_bounds__(kBlock)
wm_contexts_kernel(int n, const int* __restrict__ words, const int* __restrict__ lb,
                   const int* __restrict__ ub, const int* __restrict__ offsets,
                   unsigned call, unsigned long long seed, int* __restrict__ ctx,
                   unsigned* __restrict__ keys) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= n || words[i] < 0) return;
  int o = offsets[i];
  for (int j = lb[i]; j <= ub[i]; ++j) {
    if (j != 0 && words[i + j] >= 0) {
      ctx[o] = words[i + j];
      keys[o] = philox_word0((unsigned long long)o, kPermute, call, seed);
      ++o;
    }
  }
}

// counts[0] = number of valid pairs, counts[1] = number of groups
__global__ void wm_counts_kernel(int n, const int* __restrict__ offsets,
                                 const int* __restrict__ npairs, int nreuse, int* counts) {
  const int total = n > 0 ? offsets[n - 1] + npairs[n - 1] : 0;
  counts[0] = total;
  counts[1] = total / nreuse;
}

__global__ void __launch_bounds__(kBlock)
wm_negatives_kernel(const int* __restrict__ counts, int nneg, int vocab, double expt, int iexpt,
                    unsigned call, unsigned long long seed, int* __restrict__ negs) {
  const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
  if (i >= (long long)counts[1] * nneg) return;
  const double u = (double)uniform01(philox_word0((unsigned long long)i, kNegative, call, seed));
  double p;
  if (iexpt > 0) {  // integer exponent (4 for the default wexpt = 0.75): exact repeated products
    p = 1.0;
    for (int k = 0; k < iexpt; ++k) p *= u;
  } else {
    p = pow(u, expt);
  }
  const long long id = (long long)((double)vocab * p);
  negs[i] = (int)(id < (long long)vocab - 1 ? id : (long long)vocab - 1);
}

struct WordMatsScratch {
  int* npairs = nullptr;
  int* offsets = nullptr;
  int* ctx_raw = nullptr;
  unsigned* keys = nullptr;
  unsigned* keys_sorted = nullptr;
  void* temp = nullptr;
  size_t temp_bytes = 0;
  int n_cap = 0;
  long long pair_cap = 0;
};

thread_local WordMatsScratch t_wm[64];

static void wm_free(WordMatsScratch& s) {
  (void)hipFree(s.npairs); (void)hipFree(s.offsets); (void)hipFree(s.ctx_raw);
  (void)hipFree(s.keys); (void)hipFree(s.keys_sorted); (void)hipFree(s.temp);
  s = WordMatsScratch{};
}

static hipError_t wm_scratch(int n, int nskip, WordMatsScratch** out) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  WordMatsScratch& s = t_wm[dev];
  const long long pairs = (long long)n * 2 * nskip;
  if (s.n_cap < n || s.pair_cap < pairs) {
    wm_free(s);
    size_t t1 = 0, t2 = 0;
    err = hipcub::DeviceScan::ExclusiveSum(nullptr, t1, (int*)nullptr, (int*)nullptr, n);
    if (err != hipSuccess) return err;
    err = hipcub::DeviceRadixSort::SortPairs(nullptr, t2, (unsigned*)nullptr, (unsigned*)nullptr,
                                             (int*)nullptr, (int*)nullptr, (int)pairs, 0, 32);
    if (err != hipSuccess) return err;
    const size_t temp = t1 > t2 ? t1 : t2;
    const bool ok =
        hipMalloc(reinterpret_cast<void**>(&s.npairs), (size_t)n * 4) == hipSuccess &&
        hipMalloc(reinterpret_cast<void**>(&s.offsets), (size_t)n * 4) == hipSuccess &&
        hipMalloc(reinterpret_cast<void**>(&s.ctx_raw), (size_t)(pairs ? pairs : 1) * 4) == hipSuccess &&
        hipMalloc(reinterpret_cast<void**>(&s.keys), (size_t)(pairs ? pairs : 1) * 4) == hipSuccess &&
        hipMalloc(reinterpret_cast<void**>(&s.keys_sorted), (size_t)(pairs ? pairs : 1) * 4) == hipSuccess &&
        hipMalloc(&s.temp, temp ? temp : 1) == hipSuccess;
    if (!ok) {
      wm_free(s);
      return hipErrorOutOfMemory;
    }
    s.temp_bytes = temp;
    s.n_cap = n;
    s.pair_cap = pairs;
  }
  *out = &s;
  return hipSuccess;
}

}  // namespace w2v

extern "C" int w2v_wordmats(int n, const int* mats, int iflip, int vocab, int nskip, int nneg,
                            int nreuse, float wsample_lnv, float wexpt, unsigned long long seed,
                            unsigned call, int* words, int* lb, int* ub, int* negs, int* ctx,
                            int* counts_dev, int* counts_host) {
  using namespace w2v;
  if (n < 0 || vocab <= 0 || nskip <= 0 || nneg <= 0 || nreuse <= 0 || !(wexpt < 1.0f) ||
      (long long)n * 2 * nskip > 0x7FFFFFF0LL)
    return (int)hipErrorInvalidValue;
  if (n > 0 && (!mats || !words || !lb || !ub || !negs || !ctx)) return (int)hipErrorInvalidValue;
  if (!counts_dev) return (int)hipErrorInvalidValue;
  hipStream_t stream = reinterpret_cast<hipStream_t>(w2v_get_stream());
  hipError_t err = hipSuccess;
  if (n == 0) {
    err = hipMemsetAsync(counts_dev, 0, 8, stream);
  } else {
    WordMatsScratch* s = nullptr;
    err = wm_scratch(n, nskip, &s);
    if (err != hipSuccess) return (int)err;
    const int wrow = iflip ? 1 : 0;
    const dim3 grid((unsigned)((n + kBlock - 1) / kBlock));
    hipLaunchKernelGGL(wm_words_kernel, grid, dim3(kBlock), 0, stream, n, mats, wrow, vocab,
                       wsample_lnv, call, seed, words);
    hipLaunchKernelGGL(wm_bounds_kernel, grid, dim3(kBlock), 0, stream, n, mats, wrow, words, nskip,
                       call, seed, lb, ub, s->npairs);
    size_t temp = s->temp_bytes;
    err = hipcub::DeviceScan::ExclusiveSum(s->temp, temp, s->npairs, s->offsets, n, stream);
    if (err != hipSuccess) return (int)err;
    hipLaunchKernelGGL(wm_counts_kernel, dim3(1), dim3(1), 0, stream, n, s->offsets, s->npairs,
                       nreuse, counts_dev);
    hipLaunchKernelGGL(wm_contexts_kernel, grid, dim3(kBlock), 0, stream, n, words, lb, ub,
                       s->offsets, call, seed, s->ctx_raw, s->keys);
    err = hipGetLastError();
  }
  if (err != hipSuccess) return (int)err;
  // the number of pairs sizes the sort and the caller's next call: one small read-back
  int counts[2] = {0, 0};
  err = hipMemcpyAsync(counts, counts_dev, 8, hipMemcpyDeviceToHost, stream);
  if (err != hipSuccess) return (int)err;
  err = hipStreamSynchronize(stream);
  if (err != hipSuccess) return (int)err;
  if (counts[0] > 0) {
    WordMatsScratch* s = nullptr;
    err = wm_scratch(n, nskip, &s);
    if (err != hipSuccess) return (int)err;
    size_t temp = s->temp_bytes;
    err = hipcub::DeviceRadixSort::SortPairs(s->temp, temp, s->keys, s->keys_sorted, s->ctx_raw,
                                             ctx, counts[0], 0, 32, stream);
    if (err != hipSuccess) return (int)err;
    const double expt = 1.0 / (1.0 - (double)wexpt);
    const int iexpt = (expt == floor(expt) && expt >= 1.0 && expt <= 16.0) ? (int)expt : 0;
    const long long nn = (long long)counts[1] * nneg;
    if (nn > 0) {
      const dim3 g2((unsigned)((nn + kBlock - 1) / kBlock));
      hipLaunchKernelGGL(wm_negatives_kernel, g2, dim3(kBlock), 0, stream, counts_dev, nneg, vocab,
                         expt, iexpt, call, seed, negs);
    }
    err = hipGetLastError();
    if (err != hipSuccess) return (int)err;
    err = hipStreamSynchronize(stream);
    if (err != hipSuccess) return (int)err;
  }
  if (counts_host) {
    counts_host[0] = counts[0];
    counts_host[1] = counts[1];
  }
  return 0;
}
