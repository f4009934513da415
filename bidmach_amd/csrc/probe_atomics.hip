// Device probe: what bounds a gather-dot-scatter over 1200-byte embedding columns on this GPU.
//
// Measures, for 12 M column touches (1.2 M work units x 10 columns, the shape of one negative
// pass at vocab 1M / dim 300), the time of
//   - gathering the columns,
//   - scattering into them with float atomics (lanes on consecutive floats; the same with the
//     lanes rotated so every instruction covers two whole 128-byte lines),
//   - gather followed by atomic scatter,
//   - a plain load-add-store of the same columns (no atomics),
// for ids drawn uniformly, from Zipf(1.0), and from the mix a negative pass sees (5 ids from
// unigram^0.75 + 5 from Zipf(1.0)); the latter also with the ids below 8 (below 1024) replaced by
// uniform ones (what a perfect spreading of the hot columns would give), with shadow copies of the
// 8 hottest columns that every reader sums ("exact"), and with shadow copies of the 16 hottest
// columns that writers fold into the table every 8th write while readers read the table only
// ("combining").
// Also a plain 1.2 GB copy as the streaming reference.  The library's design decisions (few,
// line-aligned atomics; LDS tiles; shadow copies) follow from these numbers.
//
// Build: python -m bidmach_amd.build   Run: bidmach_amd/lib/probe_atomics
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#define CK(x)                                                                  \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);    \
      exit(1);                                                                 \
    }                                                                          \
  } while (0)

constexpr int R = 5, D = 300, K = 10, HOT = 8, SHADOWS = 16;

enum Mode { kGather, kAtomic, kAtomicAligned, kGatherAtomicAligned, kLoadStore, kShadowed };

template <int MODE>
__global__ void __launch_bounds__(256)
touch(const int* __restrict__ ids, int nunits, float* T, float* S, float* sink) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long unit = (long)blockIdx.x * 4 + wave;
  if (unit >= nunits) return;
  const int mine = lane < K ? ids[unit * K + lane] : 0;
  float x[K][R];
  int id[K];
  float acc = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    id[k] = __builtin_amdgcn_readlane(mine, k);
#pragma unroll
    for (int r = 0; r < R; ++r) x[k][r] = 1e-3f;
    if (MODE == kGather || MODE == kGatherAtomicAligned || MODE == kLoadStore || MODE == kShadowed) {
      const float* col = T + (long)id[k] * D;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int e = r * 64 + lane;
        x[k][r] = e < D ? col[e] : 0.f;
      }
      if (MODE == kShadowed && id[k] < HOT) {
#pragma unroll 1
        for (int s = 0; s < SHADOWS; ++s) {
          const float* sc = S + ((long)s * HOT + id[k]) * D;
#pragma unroll
          for (int r = 0; r < R; ++r) {
            const int e = r * 64 + lane;
            x[k][r] += e < D ? sc[e] : 0.f;
          }
        }
      }
    }
  }
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float* col = T + (long)id[k] * D;
    if (MODE == kShadowed && id[k] < HOT) col = S + ((long)(blockIdx.x % SHADOWS) * HOT + id[k]) * D;
    if (MODE == kGather) {
#pragma unroll
      for (int r = 0; r < R; ++r) acc += x[k][r];
    } else if (MODE == kAtomic) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int e = r * 64 + lane;
        if (e < D) unsafeAtomicAdd(col + e, x[k][r] * 1e-9f);
      }
    } else if (MODE == kLoadStore) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int e = r * 64 + lane;
        if (e < D) col[e] = x[k][r] + 1e-9f;
      }
    } else {  // line-aligned atomics
      const int mis = (int)((reinterpret_cast<uintptr_t>(col) >> 2) & 31u);
#pragma unroll
      for (int r = 0; r <= R; ++r) {
        const int e = r * 64 + lane - mis;
        if (e >= 0 && e < D) unsafeAtomicAdd(col + e, x[k][r < R ? r : 0] * 1e-9f);
      }
    }
  }
  if (MODE == kGather && acc == 123.456f) sink[0] = acc;
}

constexpr int CHOT = 16, CSHADOWS = 32, FOLD_EVERY = 8, CSTRIDE = 32;

__device__ __forceinline__ int copies_of(int w) {
  const int c = CSHADOWS >> (31 - __builtin_clz(w + 1));
  return c < 2 ? 2 : c;
}

// Gather + line-aligned atomics; the atomics for ids below CHOT go to a shadow copy, and the writer
// that brings the copy's counter to a multiple of FOLD_EVERY swaps the copy out and adds it to the
// table column.  Persistent: workgroup b walks units [b*per_wg, (b+1)*per_wg).
__global__ void __launch_bounds__(256)
touch_combining(const int* __restrict__ ids, int nunits, long per_wg, float* T, float* S,
                unsigned* C) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long ubeg = (long)blockIdx.x * per_wg;
  const long uend = ubeg + per_wg < nunits ? ubeg + per_wg : nunits;
  for (long unit = ubeg + wave; unit < uend; unit += 4) {
    const int mine = lane < K ? ids[unit * K + lane] : 0;
    // lane k takes the ticket of column k's write now, so it is back when the write happens
    unsigned ticket = 0;
    if (lane < K && mine < CHOT) {
      const int slot = blockIdx.x & (copies_of(mine) - 1);
      ticket = __hip_atomic_fetch_add(C + ((long)slot * CHOT + mine) * CSTRIDE, 1u,
                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float x[K][R];
    int id[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      id[k] = __builtin_amdgcn_readlane(mine, k);
      const float* col = T + (long)id[k] * D;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int e = r * 64 + lane;
        x[k][r] = e < D ? col[e] : 0.f;
      }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      float* const tab = T + (long)id[k] * D;
      float* col = tab;
      const bool hot = id[k] < CHOT;
      if (hot) col = S + ((long)(blockIdx.x & (copies_of(id[k]) - 1)) * CHOT + id[k]) * D;
      const int mis = (int)((reinterpret_cast<uintptr_t>(col) >> 2) & 31u);
#pragma unroll
      for (int r = 0; r <= R; ++r) {
        const int e = r * 64 + lane - mis;
        if (e >= 0 && e < D) unsafeAtomicAdd(col + e, x[k][r < R ? r : 0] * 1e-9f);
      }
      if (hot) {
        const unsigned count = (unsigned)__builtin_amdgcn_readlane((int)ticket, k) + 1u;
        if ((count & (FOLD_EVERY - 1)) == 0) {
#pragma unroll
          for (int r = 0; r < R; ++r) {
            const int e = r * 64 + lane;
            if (e < D) {
              const float v = __hip_atomic_exchange(col + e, 0.0f, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
              if (v != 0.0f) unsafeAtomicAdd(tab + e, v);
            }
          }
        }
      }
    }
  }
}

static float run_combining(const int* ids, int nunits, float* T) {
  float* S;
  unsigned* C;
  CK(hipMalloc(&S, (size_t)CSHADOWS * CHOT * D * 4));
  CK(hipMemset(S, 0, (size_t)CSHADOWS * CHOT * D * 4));
  CK(hipMalloc(&C, (size_t)CSHADOWS * CHOT * CSTRIDE * 4));
  CK(hipMemset(C, 0, (size_t)CSHADOWS * CHOT * CSTRIDE * 4));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  const int nwg = 768;
  const long per_wg = ((long)nunits + nwg - 1) / nwg;
  hipLaunchKernelGGL(touch_combining, dim3(nwg), dim3(256), 0, 0, ids, nunits, per_wg, T, S, C);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  for (int i = 0; i < 3; ++i)
    hipLaunchKernelGGL(touch_combining, dim3(nwg), dim3(256), 0, 0, ids, nunits, per_wg, T, S, C);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, e0, e1));
  CK(hipFree(S));
  CK(hipFree(C));
  return ms / 3;
}

__global__ void copy_kernel(const float4* __restrict__ a, float4* __restrict__ b, long n) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) b[i] = a[i];
}

template <int MODE>
static float run(const int* ids, int nunits, float* T, float* S, float* sink) {
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  const dim3 grid((nunits + 3) / 4);
  hipLaunchKernelGGL((touch<MODE>), grid, dim3(256), 0, 0, ids, nunits, T, S, sink);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  for (int i = 0; i < 3; ++i)
    hipLaunchKernelGGL((touch<MODE>), grid, dim3(256), 0, 0, ids, nunits, T, S, sink);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, e0, e1));
  return ms / 3;
}

int main() {
  const int V = 1000000, NU = 1200000;
  const size_t table_bytes = (size_t)V * D * 4;
  float *T, *T2, *S, *sink;
  CK(hipMalloc(&T, table_bytes));
  CK(hipMalloc(&T2, table_bytes));
  CK(hipMemset(T, 0, table_bytes));
  CK(hipMalloc(&S, (size_t)SHADOWS * HOT * D * 4));
  CK(hipMemset(S, 0, (size_t)SHADOWS * HOT * D * 4));
  CK(hipMalloc(&sink, 4));

  std::mt19937_64 rng(1);
  std::uniform_real_distribution<double> U(0, 1);
  std::vector<double> zipf(V), neg(V);
  double s = 0, s2 = 0;
  for (int i = 0; i < V; ++i) {
    s += 1.0 / (i + 1);
    zipf[i] = s;
    s2 += std::pow(1.0 / (i + 1), 0.75);
    neg[i] = s2;
  }
  for (auto& c : zipf) c /= s;
  for (auto& c : neg) c /= s2;
  auto draw = [&](const std::vector<double>& cdf) {
    return std::min<int>(V - 1, std::lower_bound(cdf.begin(), cdf.end(), U(rng)) - cdf.begin());
  };
  const size_t n = (size_t)NU * K;
  std::vector<int> ids[3];
  for (auto& v : ids) v.resize(n);
  for (size_t i = 0; i < n; ++i) {
    ids[0][i] = (int)(U(rng) * V) % V;
    ids[1][i] = draw(zipf);
    ids[2][i] = (i % K) < 5 ? draw(neg) : draw(zipf);
  }
  const char* names[3] = {"uniform", "zipf(1.0)", "5 x unigram^0.75 + 5 x zipf(1.0)"};
  int* d_ids;
  CK(hipMalloc(&d_ids, n * 4));
  const double gb = (double)n * D * 4 / 1e9;
  printf("%.1f M column touches of %d bytes (%.1f GB per direction)\n", n / 1e6, D * 4, gb);
  for (int k = 0; k < 3; ++k) {
    CK(hipMemcpy(d_ids, ids[k].data(), n * 4, hipMemcpyHostToDevice));
    const float g = run<kGather>(d_ids, NU, T, S, sink);
    const float a = run<kAtomic>(d_ids, NU, T, S, sink);
    const float al = run<kAtomicAligned>(d_ids, NU, T, S, sink);
    const float ga = run<kGatherAtomicAligned>(d_ids, NU, T, S, sink);
    const float ls = run<kLoadStore>(d_ids, NU, T, S, sink);
    printf("%-34s gather %6.2f ms (%5.0f GB/s) | atomics %6.2f ms (%4.0f GB/s) | aligned atomics "
           "%6.2f ms (%4.0f GB/s) | gather + aligned atomics %6.2f ms | load-add-store %6.2f ms\n",
           names[k], g, gb / g * 1e3, a, gb / a * 1e3, al, gb / al * 1e3, ga, ls);
    if (k == 2) {
      const float sh = run<kShadowed>(d_ids, NU, T, S, sink);
      printf("%-34s gather + aligned atomics, exact shadows (%d copies of the %d hottest columns, "
             "readers sum them) %6.2f ms\n", names[k], SHADOWS, HOT, sh);
      const float cb = run_combining(d_ids, NU, T);
      printf("%-34s gather + aligned atomics, combining shadows (%d hottest columns, folded "
             "every %d writes, readers read the table) %6.2f ms\n", names[k], CHOT, FOLD_EVERY, cb);
      for (int H : {8, 1024}) {
        std::vector<int> spread(ids[2]);
        for (auto& v : spread)
          if (v < H) v = (int)(U(rng) * V) % V;
        CK(hipMemcpy(d_ids, spread.data(), n * 4, hipMemcpyHostToDevice));
        const float ga2 = run<kGatherAtomicAligned>(d_ids, NU, T, S, sink);
        printf("%-34s gather + aligned atomics with the ids below %d made uniform %6.2f ms\n",
               names[k], H, ga2);
      }
    }
    fflush(stdout);
  }
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  copy_kernel<<<4096, 256>>>((const float4*)T, (float4*)T2, table_bytes / 16);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  for (int i = 0; i < 5; ++i)
    copy_kernel<<<4096, 256>>>((const float4*)T, (float4*)T2, table_bytes / 16);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, e0, e1));
  ms /= 5;
  printf("streaming copy of %.1f GB: %.3f ms, %.0f GB/s read + write\n", table_bytes / 1e9, ms,
         2.0 * table_bytes / ms / 1e6);
  return 0;
}
