// C ABI of the SGNS library: argument checks, per-thread stream and Eval scratch, launch,
// and the synchronous/asynchronous forms of the four operators.
#include "../../include/bidmach_w2v.h"

#include <atomic>
#include <cstring>

#include "w2v_bf16.h"
#include "w2v_internal.h"

namespace {

constexpr int kMaxDevices = 64;
constexpr int kNoIdLimit = 0x7FFFFFFF;

struct ThreadState {
  // The stream the calling thread's launches go to: the caller's (w2v_set_stream), else a stream
  // of the thread's own per device, created on its first call there.  The reference library is
  // built with --default-stream per-thread (jni/src/configure:158,196): every JVM thread launches
  // on a stream of its own that still orders with the legacy default stream, so two learner
  // threads overlap on the device.  hipStreamCreate's default flags give exactly that kind of
  // stream (blocking with respect to the null stream, default priority).
  hipStream_t user = nullptr;
  bool user_set = false;
  hipStream_t own[kMaxDevices] = {};
  double* partials[kMaxDevices] = {};
  int64_t capacity[kMaxDevices] = {};
  float* shadow[kMaxDevices] = {};  // two shadow buffers (A then B), zero between calls
  float* side16[kMaxDevices] = {};  // fp32 side buffers of the bf16 tables' frequent words
  size_t side16_floats[kMaxDevices] = {};
};

thread_local ThreadState t_state;

// create == false: never creates a stream (for the entry point that may not allocate): the
// thread's own stream if it exists already, else the legacy default stream.
hipStream_t launch_stream(bool create = true) {
  ThreadState& ts = t_state;
  if (ts.user_set) return ts.user;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  if (ts.own[dev] == nullptr && create) {
    hipStream_t s = nullptr;
    if (hipStreamCreate(&s) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;   // the legacy default stream still works
    }
    ts.own[dev] = s;
  }
  return ts.own[dev];
}

std::atomic<double> g_eval_floor{1.0e-40};
std::atomic<int> g_bf16_hot_words{1024};
constexpr int kMaxBf16HotWords = 4096;
constexpr int kMaxNwbBf16 = 64;   // a lane per B word, as for the fp32 tables

// Per-thread, per-device fp32 side buffers for the frequent words of bf16 tables (A's then B's),
// zeroed when allocated; the update launchers leave them zeroed.  They only grow.
hipError_t side_buffers(int nrows, w2v::HotCols* out) {
  const int n = g_bf16_hot_words.load();
  out->n = n;
  out->sa = out->sb = nullptr;
  if (n == 0) return hipSuccess;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  ThreadState& ts = t_state;
  const size_t need = (size_t)2 * w2v::side_columns(n) * w2v::side_stride(nrows);
  if (ts.side16_floats[dev] < need) {
    if (ts.side16[dev] != nullptr) {
      err = hipStreamSynchronize(launch_stream());
      if (err != hipSuccess) return err;
      err = hipFree(ts.side16[dev]);
      ts.side16[dev] = nullptr;
      ts.side16_floats[dev] = 0;
      if (err != hipSuccess) return err;
    }
    float* p = nullptr;
    err = hipMalloc(reinterpret_cast<void**>(&p), need * sizeof(float));
    if (err != hipSuccess) return err;
    err = hipMemsetAsync(p, 0, need * sizeof(float), launch_stream());
    if (err == hipSuccess) err = hipStreamSynchronize(launch_stream());
    if (err != hipSuccess) {
      (void)hipFree(p);
      return err;
    }
    ts.side16[dev] = p;
    ts.side16_floats[dev] = need;
  }
  out->sa = ts.side16[dev];
  out->sb = ts.side16[dev] + (size_t)w2v::side_columns(n) * w2v::side_stride(nrows);
  return hipSuccess;
}

// Per-thread, per-device buffer of per-block partial sums for the Eval kernels.  It only grows.
hipError_t eval_scratch(int64_t need, double** out) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  ThreadState& ts = t_state;
  if (ts.capacity[dev] < need) {
    if (ts.partials[dev] != nullptr) {
      err = hipStreamSynchronize(launch_stream());
      if (err != hipSuccess) return err;
      err = hipFree(ts.partials[dev]);
      ts.partials[dev] = nullptr;
      ts.capacity[dev] = 0;
      if (err != hipSuccess) return err;
    }
    int64_t cap = 4096;
    while (cap < need) cap *= 2;
    err = hipMalloc(reinterpret_cast<void**>(&ts.partials[dev]), (size_t)cap * sizeof(double));
    if (err != hipSuccess) {
      ts.partials[dev] = nullptr;
      return err;
    }
    ts.capacity[dev] = cap;
  }
  *out = ts.partials[dev];
  return hipSuccess;
}

// Per-thread, per-device shadow buffers for the hot columns and their write counters, allocated
// and zeroed on first use: [shadow of A | shadow of B | counters | word occurrence counts | read
// copies of A | read copies of B].
hipError_t shadow_buffers(w2v::Shadow* out) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  ThreadState& ts = t_state;
  const size_t bytes = w2v::shadow_bytes();
  if (ts.shadow[dev] == nullptr) {
    float* p = nullptr;
    const size_t total = 2 * bytes + w2v::shadow_counter_bytes() + w2v::occurs_bytes() +
                         2 * w2v::read_copy_bytes();
    err = hipMalloc(reinterpret_cast<void**>(&p), total);
    if (err != hipSuccess) return err;
    err = hipMemsetAsync(p, 0, total, launch_stream());
    if (err == hipSuccess) err = hipStreamSynchronize(launch_stream());  // the stream may change later
    if (err != hipSuccess) {
      (void)hipFree(p);
      return err;
    }
    ts.shadow[dev] = p;
  }
  out->a = ts.shadow[dev];
  out->b = ts.shadow[dev] + bytes / sizeof(float);
  out->count = reinterpret_cast<unsigned*>(ts.shadow[dev] + 2 * (bytes / sizeof(float)));
  out->hot_seen = reinterpret_cast<int*>(out->count + (size_t)2 * w2v::kShadows * w2v::kHotWords *
                                                          w2v::kCounterStride);
  out->occurs = reinterpret_cast<int*>(reinterpret_cast<char*>(out->count) +
                                       w2v::shadow_counter_bytes());
  out->rare_max = 0;
  out->hot_mask = out->hot_seen + 4 * w2v::kHotCountSlots;
  out->pub_a = reinterpret_cast<float*>(reinterpret_cast<char*>(out->occurs) + w2v::occurs_bytes());
  out->pub_b = out->pub_a + w2v::read_copy_bytes() / sizeof(float);
  out->xcc = 0;
  out->hot_total = 0;
  out->hot_total_a = 0;
  out->combine = 0;
  out->combine_a = 0;
  return hipSuccess;
}

// any_rows: the operator has a kernel for columns of any length (w2v_any_shape.hip)
bool bad_common(int nrows, int ncols, bool any_rows = false) {
  return nrows <= 0 || (!any_rows && nrows > w2v::max_rows()) || ncols < 0;
}

// Whether a negative-pass shape goes to the any-shape kernels: columns longer than a wave holds
// in registers, more B words than a wave has lanes, or a wide group whose A columns do not fit
// in LDS.
bool neg_needs_any(int nrows, int nwa, int nwb) {
  return nrows > w2v::max_rows() || nwb > w2v::max_nwb() ||
         (nwb > 8 && !w2v::neg_wide_fits(nrows, nwa));
}

int finish(hipError_t launch_err, bool sync) {
  if (launch_err != hipSuccess) return (int)launch_err;
  if (sync) {
    hipError_t err = hipStreamSynchronize(launch_stream());
    if (err != hipSuccess) return (int)err;
    return (int)hipGetLastError();
  }
  return 0;
}

int pos_impl(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float* A, float* B,
             float lrate, float vexp, bool sync) {
  if (bad_common(nrows, ncols, true)) return (int)hipErrorInvalidValue;
  if (ncols == 0) return 0;
  if (!W || !LB || !UB || !A || !B) return (int)hipErrorInvalidValue;
  if (nrows > w2v::max_rows())
    return finish(w2v::launch_pos_any(launch_stream(), nrows, ncols, W, LB, UB, A, B, lrate, vexp),
                  sync);
  w2v::Shadow shadow{};
  hipError_t err = shadow_buffers(&shadow);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_pos(launch_stream(), nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp,
                                shadow),
                sync);
}

int neg_impl(int nrows, int ncols, int idlimit, int nwa, int nwb, int* WA, int* WB, float* A,
             float* B, float lrate, float vexp, bool sync) {
  if (bad_common(nrows, ncols, true) || nwa < 0 || nwb < 0 || idlimit < 0)
    return (int)hipErrorInvalidValue;
  if (ncols == 0 || nwa == 0 || nwb == 0) return 0;
  if (!WA || !WB || !A || !B) return (int)hipErrorInvalidValue;
  if (neg_needs_any(nrows, nwa, nwb)) {
    if (!w2v::neg_any_fits(nwa, nwb)) return (int)hipErrorInvalidValue;
    return finish(w2v::launch_neg_any(launch_stream(), nrows, ncols, idlimit, nwa, nwb, WA, WB, A,
                                      B, lrate, vexp),
                  sync);
  }
  w2v::Shadow shadow{};
  hipError_t err = shadow_buffers(&shadow);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_neg(launch_stream(), nrows, ncols, idlimit, nwa, nwb, WA, WB, A, B,
                                lrate, vexp, shadow),
                sync);
}

int eval_pos_impl(int nrows, int ncols, int* W, int* LB, int* UB, float* A, float* B, float* r32,
                  double* r64, bool sync) {
  if (bad_common(nrows, ncols, true) || (!r32 && !r64)) return (int)hipErrorInvalidValue;
  if (ncols == 0) return 0;
  if (!W || !LB || !UB || !A || !B) return (int)hipErrorInvalidValue;
  double* partials = nullptr;
  hipError_t err = eval_scratch(w2v::eval_partials_needed(ncols), &partials);
  if (err != hipSuccess) return (int)err;
  if (nrows > w2v::max_rows())
    return finish(w2v::launch_eval_pos_any(launch_stream(), nrows, ncols, W, LB, UB, A, B,
                                           g_eval_floor.load(), partials, r32, r64),
                  sync);
  return finish(w2v::launch_eval_pos(launch_stream(), nrows, ncols, W, LB, UB, A, B,
                                     g_eval_floor.load(), partials, r32, r64),
                sync);
}

int eval_neg_impl(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float* A, float* B,
                  float* r32, double* r64, bool sync) {
  if (bad_common(nrows, ncols, true) || nwa < 0 || nwb < 0 || (!r32 && !r64))
    return (int)hipErrorInvalidValue;
  if (ncols == 0 || nwa == 0 || nwb == 0) return 0;
  if (!WA || !WB || !A || !B) return (int)hipErrorInvalidValue;
  double* partials = nullptr;
  hipError_t err = eval_scratch(w2v::eval_partials_needed(ncols), &partials);
  if (err != hipSuccess) return (int)err;
  // (the forward kernels tile over the B words, so only long columns and more than 64 B words
  // need the any-shape kernel)
  if (nrows > w2v::max_rows() || nwb > w2v::max_nwb())
    return finish(w2v::launch_eval_neg_any(launch_stream(), nrows, ncols, nwa, nwb, WA, WB, A, B,
                                           g_eval_floor.load(), partials, r32, r64, 0),
                  sync);
  return finish(w2v::launch_eval_neg(launch_stream(), nrows, ncols, nwa, nwb, WA, WB, A, B,
                                     g_eval_floor.load(), partials, r32, r64),
                sync);
}

// Checks the slicing arguments and gathers the model-matrix pointers the kernels may touch.
// With dualMode the first pair of MM belongs to the device half of a dual-mode model
// (Word2Vec.scala:118-131 of the reference) and the parts start at MM[2].
bool slice_map(float** MM, int nmats, int islice, int nslices, int maxCols, int nHead, int dualMode,
               int doHead, w2v::SliceMap* out) {
  const int offset = dualMode ? 1 : 0;
  if (!MM || nmats < 2 * (offset + 1) || (nmats & 1) || nslices < 1 || islice < 0 ||
      islice >= nslices || maxCols < 1 || nHead < 0 || doHead < 0)
    return false;
  const int nparts = nmats / 2 - offset;
  if (nparts > w2v::max_slice_parts()) return false;
  w2v::SliceMap m{};
  for (int k = 0; k < 2 * nparts; ++k) {
    m.mats[k] = MM[2 * offset + k];
    if (m.mats[k] == nullptr) return false;
  }
  m.nparts = nparts;
  m.islice = islice;
  m.nslices = nslices;
  m.nhead = nHead;
  m.maxcols = maxCols;
  m.dohead = doHead;
  *out = m;
  return true;
}

int pos_slice_impl(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float** MM, int nmats,
                   float lrate, float vexp, int islice, int nslices, int maxCols, int nHead,
                   int dualMode, int doHead) {
  w2v::SliceMap m;
  if (bad_common(nrows, ncols) ||
      !slice_map(MM, nmats, islice, nslices, maxCols, nHead, dualMode, doHead, &m))
    return (int)hipErrorInvalidValue;
  if (ncols == 0) return 0;
  if (!W || !LB || !UB) return (int)hipErrorInvalidValue;
  w2v::Shadow shadow{};
  hipError_t err = shadow_buffers(&shadow);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_slice_pos(launch_stream(), nrows, ncols, shift, W, LB, UB, m, lrate,
                                      vexp, shadow),
                true);
}

int neg_slice_impl(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float** MM, int nmats,
                   float lrate, float vexp, int islice, int nslices, int maxCols, int nHead,
                   int dualMode, int doHead) {
  w2v::SliceMap m;
  if (bad_common(nrows, ncols) || nwa < 0 || nwb < 0 || nwb > w2v::max_nwb() ||
      !slice_map(MM, nmats, islice, nslices, maxCols, nHead, dualMode, doHead, &m))
    return (int)hipErrorInvalidValue;
  if (ncols == 0 || nwa == 0 || nwb == 0) return 0;
  if (!WA || !WB) return (int)hipErrorInvalidValue;
  w2v::Shadow shadow{};
  hipError_t err = shadow_buffers(&shadow);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_slice_neg(launch_stream(), nrows, ncols, nwa, nwb, WA, WB, m, lrate,
                                      vexp, shadow),
                true);
}

int eval_pos_slice_impl(int nrows, int ncols, int* W, int* LB, int* UB, float** MM, int nmats,
                        int islice, int nslices, int maxCols, int nHead, int dualMode,
                        double* Retval) {
  w2v::SliceMap m;
  if (bad_common(nrows, ncols) || !Retval ||
      !slice_map(MM, nmats, islice, nslices, maxCols, nHead, dualMode, 0, &m))
    return (int)hipErrorInvalidValue;
  if (ncols == 0) return 0;
  if (!W || !LB || !UB) return (int)hipErrorInvalidValue;
  double* partials = nullptr;
  hipError_t err = eval_scratch(w2v::slice_eval_partials_needed(), &partials);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_slice_eval_pos(launch_stream(), nrows, ncols, W, LB, UB, m,
                                           g_eval_floor.load(), partials, nullptr, Retval),
                true);
}

int eval_neg_slice_impl(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float** MM,
                        int nmats, int islice, int nslices, int maxCols, int nHead, int dualMode,
                        double* Retval) {
  w2v::SliceMap m;
  if (bad_common(nrows, ncols) || nwa < 0 || nwb < 0 || nwb > w2v::max_nwb() || !Retval ||
      !slice_map(MM, nmats, islice, nslices, maxCols, nHead, dualMode, 0, &m))
    return (int)hipErrorInvalidValue;
  if (ncols == 0 || nwa == 0 || nwb == 0) return 0;
  if (!WA || !WB) return (int)hipErrorInvalidValue;
  double* partials = nullptr;
  hipError_t err = eval_scratch(w2v::slice_eval_partials_needed(), &partials);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_slice_eval_neg(launch_stream(), nrows, ncols, nwa, nwb, WA, WB, m,
                                           g_eval_floor.load(), partials, nullptr, Retval),
                true);
}

struct Timer {
  hipEvent_t start;
  hipEvent_t stop;
};

// ---- the entry point that allocates nothing ------------------------------------------------
//
// word2vecEvalNeg's kernels leave one partial sum per workgroup in a scratch buffer that a second
// kernel folds; the ordinary entry point takes that buffer from hipMalloc on a thread's first
// call.  word2vecEvalNegNoAlloc uses this array instead: device memory that is part of the loaded
// code object, 64 KB on every GPU the library runs on, for the life of the process.
constexpr int64_t kStaticPartials = 8192;
constexpr int kNoAllocMaxGroups = 1 << 24;
static __device__ __align__(256) double scratch[kStaticPartials];

// The array's device address, per device (each GPU holds its own copy at its own address).  In
// host code the name `scratch` is only a handle for hipGetSymbolAddress, never an address.
std::atomic<double*> g_scratch_ptr[kMaxDevices];

hipError_t static_scratch(double** out) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  double* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    // first call on this device, which is current: look the address up (threads that race here
    // all get the same answer)
    void* addr = nullptr;
    err = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return err;
    if (addr == nullptr) return hipErrorInvalidSymbol;
    p = static_cast<double*>(addr);
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return hipSuccess;
}

}  // namespace

extern "C" {

int word2vecPos(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float* A, float* B,
                float lrate, float vexp) {
  return pos_impl(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, true);
}

int word2vecNeg(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float* A, float* B,
                float lrate, float vexp) {
  return neg_impl(nrows, ncols, kNoIdLimit, nwa, nwb, WA, WB, A, B, lrate, vexp, true);
}

int word2vecNegFilt(int nrows, int ncols, int nwords, int nwa, int nwb, int* WA, int* WB, float* A,
                    float* B, float lrate, float vexp) {
  return neg_impl(nrows, ncols, nwords, nwa, nwb, WA, WB, A, B, lrate, vexp, true);
}

int word2vecPosSlice(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float** MM,
                     int nmats, float lrate, float vexp, int islice, int nslices, int maxCols,
                     int nHead, int dualMode, int doHead) {
  return pos_slice_impl(nrows, ncols, shift, W, LB, UB, MM, nmats, lrate, vexp, islice, nslices,
                        maxCols, nHead, dualMode, doHead);
}

int word2vecNegSlice(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float** MM,
                     int nmats, float lrate, float vexp, int islice, int nslices, int maxCols,
                     int nHead, int dualMode, int doHead) {
  return neg_slice_impl(nrows, ncols, nwa, nwb, WA, WB, MM, nmats, lrate, vexp, islice, nslices,
                        maxCols, nHead, dualMode, doHead);
}

int word2vecEvalPosSlice(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float** MM,
                         int nmats, int islice, int nslices, int maxCols, int nHead, int dualMode,
                         double* Retval) {
  (void)shift;
  return eval_pos_slice_impl(nrows, ncols, W, LB, UB, MM, nmats, islice, nslices, maxCols, nHead,
                             dualMode, Retval);
}

int word2vecEvalNegSlice(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float** MM,
                         int nmats, int islice, int nslices, int maxCols, int nHead, int dualMode,
                         double* Retval) {
  return eval_neg_slice_impl(nrows, ncols, nwa, nwb, WA, WB, MM, nmats, islice, nslices, maxCols,
                             nHead, dualMode, Retval);
}

int w2v_max_slice_parts(void) { return w2v::max_slice_parts(); }

int word2vecEvalPos(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float* A, float* B,
                    float* Retval) {
  (void)shift;
  return eval_pos_impl(nrows, ncols, W, LB, UB, A, B, Retval, nullptr, true);
}

int word2vecEvalNeg(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float* A, float* B,
                    float* Retval) {
  return eval_neg_impl(nrows, ncols, nwa, nwb, WA, WB, A, B, Retval, nullptr, true);
}

int word2vecEvalNegNoAlloc(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float* A,
                           float* B, float* Retval) {
  if (bad_common(nrows, ncols) || nwa < 0 || nwb < 0 || nwb > w2v::max_nwb() || !Retval)
    return (int)hipErrorInvalidValue;
  if (ncols > kNoAllocMaxGroups) return (int)hipErrorInvalidValue;   // beyond the stated maximum
  if (ncols == 0 || nwa == 0 || nwb == 0) return 0;
  if (!WA || !WB || !A || !B) return (int)hipErrorInvalidValue;
  double* partials = nullptr;
  hipError_t err = static_scratch(&partials);
  if (err != hipSuccess) return (int)err;
  // every workgroup overwrites its own partial sum and the fold reads only those: nothing in
  // the array has to start at zero.  The stream is the caller's, or the thread's own if an
  // earlier call created it, else the legacy default stream: none is created here.
  hipStream_t stream = launch_stream(false);
  hipError_t lerr = w2v::launch_eval_neg(stream, nrows, ncols, nwa, nwb, WA, WB, A, B,
                                         g_eval_floor.load(), partials, Retval, nullptr,
                                         kStaticPartials);
  if (lerr != hipSuccess) return (int)lerr;
  lerr = hipStreamSynchronize(stream);
  if (lerr != hipSuccess) return (int)lerr;
  return (int)hipGetLastError();
}

int w2v_no_alloc_max_groups(void) { return kNoAllocMaxGroups; }

int word2vecEvalPosF64(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float* A,
                       float* B, double* Retval) {
  (void)shift;
  return eval_pos_impl(nrows, ncols, W, LB, UB, A, B, nullptr, Retval, true);
}

int word2vecEvalNegF64(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float* A,
                       float* B, double* Retval) {
  return eval_neg_impl(nrows, ncols, nwa, nwb, WA, WB, A, B, nullptr, Retval, true);
}

int word2vecPosAsync(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float* A, float* B,
                     float lrate, float vexp) {
  return pos_impl(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, false);
}

int word2vecNegAsync(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float* A, float* B,
                     float lrate, float vexp) {
  return neg_impl(nrows, ncols, kNoIdLimit, nwa, nwb, WA, WB, A, B, lrate, vexp, false);
}

int word2vecEvalPosAsync(int nrows, int ncols, int shift, int* W, int* LB, int* UB, float* A,
                         float* B, float* Retval) {
  (void)shift;
  return eval_pos_impl(nrows, ncols, W, LB, UB, A, B, Retval, nullptr, false);
}

int word2vecEvalNegAsync(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, float* A,
                         float* B, float* Retval) {
  return eval_neg_impl(nrows, ncols, nwa, nwb, WA, WB, A, B, Retval, nullptr, false);
}

// ---- bfloat16 tables ------------------------------------------------------------------------

static int pos_bf16_impl(int nrows, int ncols, int shift, int* W, int* LB, int* UB,
                         unsigned short* A, unsigned short* B, float lrate, float vexp,
                         unsigned long long seed, bool sync) {
  if (bad_common(nrows, ncols)) return (int)hipErrorInvalidValue;
  if (ncols == 0) return 0;
  if (!W || !LB || !UB || !A || !B) return (int)hipErrorInvalidValue;
  w2v::HotCols hot{};
  hipError_t err = side_buffers(nrows, &hot);
  if (err != hipSuccess) return (int)err;
  w2v::Shadow shadow{};   // for its hot-word counters: the launch may run in its ordered form
  err = shadow_buffers(&shadow);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_pos_bf16(launch_stream(), nrows, ncols, shift, W, LB, UB, A, B, lrate,
                                     vexp, seed, hot, shadow),
                sync);
}

int word2vecPosBf16(int nrows, int ncols, int shift, int* W, int* LB, int* UB, unsigned short* A,
                    unsigned short* B, float lrate, float vexp, unsigned long long seed) {
  return pos_bf16_impl(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, seed, true);
}

int word2vecPosBf16Async(int nrows, int ncols, int shift, int* W, int* LB, int* UB,
                         unsigned short* A, unsigned short* B, float lrate, float vexp,
                         unsigned long long seed) {
  return pos_bf16_impl(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, seed, false);
}

static int neg_bf16_impl(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB,
                         unsigned short* A, unsigned short* B, float lrate, float vexp,
                         unsigned long long seed, bool sync) {
  if (bad_common(nrows, ncols) || nwa < 0 || nwb < 0 || nwb > kMaxNwbBf16)
    return (int)hipErrorInvalidValue;
  if (ncols == 0 || nwa == 0 || nwb == 0) return 0;
  if (!WA || !WB || !A || !B) return (int)hipErrorInvalidValue;
  w2v::HotCols hot{};
  hipError_t err = side_buffers(nrows, &hot);
  if (err != hipSuccess) return (int)err;
  w2v::Shadow shadow{};
  err = shadow_buffers(&shadow);
  if (err != hipSuccess) return (int)err;
  return finish(w2v::launch_neg_bf16(launch_stream(), nrows, ncols, nwa, nwb, WA, WB, A, B, lrate,
                                     vexp, seed, hot, shadow),
                sync);
}

int word2vecNegBf16(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB, unsigned short* A,
                    unsigned short* B, float lrate, float vexp, unsigned long long seed) {
  return neg_bf16_impl(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, true);
}

int word2vecNegBf16Async(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB,
                         unsigned short* A, unsigned short* B, float lrate, float vexp,
                         unsigned long long seed) {
  return neg_bf16_impl(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, false);
}

int word2vecEvalPosBf16(int nrows, int ncols, int shift, int* W, int* LB, int* UB,
                        unsigned short* A, unsigned short* B, double* Retval) {
  (void)shift;
  if (bad_common(nrows, ncols) || !Retval) return (int)hipErrorInvalidValue;
  if (ncols == 0) return 0;
  if (!W || !LB || !UB || !A || !B) return (int)hipErrorInvalidValue;
  return finish(w2v::launch_eval_pos_bf16(launch_stream(), nrows, ncols, W, LB, UB, A, B,
                                          g_eval_floor.load(), Retval),
                true);
}

int word2vecEvalNegBf16(int nrows, int ncols, int nwa, int nwb, int* WA, int* WB,
                        unsigned short* A, unsigned short* B, double* Retval) {
  if (bad_common(nrows, ncols) || nwa < 0 || nwb < 0 || nwb > kMaxNwbBf16 || !Retval)
    return (int)hipErrorInvalidValue;
  if (ncols == 0 || nwa == 0 || nwb == 0) return 0;
  if (!WA || !WB || !A || !B) return (int)hipErrorInvalidValue;
  return finish(w2v::launch_eval_neg_bf16(launch_stream(), nrows, ncols, nwa, nwb, WA, WB, A, B,
                                          g_eval_floor.load(), Retval),
                true);
}

int w2v_set_bf16_hot_words(int n) {
  if (n < 0 || n > kMaxBf16HotWords) return (int)hipErrorInvalidValue;
  g_bf16_hot_words.store(n);
  return 0;
}
int w2v_get_bf16_hot_words(void) { return g_bf16_hot_words.load(); }

int w2v_f32_to_bf16(size_t n, const float* src, unsigned short* dst) {
  if (n == 0) return 0;
  if (!src || !dst) return (int)hipErrorInvalidValue;
  return finish(w2v::launch_f32_to_bf16(launch_stream(), n, src, dst), true);
}

int w2v_bf16_to_f32(size_t n, const unsigned short* src, float* dst) {
  if (n == 0) return 0;
  if (!src || !dst) return (int)hipErrorInvalidValue;
  return finish(w2v::launch_bf16_to_f32(launch_stream(), n, src, dst), true);
}

void w2v_set_eval_floor(double floor_value) { g_eval_floor.store(floor_value); }
double w2v_get_eval_floor(void) { return g_eval_floor.load(); }

int w2v_set_stream(void* stream) {
  t_state.user = reinterpret_cast<hipStream_t>(stream);
  t_state.user_set = true;
  return 0;
}
int w2v_reset_stream(void) {
  t_state.user = nullptr;
  t_state.user_set = false;
  return 0;
}
void* w2v_get_stream(void) { return reinterpret_cast<void*>(launch_stream()); }
int w2v_synchronize(void) { return (int)hipStreamSynchronize(launch_stream()); }

int w2v_release_thread(void) {
  ThreadState& ts = t_state;
  bool held = false;
  for (int dev = 0; dev < kMaxDevices; ++dev)
    held = held || ts.partials[dev] || ts.shadow[dev] || ts.side16[dev] || ts.own[dev];
  if (!held) return 0;
  hipError_t first = hipStreamSynchronize(launch_stream(false));   // nothing may still be using the scratch
  for (int dev = 0; dev < kMaxDevices; ++dev) {
    if (ts.own[dev] != nullptr) {
      hipError_t err = hipStreamSynchronize(ts.own[dev]);
      if (err == hipSuccess) err = hipStreamDestroy(ts.own[dev]);
      if (first == hipSuccess) first = err;
      ts.own[dev] = nullptr;
    }
  }
  auto release = [&first](auto*& p) {
    if (p != nullptr) {
      const hipError_t err = hipFree(p);
      if (first == hipSuccess) first = err;
      p = nullptr;
    }
  };
  for (int dev = 0; dev < kMaxDevices; ++dev) {
    release(ts.partials[dev]);
    ts.capacity[dev] = 0;
    release(ts.shadow[dev]);
    release(ts.side16[dev]);
    ts.side16_floats[dev] = 0;
  }
  return (int)first;
}

int w2v_set_max_workgroups(int n) {
  w2v::set_max_workgroups(n);
  return 0;
}
int w2v_get_max_workgroups(void) { return w2v::get_max_workgroups(); }

int w2v_set_ordered_mode(int mode) {
  w2v::set_ordered_mode(mode);
  return 0;
}
int w2v_get_ordered_mode(void) { return w2v::get_ordered_mode(); }

int w2v_last_launch_form(void) {
  const w2v::Shadow* sh = w2v::last_launch_shadow();
  if (sh == nullptr) return -1;
  if (sh->ordered == 2) return 1;
  if (sh->ordered == 0 || sh->hot_total <= 0 || sh->hot_seen == nullptr) return 0;
  // the counts the kernels of that launch looked at (launch_is_ordered, w2v_device.h)
  hipStream_t stream = launch_stream(false);
  int seen[4 * w2v::kHotCountSlots];
  hipError_t err = hipMemcpyAsync(seen, sh->hot_seen, sizeof(seen), hipMemcpyDeviceToHost, stream);
  if (err == hipSuccess) err = hipStreamSynchronize(stream);
  if (err != hipSuccess) return -1;
  long long sum[4] = {0, 0, 0, 0};
  for (int t = 0; t < 4; ++t)
    for (int k = 0; k < w2v::kHotCountSlots; ++k) sum[t] += seen[t * w2v::kHotCountSlots + k];
  const bool hot_b = w2v::ids_are_hot(sum[0], sum[1], sh->hot_total);
  const bool hot_a =
      sh->hot_total_a > 0 ? w2v::ids_are_hot(sum[2], sum[3], sh->hot_total_a) : hot_b;
  return (hot_a || hot_b) ? 1 : 0;
}
int w2v_set_ordered_workers(int pos_workers, int neg_workers) {
  if (pos_workers < 0 || neg_workers < 0) return (int)hipErrorInvalidValue;
  w2v::set_ordered_workers(pos_workers, neg_workers);
  return 0;
}

int w2v_set_ordered_copies(int copies, int twins) {
  if (copies < 0 || copies > w2v::kGridMaxC || twins < 1 || copies * twins > w2v::kShadows)
    return (int)hipErrorInvalidValue;
  w2v::set_ordered_copies(copies, twins);
  return 0;
}

int w2v_set_rare_update_mode(int mode) {
  w2v::set_rare_update_mode(mode);
  return 0;
}
int w2v_get_rare_update_mode(void) { return w2v::get_rare_update_mode(); }

int w2v_set_hot_update_mode(int mode) {
  w2v::set_hot_update_mode(mode);
  return 0;
}
int w2v_get_hot_update_mode(void) { return w2v::get_hot_update_mode(); }

int w2v_max_rows(void) { return w2v::max_rows(); }
int w2v_max_nwb(void) { return w2v::max_nwb(); }

int w2v_malloc(void** dev_ptr, size_t bytes) {
  if (!dev_ptr) return (int)hipErrorInvalidValue;
  return (int)hipMalloc(dev_ptr, bytes);
}
int w2v_free(void* dev_ptr) { return (int)hipFree(dev_ptr); }
int w2v_memcpy_h2d(void* dev_dst, const void* host_src, size_t bytes) {
  hipError_t err = hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice, launch_stream());
  if (err != hipSuccess) return (int)err;
  return (int)hipStreamSynchronize(launch_stream());
}
int w2v_memcpy_d2h(void* host_dst, const void* dev_src, size_t bytes) {
  hipError_t err = hipMemcpyAsync(host_dst, dev_src, bytes, hipMemcpyDeviceToHost, launch_stream());
  if (err != hipSuccess) return (int)err;
  return (int)hipStreamSynchronize(launch_stream());
}
int w2v_memset(void* dev_ptr, int value, size_t bytes) {
  hipError_t err = hipMemsetAsync(dev_ptr, value, bytes, launch_stream());
  if (err != hipSuccess) return (int)err;
  return (int)hipStreamSynchronize(launch_stream());
}

int w2v_timer_create(void** timer) {
  if (!timer) return (int)hipErrorInvalidValue;
  Timer* t = new (std::nothrow) Timer();
  if (!t) return (int)hipErrorOutOfMemory;
  hipError_t err = hipEventCreate(&t->start);
  if (err != hipSuccess) {
    delete t;
    return (int)err;
  }
  err = hipEventCreate(&t->stop);
  if (err != hipSuccess) {
    (void)hipEventDestroy(t->start);
    delete t;
    return (int)err;
  }
  *timer = t;
  return 0;
}
int w2v_timer_destroy(void* timer) {
  if (!timer) return 0;
  Timer* t = static_cast<Timer*>(timer);
  hipError_t e1 = hipEventDestroy(t->start);
  hipError_t e2 = hipEventDestroy(t->stop);
  delete t;
  return (int)(e1 != hipSuccess ? e1 : e2);
}
int w2v_timer_start(void* timer) {
  if (!timer) return (int)hipErrorInvalidValue;
  return (int)hipEventRecord(static_cast<Timer*>(timer)->start, launch_stream());
}
int w2v_timer_stop(void* timer) {
  if (!timer) return (int)hipErrorInvalidValue;
  return (int)hipEventRecord(static_cast<Timer*>(timer)->stop, launch_stream());
}
int w2v_timer_elapsed_ms(void* timer, float* ms) {
  if (!timer || !ms) return (int)hipErrorInvalidValue;
  Timer* t = static_cast<Timer*>(timer);
  hipError_t err = hipEventSynchronize(t->stop);
  if (err != hipSuccess) return (int)err;
  return (int)hipEventElapsedTime(ms, t->start, t->stop);
}

const char* w2v_error_string(int err) { return hipGetErrorString((hipError_t)err); }

}  // extern "C"
