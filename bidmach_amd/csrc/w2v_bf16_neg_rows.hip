// The ordered negative pass on bfloat16 tables (w2v_bf16_neg_rows.h): the instances for tables
// whose columns start on 4-byte boundaries, and the entry points.
#include "w2v_bf16_neg_rows.h"

namespace w2v {

bool neg_rows_bf16_available(int nrows, int nwa) { return rows16::has_instance(nrows, nwa); }

hipError_t launch_neg_rows_bf16(hipStream_t stream, int nrows, int ncols, int nwa, int nwb,
                                const int* WA, const int* WB, uint16_t* A, uint16_t* B,
                                float lrate, float vexp, uint64_t seed, HotCols hot,
                                int64_t chains, const Shadow& shadow) {
  const bool aligned = (nrows & 1) == 0 && (reinterpret_cast<uintptr_t>(A) & 3) == 0 &&
                       (reinterpret_cast<uintptr_t>(B) & 3) == 0;
  if (aligned)
    return rows16::dispatch<true>(stream, nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp,
                                    seed, hot, chains, shadow);
  return launch_neg_rows_bf16_unaligned(stream, nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp,
                                        seed, hot, chains, shadow);
}

}  // namespace w2v
