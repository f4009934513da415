// The ordered negative pass on bfloat16 tables (w2v_bf16_neg_rows.h): the instances for tables on
// 2-byte boundaries or with an odd number of rows, a translation unit of their own so that the
// two sets compile side by side.
#include "w2v_bf16_neg_rows.h"

namespace w2v {

hipError_t launch_neg_rows_bf16_unaligned(hipStream_t stream, int nrows, int ncols, int nwa,
                                          int nwb, const int* WA, const int* WB, uint16_t* A,
                                          uint16_t* B, float lrate, float vexp, uint64_t seed,
                                          HotCols hot, int64_t chains, const Shadow& shadow) {
  return rows16::dispatch<false>(stream, nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed,
                                   hot, chains, shadow);
}

}  // namespace w2v
