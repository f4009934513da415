/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU statement of the reduced-precision storage variant of the skip-gram negative-sampling
 * functions: the same loop nests as oracle_word2vecPos / Neg / EvalPos / EvalNeg in
 * w2v_oracle.c (which follow jni/src/BIDMach_CPUMACH.c:10-78, :186-264, :368-427, :429-483 of the
 * reference), with both tables stored as bfloat16.  The reference has no such variant; what is
 * kept from it is the arithmetic between a load and a store: every column is widened to fp32
 * when it is read, dots, sigmoid, scales and deltas are the fp32 (double inside exp / pow / log)
 * expressions of the reference, and a column is narrowed again only when it is written back.
 *
 * Narrowing is stochastic rounding with a counter-based generator, so that the HIP library and
 * this file round every element with the same 16 random bits:
 *   key  = mix64(seed ^ mix64((unit << 32) | slot))         unit = token / group index of the call
 *   r16  = fmix32((uint32)(key >> 32) ^ (row * 0x9E3779B9)) >> 16
 *   bf16 = (bits(x) + r16) >> 16                             (magnitude rounds up with
 *                                                             probability low16(x) / 65536)
 * slot names the write inside the unit: positive pass, context at offset j: (uint32)j, centre
 * column: 0; negative pass, B column k: k, A column j: 0x10000 + j.  The columns of the first
 * hot_n words go through an fp32 side buffer and are narrowed once, at the end of the call (see
 * bf16_fold below), as the HIP library does for the words it treats as frequent.
 *
 * Parity pins (tests/test_oracle_bf16.py): the narrowing returns one of the two bfloat16
 * neighbours of its argument, is exact on representable values, and picks the upper neighbour
 * with probability equal to the dropped fraction (over rows and over keys); keys differ between
 * units, slots and seeds; the forward sums equal the fp32 oracle's on the widened tables bit for
 * bit; on collision-free minibatches every stored element is one of the two neighbours of the
 * fp32 oracle's result, with and without side buffers, and untouched columns keep their bits; the
 * mean over 400 seeds approaches the fp32 result as 1/sqrt(n); with every word routed through the
 * side buffers a colliding Zipf minibatch ends within one bfloat16 step of the sequential fp32
 * run.  The reference has no reduced-precision variant, so none of its files can pin this one.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_oracle_sigmoid(float cv) {
  /* BIDMach_CPUMACH.c:48-55 */
  if (cv > 16.0f) {
    cv = 1.0f;
  } else if (cv < -16.0f) {
    cv = 0.0f;
  } else {
    cv = exp(cv);
    cv = cv / (1.0f + cv);
  }
  return cv;
}

static inline float bf16_widen(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint64_t bf16_mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ULL;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

static inline uint32_t bf16_fmix32(uint32_t h) {
  h ^= h >> 16;
  h *= 0x85EBCA6BU;
  h ^= h >> 13;
  h *= 0xC2B2AE35U;
  h ^= h >> 16;
  return h;
}

uint32_t oracle_bf16_key(uint64_t seed, uint32_t unit, uint32_t slot) {
  return (uint32_t)(bf16_mix64(seed ^ bf16_mix64(((uint64_t)unit << 32) | slot)) >> 32);
}

uint16_t oracle_bf16_narrow(float x, uint32_t key, uint32_t row) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if ((u & 0x7F800000U) == 0x7F800000U) /* infinity or NaN: keep the class */
    return (uint16_t)((u >> 16) | ((u & 0x007FFFFFU) ? 0x40U : 0U));
  return (uint16_t)((u + (bf16_fmix32(key ^ (row * 0x9E3779B9U)) >> 16)) >> 16);
}

/* Frequent words (ids below hot_n): during a call their columns are table + an fp32 side buffer;
 * reads add the two in fp32, writes add the delta to the side buffer, and the end of the call
 * narrows the sum back into the table with one rounding per element (unit 0xFFFFFFFF, slot
 * (table << 31) | word; table 0 = A, 1 = B).  Elements whose side buffer is zero are left alone. */
static float *bf16_side_alloc(int hot_n, int nrows) {
  return (float *)calloc((size_t)(hot_n > 0 ? hot_n : 1) * nrows, sizeof(float));
}

static inline float bf16_read(const uint16_t *T, const float *side, int hot_n, int word,
                              int64_t off, int nrows, int c) {
  float v = bf16_widen(T[c + off]);
  if (word < hot_n) v += side[(int64_t)word * nrows + c];
  return v;
}

static void bf16_fold(uint16_t *T, float *side, int hot_n, int nrows, uint64_t seed, int table) {
  int w, c;
  for (w = 0; w < hot_n; w++) {
    uint32_t key = oracle_bf16_key(seed, 0xFFFFFFFFU, ((uint32_t)table << 31) | (uint32_t)w);
    for (c = 0; c < nrows; c++) {
      float v = side[(int64_t)w * nrows + c];
      if (v != 0.0f) {
        int64_t at = (int64_t)w * nrows + c;
        T[at] = oracle_bf16_narrow(bf16_widen(T[at]) + v, key, (uint32_t)c);
      }
    }
  }
}

void oracle_word2vecPosBf16(int nrows, int ncols, int skip, const int *W, const int *LB,
                            const int *UB, uint16_t *A, uint16_t *B, float lrate, float vexp,
                            uint64_t seed, int hot_n) {
  int i, j, c, wa, wb;
  int64_t ia, ib;
  float cv, ascale, bscale;
  float *daa = (float *)malloc((size_t)nrows * sizeof(float));
  float *sa = bf16_side_alloc(hot_n, nrows), *sb = bf16_side_alloc(hot_n, nrows);
  (void)skip;
  for (i = 0; i < ncols; i++) {
    wa = W[i];
    if (wa < 0) continue;
    ia = (int64_t)nrows * wa;
    ascale = pow(1 + wa, vexp);
    for (c = 0; c < nrows; c++) daa[c] = 0;
    for (j = LB[i]; j <= UB[i]; j++) {
      if (j != 0 && i + j >= 0 && i + j < ncols) {
        wb = W[i + j];
        if (wb >= 0) {
          uint32_t key = oracle_bf16_key(seed, (uint32_t)i, (uint32_t)j);
          ib = (int64_t)nrows * wb;
          bscale = pow(1 + wb, vexp);
          cv = 0;
          for (c = 0; c < nrows; c++)
            cv += bf16_read(A, sa, hot_n, wa, ia, nrows, c) * bf16_read(B, sb, hot_n, wb, ib, nrows, c);
          cv = bf16_oracle_sigmoid(cv);
          cv = lrate * (1.0f - cv);
          for (c = 0; c < nrows; c++) {
            float a = bf16_read(A, sa, hot_n, wa, ia, nrows, c);
            float b = bf16_read(B, sb, hot_n, wb, ib, nrows, c);
            float db = bscale * cv * a;
            daa[c] += ascale * cv * b;
            if (wb < hot_n)
              sb[(int64_t)wb * nrows + c] += db;
            else
              B[c + ib] = oracle_bf16_narrow(b + db, key, (uint32_t)c);
          }
        }
      }
    }
    {
      uint32_t key = oracle_bf16_key(seed, (uint32_t)i, 0U);
      for (c = 0; c < nrows; c++) {
        if (wa < hot_n)
          sa[(int64_t)wa * nrows + c] += daa[c];
        else
          A[c + ia] = oracle_bf16_narrow(bf16_widen(A[c + ia]) + daa[c], key, (uint32_t)c);
      }
    }
  }
  bf16_fold(A, sa, hot_n, nrows, seed, 0);
  bf16_fold(B, sb, hot_n, nrows, seed, 1);
  free(sb);
  free(sa);
  free(daa);
}

void oracle_word2vecNegBf16(int nrows, int ncols, int nwa, int nwb, const int *WA, const int *WB,
                            uint16_t *A, uint16_t *B, float lrate, float vexp, uint64_t seed,
                            int hot_n) {
  int i, j, k, c, wa, wb;
  int64_t ia, ib, ja;
  float cv, ascale, bscale;
  float *daa = (float *)malloc((size_t)(nwa > 0 ? nwa : 1) * nrows * sizeof(float));
  float *dbb = (float *)malloc((size_t)nrows * sizeof(float));
  float *sa = bf16_side_alloc(hot_n, nrows), *sb = bf16_side_alloc(hot_n, nrows);
  for (i = 0; i < ncols; i++) {
    for (c = 0; c < nwa * nrows; c++) daa[c] = 0;
    for (k = 0; k < nwb; k++) {
      uint32_t key = oracle_bf16_key(seed, (uint32_t)i, (uint32_t)k);
      wb = WB[k + (int64_t)i * nwb];
      if (wb < 0) continue; /* a dropped word skips its pairs, as in the fp32 library */
      ib = (int64_t)nrows * wb;
      bscale = pow(1 + wb, vexp);
      for (c = 0; c < nrows; c++) dbb[c] = 0;
      for (j = 0; j < nwa; j++) {
        wa = WA[j + (int64_t)i * nwa];
        if (wa < 0) continue;
        ia = (int64_t)nrows * wa;
        ascale = pow(1 + wa, vexp);
        cv = 0;
        for (c = 0; c < nrows; c++)
          cv += bf16_read(A, sa, hot_n, wa, ia, nrows, c) * bf16_read(B, sb, hot_n, wb, ib, nrows, c);
        cv = bf16_oracle_sigmoid(cv);
        cv = -lrate * cv;
        ja = (int64_t)j * nrows;
        for (c = 0; c < nrows; c++) {
          dbb[c] += bscale * cv * bf16_read(A, sa, hot_n, wa, ia, nrows, c);
          daa[c + ja] += ascale * cv * bf16_read(B, sb, hot_n, wb, ib, nrows, c);
        }
      }
      for (c = 0; c < nrows; c++) {
        if (wb < hot_n)
          sb[(int64_t)wb * nrows + c] += dbb[c];
        else
          B[c + ib] = oracle_bf16_narrow(bf16_widen(B[c + ib]) + dbb[c], key, (uint32_t)c);
      }
    }
    for (j = 0; j < nwa; j++) {
      uint32_t key = oracle_bf16_key(seed, (uint32_t)i, 0x10000U + (uint32_t)j);
      ja = (int64_t)j * nrows;
      wa = WA[j + (int64_t)i * nwa];
      if (wa < 0) continue;
      ia = (int64_t)nrows * wa;
      for (c = 0; c < nrows; c++) {
        if (wa < hot_n)
          sa[(int64_t)wa * nrows + c] += daa[c + ja];
        else
          A[c + ia] = oracle_bf16_narrow(bf16_widen(A[c + ia]) + daa[c + ja], key, (uint32_t)c);
      }
    }
  }
  bf16_fold(A, sa, hot_n, nrows, seed, 0);
  bf16_fold(B, sb, hot_n, nrows, seed, 1);
  free(sb);
  free(sa);
  free(dbb);
  free(daa);
}

double oracle_word2vecEvalPosBf16(int nrows, int ncols, int skip, const int *W, const int *LB,
                                  const int *UB, const uint16_t *A, const uint16_t *B,
                                  double floorv) {
  int ii, j, c;
  int64_t ia, ib;
  float cv;
  double dv = 0;
  (void)skip;
  for (ii = 0; ii < ncols; ii++) {
    if (W[ii] < 0) continue;
    ia = (int64_t)nrows * W[ii];
    for (j = LB[ii]; j <= UB[ii]; j++) {
      if (j != 0 && ii + j >= 0 && ii + j < ncols && W[ii + j] >= 0) {
        ib = (int64_t)nrows * W[ii + j];
        cv = 0;
        for (c = 0; c < nrows; c++) cv += bf16_widen(A[c + ia]) * bf16_widen(B[c + ib]);
        cv = bf16_oracle_sigmoid(cv);
        dv += log(fmax((double)cv, floorv));
      }
    }
  }
  return dv;
}

double oracle_word2vecEvalNegBf16(int nrows, int ncols, int nwa, int nwb, const int *WA,
                                  const int *WB, const uint16_t *A, const uint16_t *B,
                                  double floorv) {
  int ii, j, k, c;
  int64_t ia, ib;
  float cv;
  double dv = 0;
  for (ii = 0; ii < ncols; ii++) {
    for (k = 0; k < nwb; k++) {
      if (WB[k + (int64_t)ii * nwb] < 0) continue;
      ib = (int64_t)nrows * WB[k + (int64_t)ii * nwb];
      for (j = 0; j < nwa; j++) {
        if (WA[j + (int64_t)ii * nwa] < 0) continue;
        ia = (int64_t)nrows * WA[j + (int64_t)ii * nwa];
        cv = 0;
        for (c = 0; c < nrows; c++) cv += bf16_widen(A[c + ia]) * bf16_widen(B[c + ib]);
        cv = bf16_oracle_sigmoid(cv);
        dv += log(fmax(1.0 - (double)cv, floorv));
      }
    }
  }
  return dv;
}
