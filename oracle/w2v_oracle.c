/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of BIDMach's CPUMACH skip-gram negative-sampling functions,
 * used as the parity oracle for the HIP library and as the timed host baseline.
 * Nothing in the shipped library links or calls this file.
 *
 * It follows jni/src/BIDMach_CPUMACH.c of the reference:
 *   oracle_word2vecPos      <- :10-78
 *   oracle_word2vecNeg      <- :186-264
 *   oracle_word2vecEvalPos  <- :368-427
 *   oracle_word2vecEvalNeg  <- :429-483
 *   oracle_word2vecNegFilt  <- the same arithmetic as word2vecNeg under the id filter of the
 *                              reference's GPU-only __word2vecNegFilt (jni/src/DNN127.cu:690-711):
 *                              a word id >= nwords drops every pair it takes part in
 *   oracle_word2vec{Pos,Neg}Slice     <- :80-184, :267-366 (multi-part, sliced model)
 *   oracle_word2vecEval{Pos,Neg}Slice <- the Scala-only forward twins,
 *                              src/main/scala/BIDMach/networks/Word2Vec.scala:1007-1069, :1134-1200
 * with the JNI array pinning replaced by plain pointers.  Arithmetic order is
 * kept (fp32 multiply then add in ascending row order, exp/pow/log in double,
 * B updated inside the window loop, A after it) so that a single-threaded run
 * defines the sequential result on colliding minibatches as well.
 *
 * Deliberate differences from the reference text:
 *   - column offsets are 64-bit and validity is tested on the word id (id >= 0)
 *     instead of on the 32-bit product nrows*id (:31-32); the two agree
 *     wherever the reference's product does not overflow;
 *   - the Eval accumulators start at zero; the reference leaves `double sum`
 *     uninitialised (:379, :439);
 *   - in the sliced variants the column inside a part is newi - (newi / maxCols) * maxCols; the
 *     reference subtracts (newi / maxCols + offset) * maxCols (:87), which with dualMode (offset 1)
 *     points maxCols columns before the start of the part;
 *   - the Eval floor is a parameter (the C reference uses 1e-40, the Scala and
 *     CUDA twins 1e-20: Word2Vec.scala:995,1123, DNN127.cu:310,916).
 *
 * Parity pins (tests/test_oracle.py): float64 closed forms on collision-free
 * minibatches, brute-force enumeration on tiny inputs, clamp and floor special
 * cases, no-op invariants, and two-pair analytic cases that fix the update
 * order (B immediate, A deferred).  The reference C file itself cannot be built
 * in this image (it needs jni.h, which is absent).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <omp.h>

static inline float oracle_sigmoid(float cv) {
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

void oracle_word2vecPos(int nrows, int ncols, int skip, const int *W, const int *LB, const int *UB,
                        float *A, float *B, float lrate, float vexp, int nthreads) {
  int ithread;
  (void)skip; /* unused on the CPU path, as in the reference (:11) */
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    int i, j, c, itmp;
    int64_t ia, ib;
    float cv, ascale, bscale;
    float *daa = (float *)malloc((size_t)nrows * sizeof(float));

    for (i = istart; i < iend; i++) {
      itmp = W[i];
      if (itmp >= 0) {
        ia = (int64_t)nrows * itmp;
        ascale = pow(1 + itmp, vexp);
        for (c = 0; c < nrows; c++) daa[c] = 0;
        for (j = LB[i]; j <= UB[i]; j++) {
          if (j != 0 && i + j >= 0 && i + j < ncols) {
            itmp = W[i + j];
            if (itmp >= 0) {
              ib = (int64_t)nrows * itmp;
              bscale = pow(1 + itmp, vexp);
              cv = 0;
              for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
              cv = oracle_sigmoid(cv);
              cv = lrate * (1.0f - cv);
              for (c = 0; c < nrows; c++) {
                daa[c] += ascale * cv * B[c + ib];
                B[c + ib] += bscale * cv * A[c + ia];
              }
            }
          }
        }
        for (c = 0; c < nrows; c++) A[c + ia] += daa[c];
      }
    }
    free(daa);
  }
}

void oracle_word2vecNeg(int nrows, int ncols, int nwa, int nwb, const int *WA, const int *WB,
                        float *A, float *B, float lrate, float vexp, int nthreads) {
  int ithread;
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int i, j, k, c, itmp;
    int64_t ia, ib, ja;
    float cv, ascale, bscale;
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    float *daa = (float *)malloc((size_t)nwa * nrows * sizeof(float));
    float *dbb = (float *)malloc((size_t)nrows * sizeof(float));

    for (i = istart; i < iend; i++) {
      for (c = 0; c < nwa * nrows; c++) daa[c] = 0;
      for (k = 0; k < nwb; k++) {
        itmp = WB[k + (int64_t)i * nwb];
        ib = (int64_t)nrows * itmp;
        bscale = pow(1 + itmp, vexp);
        for (c = 0; c < nrows; c++) dbb[c] = 0;
        for (j = 0; j < nwa; j++) {
          itmp = WA[j + (int64_t)i * nwa];
          ia = (int64_t)nrows * itmp;
          ascale = pow(1 + itmp, vexp);
          cv = 0;
          for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
          cv = oracle_sigmoid(cv);
          cv = -lrate * cv;
          ja = (int64_t)j * nrows;
          for (c = 0; c < nrows; c++) {
            dbb[c] += bscale * cv * A[c + ia];
            daa[c + ja] += ascale * cv * B[c + ib];
          }
        }
        for (c = 0; c < nrows; c++) B[c + ib] += dbb[c];
      }
      for (j = 0; j < nwa; j++) {
        ja = (int64_t)j * nrows;
        ia = (int64_t)nrows * WA[j + (int64_t)i * nwa];
        for (c = 0; c < nrows; c++) A[c + ia] += daa[c + ja];
      }
    }
    free(dbb);
    free(daa);
  }
}

void oracle_word2vecNegFilt(int nrows, int ncols, int nwords, int nwa, int nwb, const int *WA,
                            const int *WB, float *A, float *B, float lrate, float vexp,
                            int nthreads) {
  /* Groups are rebuilt without the filtered ids and handed to the plain routine one at a time:
   * dropping an id removes exactly the dot products and updates it would have taken part in. */
  int i, j, k;
  int *wa = (int *)malloc((size_t)(nwa > 0 ? nwa : 1) * sizeof(int));
  int *wb = (int *)malloc((size_t)(nwb > 0 ? nwb : 1) * sizeof(int));
  (void)nthreads;
  for (i = 0; i < ncols; i++) {
    int na = 0, nb = 0;
    for (j = 0; j < nwa; j++) {
      int id = WA[j + (int64_t)i * nwa];
      if (id >= 0 && id < nwords) wa[na++] = id;
    }
    for (k = 0; k < nwb; k++) {
      int id = WB[k + (int64_t)i * nwb];
      if (id >= 0 && id < nwords) wb[nb++] = id;
    }
    if (na > 0 && nb > 0) oracle_word2vecNeg(nrows, 1, na, nb, wa, wb, A, B, lrate, vexp, 1);
  }
  free(wb);
  free(wa);
}

double oracle_word2vecEvalPos(int nrows, int ncols, int skip, const int *W, const int *LB,
                              const int *UB, const float *A, const float *B, double floorv,
                              int nthreads) {
  int i, ithread;
  double *pv = (double *)malloc((size_t)nthreads * sizeof(double));
  double sum = 0;
  (void)skip;
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    int ii, j, c;
    int64_t ia, ib;
    float cv;
    double dv = 0;
    for (ii = istart; ii < iend; ii++) {
      if (W[ii] >= 0) {
        ia = (int64_t)nrows * W[ii];
        for (j = LB[ii]; j <= UB[ii]; j++) {
          if (j != 0 && ii + j >= 0 && ii + j < ncols) {
            if (W[ii + j] >= 0) {
              ib = (int64_t)nrows * W[ii + j];
              cv = 0;
              for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
              cv = oracle_sigmoid(cv);
              dv += log(fmax((double)cv, floorv));
            }
          }
        }
      }
    }
    pv[ithread] = dv;
  }
  for (i = 0; i < nthreads; i++) sum += pv[i];
  free(pv);
  return sum;
}

double oracle_word2vecEvalNeg(int nrows, int ncols, int nwa, int nwb, const int *WA, const int *WB,
                              const float *A, const float *B, double floorv, int nthreads) {
  int i, ithread;
  double *pv = (double *)malloc((size_t)nthreads * sizeof(double));
  double sum = 0;
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int ii, j, k, c;
    int64_t ia, ib;
    float cv;
    double dv = 0;
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    for (ii = istart; ii < iend; ii++) {
      for (k = 0; k < nwb; k++) {
        ib = (int64_t)nrows * WB[k + (int64_t)ii * nwb];
        for (j = 0; j < nwa; j++) {
          ia = (int64_t)nrows * WA[j + (int64_t)ii * nwa];
          cv = 0;
          for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
          cv = oracle_sigmoid(cv);
          dv += log(fmax(1.0 - (double)cv, floorv));
        }
      }
    }
    pv[ithread] = dv;
  }
  for (i = 0; i < nthreads; i++) sum += pv[i];
  free(pv);
  return sum;
}

/* Where word `indx` of a sliced, multi-part model lives (BIDMach_CPUMACH.c:80-88): ids below nhead
 * ("head") keep their column and exist on every slice; the others ("tail") are dealt round-robin
 * to nslices slices and packed after the head.  Part m of the model holds columns
 * [m*maxcols, (m+1)*maxcols); its B table is MM[2*(m+offset)], its A table MM[2*(m+offset)+1]. */
static void oracle_map_index(int *mm, int64_t *ii, int *ismine, int *ishead, int indx, int islice,
                             int nslices, int nhead, int maxcols, int nrows, int offset) {
  int newi = indx;
  int part;
  if (indx >= nhead) newi = (indx - nhead) / nslices + nhead;
  part = newi / maxcols;
  *mm = part + offset;
  *ismine = (indx >= nhead) && (indx % nslices == islice);
  *ishead = (indx < nhead);
  *ii = (int64_t)nrows * (newi - part * maxcols);
}

static int oracle_pair_trained(int aismine, int aishead, int bismine, int bishead, int doHead) {
  /* BIDMach_CPUMACH.c:137, :315 */
  return (doHead > 1 && aishead && bishead) || (aismine && bishead) || (bismine && aishead) ||
         (aismine && bismine);
}

void oracle_word2vecPosSlice(int nrows, int ncols, int skip, const int *W, const int *LB,
                             const int *UB, float **MM, float lrate, float vexp, int nthreads,
                             int islice, int nslices, int maxCols, int nHead, int dualMode,
                             int doHead) {
  int ithread;
  const int offset = dualMode ? 1 : 0;
  (void)skip;
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    int i, j, c, iac, ibc, touched;
    int64_t ia, ib;
    int aismine, bismine, aishead, bishead, ma, mb;
    float cv, ascale, bscale;
    float *A, *B;
    float *daa = (float *)malloc((size_t)nrows * sizeof(float));

    for (i = istart; i < iend; i++) {
      iac = W[i];
      if (iac >= 0) {
        oracle_map_index(&ma, &ia, &aismine, &aishead, iac, islice, nslices, nHead, maxCols, nrows,
                         offset);
        A = MM[2 * ma + 1];
        ascale = pow(1 + iac, vexp);
        for (c = 0; c < nrows; c++) daa[c] = 0;
        touched = 0;
        for (j = LB[i]; j <= UB[i]; j++) {
          if (j != 0 && i + j >= 0 && i + j < ncols) {
            ibc = W[i + j];
            if (ibc >= 0) {
              oracle_map_index(&mb, &ib, &bismine, &bishead, ibc, islice, nslices, nHead, maxCols,
                               nrows, offset);
              B = MM[2 * mb];
              bscale = pow(1 + ibc, vexp);
              if (oracle_pair_trained(aismine, aishead, bismine, bishead, doHead)) {
                touched = 1;
                cv = 0;
                for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
                cv = oracle_sigmoid(cv);
                cv = lrate * (1.0f - cv);
                for (c = 0; c < nrows; c++) daa[c] += ascale * cv * B[c + ib];
                if (bismine || (bishead && doHead)) {
                  for (c = 0; c < nrows; c++) B[c + ib] += bscale * cv * A[c + ia];
                }
              }
            }
          }
        }
        if (touched && (aismine || (aishead && doHead))) {
          for (c = 0; c < nrows; c++) A[c + ia] += daa[c];
        }
      }
    }
    free(daa);
  }
}

void oracle_word2vecNegSlice(int nrows, int ncols, int nwa, int nwb, const int *WA, const int *WB,
                             float **MM, float lrate, float vexp, int nthreads, int islice,
                             int nslices, int maxCols, int nHead, int dualMode, int doHead) {
  int ithread;
  const int offset = dualMode ? 1 : 0;
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int i, j, k, c, iac, ibc;
    int64_t ia, ib, ja;
    float cv, ascale, bscale;
    float *A, *B;
    int aismine, bismine, aishead, bishead, ma, mb;
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    float *daa = (float *)malloc((size_t)nwa * nrows * sizeof(float));
    float *dbb = (float *)malloc((size_t)nrows * sizeof(float));

    for (i = istart; i < iend; i++) {
      for (c = 0; c < nwa * nrows; c++) daa[c] = 0;
      for (k = 0; k < nwb; k++) {
        ibc = WB[k + (int64_t)i * nwb];
        oracle_map_index(&mb, &ib, &bismine, &bishead, ibc, islice, nslices, nHead, maxCols, nrows,
                         offset);
        B = MM[2 * mb];
        bscale = pow(1 + ibc, vexp);
        for (c = 0; c < nrows; c++) dbb[c] = 0;
        for (j = 0; j < nwa; j++) {
          iac = WA[j + (int64_t)i * nwa];
          oracle_map_index(&ma, &ia, &aismine, &aishead, iac, islice, nslices, nHead, maxCols, nrows,
                           offset);
          A = MM[2 * ma + 1];
          ascale = pow(1 + iac, vexp);
          if (oracle_pair_trained(aismine, aishead, bismine, bishead, doHead)) {
            cv = 0;
            for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
            cv = oracle_sigmoid(cv);
            cv = -lrate * cv;
            ja = (int64_t)j * nrows;
            for (c = 0; c < nrows; c++) {
              dbb[c] += bscale * cv * A[c + ia];
              daa[c + ja] += ascale * cv * B[c + ib];
            }
          }
        }
        if (bismine || (bishead && doHead)) {
          for (c = 0; c < nrows; c++) B[c + ib] += dbb[c];
        }
      }
      for (j = 0; j < nwa; j++) {
        ja = (int64_t)j * nrows;
        iac = WA[j + (int64_t)i * nwa];
        oracle_map_index(&ma, &ia, &aismine, &aishead, iac, islice, nslices, nHead, maxCols, nrows,
                         offset);
        A = MM[2 * ma + 1];
        if (aismine || (aishead && doHead)) {
          for (c = 0; c < nrows; c++) A[c + ia] += daa[c + ja];
        }
      }
    }
    free(dbb);
    free(daa);
  }
}

/* Word2Vec.scala:1007-1069: a pair is scored iff both words are resident (mine or head). */
double oracle_word2vecEvalPosSlice(int nrows, int ncols, int skip, const int *W, const int *LB,
                                   const int *UB, float **MM, double floorv, int nthreads,
                                   int islice, int nslices, int maxCols, int nHead, int dualMode) {
  int i, ithread;
  const int offset = dualMode ? 1 : 0;
  double *pv = (double *)malloc((size_t)nthreads * sizeof(double));
  double sum = 0;
  (void)skip;
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    int ii, j, c, ma, mb, aismine, aishead, bismine, bishead;
    int64_t ia, ib;
    float cv;
    const float *A, *B;
    double dv = 0;
    for (ii = istart; ii < iend; ii++) {
      if (W[ii] >= 0) {
        oracle_map_index(&ma, &ia, &aismine, &aishead, W[ii], islice, nslices, nHead, maxCols,
                         nrows, offset);
        if (aismine || aishead) {
          A = MM[2 * ma + 1];
          for (j = LB[ii]; j <= UB[ii]; j++) {
            if (j != 0 && ii + j >= 0 && ii + j < ncols && W[ii + j] >= 0) {
              oracle_map_index(&mb, &ib, &bismine, &bishead, W[ii + j], islice, nslices, nHead,
                               maxCols, nrows, offset);
              if (bismine || bishead) {
                B = MM[2 * mb];
                cv = 0;
                for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
                cv = oracle_sigmoid(cv);
                dv += log(fmax((double)cv, floorv));
              }
            }
          }
        }
      }
    }
    pv[ithread] = dv;
  }
  for (i = 0; i < nthreads; i++) sum += pv[i];
  free(pv);
  return sum;
}

/* Word2Vec.scala:1134-1200 */
double oracle_word2vecEvalNegSlice(int nrows, int ncols, int nwa, int nwb, const int *WA,
                                   const int *WB, float **MM, double floorv, int nthreads,
                                   int islice, int nslices, int maxCols, int nHead, int dualMode) {
  int i, ithread;
  const int offset = dualMode ? 1 : 0;
  double *pv = (double *)malloc((size_t)nthreads * sizeof(double));
  double sum = 0;
#pragma omp parallel for num_threads(nthreads)
  for (ithread = 0; ithread < nthreads; ithread++) {
    int ii, j, k, c, ma, mb, aismine, aishead, bismine, bishead;
    int64_t ia, ib;
    float cv;
    const float *A, *B;
    double dv = 0;
    int istart = (int)((1L * ithread * ncols) / nthreads);
    int iend = (int)((1L * (ithread + 1) * ncols) / nthreads);
    for (ii = istart; ii < iend; ii++) {
      for (k = 0; k < nwb; k++) {
        oracle_map_index(&mb, &ib, &bismine, &bishead, WB[k + (int64_t)ii * nwb], islice, nslices,
                         nHead, maxCols, nrows, offset);
        if (bismine || bishead) {
          B = MM[2 * mb];
          for (j = 0; j < nwa; j++) {
            oracle_map_index(&ma, &ia, &aismine, &aishead, WA[j + (int64_t)ii * nwa], islice,
                             nslices, nHead, maxCols, nrows, offset);
            if (aismine || aishead) {
              A = MM[2 * ma + 1];
              cv = 0;
              for (c = 0; c < nrows; c++) cv += A[c + ia] * B[c + ib];
              cv = oracle_sigmoid(cv);
              dv += log(fmax(1.0 - (double)cv, floorv));
            }
          }
        }
      }
    }
    pv[ithread] = dv;
  }
  for (i = 0; i < nthreads; i++) sum += pv[i];
  free(pv);
  return sum;
}

int oracle_max_threads(void) { return omp_get_max_threads(); }
