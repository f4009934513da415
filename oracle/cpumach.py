"""ctypes binding of the C oracle, shaped like the reference's CPU operator class.

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
import this module.  The method names and argument lists are those of
src/main/java/edu/berkeley/bid/CPUMACH.java:12,14,17,19,26,28 of the reference (numpy arrays stand
in for Java primitive arrays; A and B are updated in place).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libw2v_oracle.so")
_lib = None

C_FLOOR = 1.0e-40      # jni/src/BIDMach_CPUMACH.c:409,467
SCALA_FLOOR = 1.0e-20  # Word2Vec.scala:995,1123 and DNN127.cu:310,916


def build(force=False):
    """Compile the oracle with the reference's CPU flags (oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    ip = ctypes.POINTER(ctypes.c_int)
    fp = ctypes.POINTER(ctypes.c_float)
    ci, cf, cd = ctypes.c_int, ctypes.c_float, ctypes.c_double
    lib.oracle_word2vecPos.argtypes = [ci, ci, ci, ip, ip, ip, fp, fp, cf, cf, ci]
    lib.oracle_word2vecPos.restype = None
    lib.oracle_word2vecNeg.argtypes = [ci, ci, ci, ci, ip, ip, fp, fp, cf, cf, ci]
    lib.oracle_word2vecNeg.restype = None
    lib.oracle_word2vecNegFilt.argtypes = [ci, ci, ci, ci, ci, ip, ip, fp, fp, cf, cf, ci]
    lib.oracle_word2vecNegFilt.restype = None
    lib.oracle_word2vecEvalPos.argtypes = [ci, ci, ci, ip, ip, ip, fp, fp, cd, ci]
    lib.oracle_word2vecEvalPos.restype = cd
    lib.oracle_word2vecEvalNeg.argtypes = [ci, ci, ci, ci, ip, ip, fp, fp, cd, ci]
    lib.oracle_word2vecEvalNeg.restype = cd
    fpp = ctypes.POINTER(fp)
    lib.oracle_word2vecPosSlice.argtypes = [ci, ci, ci, ip, ip, ip, fpp, cf, cf, ci,
                                            ci, ci, ci, ci, ci, ci]
    lib.oracle_word2vecPosSlice.restype = None
    lib.oracle_word2vecNegSlice.argtypes = [ci, ci, ci, ci, ip, ip, fpp, cf, cf, ci,
                                            ci, ci, ci, ci, ci, ci]
    lib.oracle_word2vecNegSlice.restype = None
    lib.oracle_word2vecEvalPosSlice.argtypes = [ci, ci, ci, ip, ip, ip, fpp, cd, ci,
                                                ci, ci, ci, ci, ci]
    lib.oracle_word2vecEvalPosSlice.restype = cd
    lib.oracle_word2vecEvalNegSlice.argtypes = [ci, ci, ci, ci, ip, ip, fpp, cd, ci,
                                                ci, ci, ci, ci, ci]
    lib.oracle_word2vecEvalNegSlice.restype = cd
    lib.oracle_max_threads.restype = ci
    hp = ctypes.POINTER(ctypes.c_uint16)
    cu64, cu32 = ctypes.c_uint64, ctypes.c_uint32
    lib.oracle_word2vecPosBf16.argtypes = [ci, ci, ci, ip, ip, ip, hp, hp, cf, cf, cu64, ci]
    lib.oracle_word2vecPosBf16.restype = None
    lib.oracle_word2vecNegBf16.argtypes = [ci, ci, ci, ci, ip, ip, hp, hp, cf, cf, cu64, ci]
    lib.oracle_word2vecNegBf16.restype = None
    lib.oracle_word2vecEvalPosBf16.argtypes = [ci, ci, ci, ip, ip, ip, hp, hp, cd]
    lib.oracle_word2vecEvalPosBf16.restype = cd
    lib.oracle_word2vecEvalNegBf16.argtypes = [ci, ci, ci, ci, ip, ip, hp, hp, cd]
    lib.oracle_word2vecEvalNegBf16.restype = cd
    lib.oracle_bf16_key.argtypes = [cu64, cu32, cu32]
    lib.oracle_bf16_key.restype = cu32
    lib.oracle_bf16_narrow.argtypes = [cf, cu32, cu32]
    lib.oracle_bf16_narrow.restype = ctypes.c_uint16
    _lib = lib
    return lib


def _i(a):
    assert a.dtype == np.int32 and (a.flags.c_contiguous or a.flags.f_contiguous)
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int))


def _f(a):
    assert a.dtype == np.float32 and (a.flags.c_contiguous or a.flags.f_contiguous)
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _h(a):
    assert a.dtype == np.uint16 and (a.flags.c_contiguous or a.flags.f_contiguous)
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16))


def bf16_widen(h):
    """bfloat16 bit patterns (uint16) -> float32, exact."""
    return (np.asarray(h, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def bf16_truncate(x):
    """float32 -> bfloat16 bit patterns by dropping the low 16 bits (round toward zero)."""
    return (np.ascontiguousarray(x, np.float32).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def bf16_key(seed, unit, slot):
    return int(_load().oracle_bf16_key(seed, unit, slot))


def bf16_narrow(x, key, row):
    return int(_load().oracle_bf16_narrow(float(x), key, row))


def _mm(mats):
    """float** over a list of model matrices (B of part m at 2m, A at 2m+1)."""
    arr = (ctypes.POINTER(ctypes.c_float) * len(mats))()
    for k, m in enumerate(mats):
        arr[k] = _f(m) if m is not None else None
    return arr


def max_threads():
    return int(_load().oracle_max_threads())


class CPUMACH:
    """Same static-method surface as edu.berkeley.bid.CPUMACH for the four SGNS calls.

    Model matrices are nrows x vocab, column-major: pass numpy arrays of shape (vocab, nrows)
    in C order (word w's vector is row w), which is the same memory layout.
    """

    @staticmethod
    def word2vecPos(nrows, ncols, skip, W, LB, UB, A, B, lrate, vexp, nthreads):
        _load().oracle_word2vecPos(nrows, ncols, skip, _i(W), _i(LB), _i(UB), _f(A), _f(B),
                                   lrate, vexp, nthreads)

    @staticmethod
    def word2vecNeg(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, nthreads):
        _load().oracle_word2vecNeg(nrows, ncols, nwa, nwb, _i(WA), _i(WB), _f(A), _f(B),
                                   lrate, vexp, nthreads)

    @staticmethod
    def word2vecNegFilt(nrows, ncols, nwords, nwa, nwb, WA, WB, A, B, lrate, vexp, nthreads):
        """CPU statement of the reference's GPU-only filtered negative pass (CUMACH.java:94)."""
        _load().oracle_word2vecNegFilt(nrows, ncols, nwords, nwa, nwb, _i(WA), _i(WB), _f(A),
                                       _f(B), lrate, vexp, nthreads)

    @staticmethod
    def word2vecEvalPos(nrows, ncols, skip, W, LB, UB, A, B, nthreads, floor=C_FLOOR):
        return float(_load().oracle_word2vecEvalPos(nrows, ncols, skip, _i(W), _i(LB), _i(UB),
                                                    _f(A), _f(B), floor, nthreads))

    @staticmethod
    def word2vecEvalNeg(nrows, ncols, nwa, nwb, WA, WB, A, B, nthreads, floor=C_FLOOR):
        return float(_load().oracle_word2vecEvalNeg(nrows, ncols, nwa, nwb, _i(WA), _i(WB),
                                                    _f(A), _f(B), floor, nthreads))

    # ---- bfloat16 tables (no counterpart in the reference; oracle/w2v_oracle_bf16.c) ---------
    @staticmethod
    def word2vecPosBf16(nrows, ncols, skip, W, LB, UB, A, B, lrate, vexp, seed, hot_n=0):
        _load().oracle_word2vecPosBf16(nrows, ncols, skip, _i(W), _i(LB), _i(UB), _h(A), _h(B),
                                       lrate, vexp, seed, hot_n)

    @staticmethod
    def word2vecNegBf16(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed, hot_n=0):
        _load().oracle_word2vecNegBf16(nrows, ncols, nwa, nwb, _i(WA), _i(WB), _h(A), _h(B),
                                       lrate, vexp, seed, hot_n)

    @staticmethod
    def word2vecEvalPosBf16(nrows, ncols, skip, W, LB, UB, A, B, floor=C_FLOOR):
        return float(_load().oracle_word2vecEvalPosBf16(nrows, ncols, skip, _i(W), _i(LB),
                                                        _i(UB), _h(A), _h(B), floor))

    @staticmethod
    def word2vecEvalNegBf16(nrows, ncols, nwa, nwb, WA, WB, A, B, floor=C_FLOOR):
        return float(_load().oracle_word2vecEvalNegBf16(nrows, ncols, nwa, nwb, _i(WA), _i(WB),
                                                        _h(A), _h(B), floor))

    # ---- sliced, multi-part models (CPUMACH.java:14,19; Scala-only forward twins) ----------
    @staticmethod
    def word2vecPosSlice(nrows, ncols, skip, W, LB, UB, MM, lrate, vexp, nthreads, islice,
                         nslices, maxCols, nHead, dualMode, doHead):
        _load().oracle_word2vecPosSlice(nrows, ncols, skip, _i(W), _i(LB), _i(UB), _mm(MM), lrate,
                                        vexp, nthreads, islice, nslices, maxCols, nHead,
                                        int(dualMode), doHead)

    @staticmethod
    def word2vecNegSlice(nrows, ncols, nwa, nwb, WA, WB, MM, lrate, vexp, nthreads, islice,
                         nslices, maxCols, nHead, dualMode, doHead):
        _load().oracle_word2vecNegSlice(nrows, ncols, nwa, nwb, _i(WA), _i(WB), _mm(MM), lrate,
                                        vexp, nthreads, islice, nslices, maxCols, nHead,
                                        int(dualMode), doHead)

    @staticmethod
    def word2vecEvalPosSlice(nrows, ncols, skip, W, LB, UB, MM, nthreads, islice, nslices,
                             maxCols, nHead, dualMode, floor=SCALA_FLOOR):
        return float(_load().oracle_word2vecEvalPosSlice(
            nrows, ncols, skip, _i(W), _i(LB), _i(UB), _mm(MM), floor, nthreads, islice, nslices,
            maxCols, nHead, int(dualMode)))

    @staticmethod
    def word2vecEvalNegSlice(nrows, ncols, nwa, nwb, WA, WB, MM, nthreads, islice, nslices,
                             maxCols, nHead, dualMode, floor=SCALA_FLOOR):
        return float(_load().oracle_word2vecEvalNegSlice(
            nrows, ncols, nwa, nwb, _i(WA), _i(WB), _mm(MM), floor, nthreads, islice, nslices,
            maxCols, nHead, int(dualMode)))
