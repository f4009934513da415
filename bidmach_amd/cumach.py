"""ctypes binding of the HIP library, shaped like the reference's GPU operator class.

`CUMACH.word2vecPos/Neg/EvalPos/EvalNeg` keep the argument lists of the static natives in
src/main/java/edu/berkeley/bid/CUMACH.java:90,92,96,98 of the reference.  Where the Java side
passes a jcuda.Pointer, this binding takes anything that exposes a device address: a torch
tensor on the GPU (its data_ptr() is used), an object with a `.ptr` attribute, or a plain int.
Return value: 0 or a HIP error code, exactly what the native call returned; `check()` turns a
non-zero code into the RuntimeException-like error the Scala caller raises
(Word2Vec.scala:374,393,478,512).

The shared library must have been built (python -m bidmach_amd.build); loading fails loudly
otherwise.  Nothing here computes on the CPU.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libbidmachhip-linux-x86_64.so"
_lib = None


class W2VLibraryError(RuntimeError):
    pass


def lib_path():
    """Path of the HIP library; BIDMACH_W2V_LIB overrides the in-tree default."""
    return os.environ.get("BIDMACH_W2V_LIB") or os.path.join(_HERE, "lib", _LIB_NAME)


# name -> (restype, argtypes); every symbol include/bidmach_w2v.h declares.
_I, _F, _D, _P, _SZ = ctypes.c_int, ctypes.c_float, ctypes.c_double, ctypes.c_void_p, ctypes.c_size_t
_PP = ctypes.POINTER(ctypes.c_void_p)
_POS = [_I, _I, _I, _P, _P, _P, _P, _P, _F, _F]
_NEG = [_I, _I, _I, _I, _P, _P, _P, _P, _F, _F]
_EPOS = [_I, _I, _I, _P, _P, _P, _P, _P, _P]
_ENEG = [_I, _I, _I, _I, _P, _P, _P, _P, _P]
SYMBOLS = {
    "word2vecPos": (_I, _POS),
    "word2vecNeg": (_I, _NEG),
    "word2vecNegFilt": (_I, [_I, _I, _I, _I, _I, _P, _P, _P, _P, _F, _F]),
    "word2vecPosSlice": (_I, [_I, _I, _I, _P, _P, _P, _PP, _I, _F, _F, _I, _I, _I, _I, _I, _I]),
    "word2vecNegSlice": (_I, [_I, _I, _I, _I, _P, _P, _PP, _I, _F, _F, _I, _I, _I, _I, _I, _I]),
    "word2vecEvalPosSlice": (_I, [_I, _I, _I, _P, _P, _P, _PP, _I, _I, _I, _I, _I, _I, _P]),
    "word2vecEvalNegSlice": (_I, [_I, _I, _I, _I, _P, _P, _PP, _I, _I, _I, _I, _I, _I, _P]),
    "w2v_max_slice_parts": (_I, []),
    "word2vecEvalPos": (_I, _EPOS),
    "word2vecEvalNeg": (_I, _ENEG),
    "word2vecEvalPosF64": (_I, _EPOS),
    "word2vecEvalNegF64": (_I, _ENEG),
    "word2vecEvalNegNoAlloc": (_I, _ENEG),
    "w2v_no_alloc_max_groups": (_I, []),
    "word2vecPosAsync": (_I, _POS),
    "word2vecNegAsync": (_I, _NEG),
    "word2vecEvalPosAsync": (_I, _EPOS),
    "word2vecEvalNegAsync": (_I, _ENEG),
    "word2vecPosBf16": (_I, _POS + [ctypes.c_ulonglong]),
    "word2vecNegBf16": (_I, _NEG + [ctypes.c_ulonglong]),
    "word2vecPosBf16Async": (_I, _POS + [ctypes.c_ulonglong]),
    "word2vecNegBf16Async": (_I, _NEG + [ctypes.c_ulonglong]),
    "word2vecEvalPosBf16": (_I, _EPOS),
    "word2vecEvalNegBf16": (_I, _ENEG),
    "w2v_set_bf16_hot_words": (_I, [_I]),
    "w2v_get_bf16_hot_words": (_I, []),
    "w2v_f32_to_bf16": (_I, [_SZ, _P, _P]),
    "w2v_bf16_to_f32": (_I, [_SZ, _P, _P]),
    "w2v_set_eval_floor": (None, [_D]),
    "w2v_get_eval_floor": (_D, []),
    "w2v_set_stream": (_I, [_P]),
    "w2v_reset_stream": (_I, []),
    "w2v_get_stream": (_P, []),
    "w2v_synchronize": (_I, []),
    "w2v_release_thread": (_I, []),
    "w2v_set_max_workgroups": (_I, [_I]),
    "w2v_get_max_workgroups": (_I, []),
    "w2v_set_ordered_mode": (_I, [_I]),
    "w2v_get_ordered_mode": (_I, []),
    "w2v_last_launch_form": (_I, []),
    "w2v_set_ordered_workers": (_I, [_I, _I]),
    "w2v_set_ordered_copies": (_I, [_I, _I]),
    "w2v_set_hot_update_mode": (_I, [_I]),
    "w2v_get_hot_update_mode": (_I, []),
    "w2v_set_rare_update_mode": (_I, [_I]),
    "w2v_get_rare_update_mode": (_I, []),
    "w2v_max_rows": (_I, []),
    "w2v_max_nwb": (_I, []),
    "w2v_malloc": (_I, [ctypes.POINTER(_P), _SZ]),
    "w2v_free": (_I, [_P]),
    "w2v_memcpy_h2d": (_I, [_P, _P, _SZ]),
    "w2v_memcpy_d2h": (_I, [_P, _P, _SZ]),
    "w2v_memset": (_I, [_P, _I, _SZ]),
    "w2v_wordmats": (_I, [_I, _P, _I, _I, _I, _I, _I, _F, _F, ctypes.c_ulonglong, ctypes.c_uint,
                          _P, _P, _P, _P, _P, _P, ctypes.POINTER(_I)]),
    "w2v_timer_create": (_I, [ctypes.POINTER(_P)]),
    "w2v_timer_destroy": (_I, [_P]),
    "w2v_timer_start": (_I, [_P]),
    "w2v_timer_stop": (_I, [_P]),
    "w2v_timer_elapsed_ms": (_I, [_P, ctypes.POINTER(_F)]),
    "w2v_error_string": (ctypes.c_char_p, [_I]),
    "w2v_lz4_compress_bound": (_SZ, [_SZ]),
    "w2v_lz4_compress": (ctypes.c_longlong, [_P, _SZ, _P, _SZ]),
    "w2v_lz4_decompress": (ctypes.c_longlong, [_P, _SZ, _P, _SZ]),
}


def load_library(path=None):
    """Loads the HIP library and declares every exported symbol's signature."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or lib_path()
    # PyTorch-ROCm ships its own copy of the HIP runtime.  If it is going to be used in this
    # process (it owns the device buffers in the tests and the benchmark) it has to be loaded
    # first, so that this library binds to the same runtime instance instead of bringing in the
    # system copy next to it.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    if not os.path.exists(p):
        raise W2VLibraryError(
            "HIP library %s is missing: build it with `python -m bidmach_amd.build` "
            "(there is no CPU fallback)" % p)
    try:
        lib = ctypes.CDLL(p)
    except OSError as e:
        raise W2VLibraryError("cannot load %s: %s" % (p, e)) from e
    for name, (res, args) in SYMBOLS.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise W2VLibraryError("%s does not export %s" % (p, name)) from e
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def _ptr(x):
    """Device address of a Pointer-like argument."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        if hasattr(x, "is_cuda") and not x.is_cuda:
            raise W2VLibraryError("host tensor passed where a device pointer is required")
        return x.data_ptr()
    if hasattr(x, "ptr"):
        return int(x.ptr)
    raise TypeError("not a device pointer: %r" % type(x))


def _ptr_array(mats):
    """Host array of device addresses for a list of model matrices (a float** argument)."""
    arr = (ctypes.c_void_p * len(mats))()
    for k, m in enumerate(mats):
        arr[k] = _ptr(m)
    return arr


def error_string(err):
    return load_library().w2v_error_string(int(err)).decode()


def check(err, what):
    """Raises like the Scala caller does on a non-zero return (Word2Vec.scala:374)."""
    if err != 0:
        raise W2VLibraryError("CUMACH.%s error %s" % (what, error_string(err)))


class CUMACH:
    """The four SGNS natives of edu.berkeley.bid.CUMACH (CUMACH.java:90,92,96,98)."""

    @staticmethod
    def word2vecPos(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp):
        return load_library().word2vecPos(nrows, ncols, shift, _ptr(W), _ptr(LB), _ptr(UB),
                                          _ptr(A), _ptr(B), lrate, vexp)

    @staticmethod
    def word2vecNeg(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp):
        return load_library().word2vecNeg(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB), _ptr(A),
                                          _ptr(B), lrate, vexp)

    @staticmethod
    def word2vecNegFilt(nrows, ncols, nwords, nwa, nwb, WA, WB, A, B, lrate, vexp):
        """CUMACH.java:94."""
        return load_library().word2vecNegFilt(nrows, ncols, nwords, nwa, nwb, _ptr(WA), _ptr(WB),
                                              _ptr(A), _ptr(B), lrate, vexp)

    @staticmethod
    def word2vecEvalPos(nrows, ncols, shift, W, LB, UB, A, B, retVal):
        return load_library().word2vecEvalPos(nrows, ncols, shift, _ptr(W), _ptr(LB), _ptr(UB),
                                              _ptr(A), _ptr(B), _ptr(retVal))

    @staticmethod
    def word2vecEvalNeg(nrows, ncols, nwa, nwb, WA, WB, A, B, retVal):
        return load_library().word2vecEvalNeg(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB),
                                              _ptr(A), _ptr(B), _ptr(retVal))

    # -- sliced, multi-part models: device counterparts of CPUMACH.java:14,19 and of the Scala
    # -- forward twins (Word2Vec.scala:1007-1069, 1134-1200); MM is the list of model matrices

    @staticmethod
    def word2vecPosSlice(nrows, ncols, shift, W, LB, UB, MM, lrate, vexp, islice, nslices,
                         maxCols, nHead, dualMode, doHead):
        return load_library().word2vecPosSlice(
            nrows, ncols, shift, _ptr(W), _ptr(LB), _ptr(UB), _ptr_array(MM), len(MM), lrate, vexp,
            islice, nslices, maxCols, nHead, int(dualMode), doHead)

    @staticmethod
    def word2vecNegSlice(nrows, ncols, nwa, nwb, WA, WB, MM, lrate, vexp, islice, nslices,
                         maxCols, nHead, dualMode, doHead):
        return load_library().word2vecNegSlice(
            nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB), _ptr_array(MM), len(MM), lrate, vexp,
            islice, nslices, maxCols, nHead, int(dualMode), doHead)

    @staticmethod
    def word2vecEvalPosSlice(nrows, ncols, shift, W, LB, UB, MM, islice, nslices, maxCols, nHead,
                             dualMode, retVal):
        return load_library().word2vecEvalPosSlice(
            nrows, ncols, shift, _ptr(W), _ptr(LB), _ptr(UB), _ptr_array(MM), len(MM), islice,
            nslices, maxCols, nHead, int(dualMode), _ptr(retVal))

    @staticmethod
    def word2vecEvalNegSlice(nrows, ncols, nwa, nwb, WA, WB, MM, islice, nslices, maxCols, nHead,
                             dualMode, retVal):
        return load_library().word2vecEvalNegSlice(
            nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB), _ptr_array(MM), len(MM), islice, nslices,
            maxCols, nHead, int(dualMode), _ptr(retVal))

    # -- extensions of the library (no Java counterpart) ---------------------------------

    @staticmethod
    def word2vecEvalPosF64(nrows, ncols, shift, W, LB, UB, A, B, retVal):
        return load_library().word2vecEvalPosF64(nrows, ncols, shift, _ptr(W), _ptr(LB),
                                                 _ptr(UB), _ptr(A), _ptr(B), _ptr(retVal))

    @staticmethod
    def word2vecEvalNegF64(nrows, ncols, nwa, nwb, WA, WB, A, B, retVal):
        return load_library().word2vecEvalNegF64(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB),
                                                 _ptr(A), _ptr(B), _ptr(retVal))

    @staticmethod
    def word2vecPosAsync(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp):
        return load_library().word2vecPosAsync(nrows, ncols, shift, _ptr(W), _ptr(LB), _ptr(UB),
                                               _ptr(A), _ptr(B), lrate, vexp)

    @staticmethod
    def word2vecNegAsync(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp):
        return load_library().word2vecNegAsync(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB),
                                               _ptr(A), _ptr(B), lrate, vexp)

    @staticmethod
    def word2vecEvalPosAsync(nrows, ncols, shift, W, LB, UB, A, B, retVal):
        return load_library().word2vecEvalPosAsync(nrows, ncols, shift, _ptr(W), _ptr(LB),
                                                   _ptr(UB), _ptr(A), _ptr(B), _ptr(retVal))

    @staticmethod
    def word2vecEvalNegAsync(nrows, ncols, nwa, nwb, WA, WB, A, B, retVal):
        return load_library().word2vecEvalNegAsync(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB),
                                                   _ptr(A), _ptr(B), _ptr(retVal))

    # -- bfloat16 tables (no Java counterpart): stochastic-rounded, atomic-free write-back -----

    @staticmethod
    def word2vecPosBf16(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, seed):
        return load_library().word2vecPosBf16(nrows, ncols, shift, _ptr(W), _ptr(LB), _ptr(UB),
                                              _ptr(A), _ptr(B), lrate, vexp, seed)

    @staticmethod
    def word2vecNegBf16(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed):
        return load_library().word2vecNegBf16(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB), _ptr(A),
                                              _ptr(B), lrate, vexp, seed)

    @staticmethod
    def word2vecPosBf16Async(nrows, ncols, shift, W, LB, UB, A, B, lrate, vexp, seed):
        return load_library().word2vecPosBf16Async(nrows, ncols, shift, _ptr(W), _ptr(LB),
                                                   _ptr(UB), _ptr(A), _ptr(B), lrate, vexp, seed)

    @staticmethod
    def word2vecNegBf16Async(nrows, ncols, nwa, nwb, WA, WB, A, B, lrate, vexp, seed):
        return load_library().word2vecNegBf16Async(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB),
                                                   _ptr(A), _ptr(B), lrate, vexp, seed)

    @staticmethod
    def word2vecEvalPosBf16(nrows, ncols, shift, W, LB, UB, A, B, retVal):
        return load_library().word2vecEvalPosBf16(nrows, ncols, shift, _ptr(W), _ptr(LB),
                                                  _ptr(UB), _ptr(A), _ptr(B), _ptr(retVal))

    @staticmethod
    def word2vecEvalNegBf16(nrows, ncols, nwa, nwb, WA, WB, A, B, retVal):
        return load_library().word2vecEvalNegBf16(nrows, ncols, nwa, nwb, _ptr(WA), _ptr(WB),
                                                  _ptr(A), _ptr(B), _ptr(retVal))


def f32_to_bf16(n, src, dst):
    check(load_library().w2v_f32_to_bf16(n, _ptr(src), _ptr(dst)), "w2v_f32_to_bf16")


def bf16_to_f32(n, src, dst):
    check(load_library().w2v_bf16_to_f32(n, _ptr(src), _ptr(dst)), "w2v_bf16_to_f32")


def wordmats(n, mats, iflip, vocab, nskip, nneg, nreuse, wsample_lnv, wexpt, seed, call, words,
             lb, ub, negs, ctx, counts):
    """w2v_wordmats on device buffers; returns (number of valid pairs, number of groups)."""
    host = (ctypes.c_int * 2)()
    err = load_library().w2v_wordmats(n, _ptr(mats), int(bool(iflip)), vocab, nskip, nneg, nreuse,
                                      wsample_lnv, wexpt, seed, call, _ptr(words), _ptr(lb),
                                      _ptr(ub), _ptr(negs), _ptr(ctx), _ptr(counts), host)
    check(err, "w2v_wordmats")
    return int(host[0]), int(host[1])


class Timer:
    """HIP event pair on the library's launch stream of the calling thread."""

    def __init__(self):
        self._lib = load_library()
        self._h = ctypes.c_void_p()
        err = self._lib.w2v_timer_create(ctypes.byref(self._h))
        if err:
            raise W2VLibraryError("w2v_timer_create: " + error_string(err))

    def start(self):
        err = self._lib.w2v_timer_start(self._h)
        if err:
            raise W2VLibraryError("w2v_timer_start: " + error_string(err))

    def stop(self):
        err = self._lib.w2v_timer_stop(self._h)
        if err:
            raise W2VLibraryError("w2v_timer_stop: " + error_string(err))

    def elapsed_ms(self):
        ms = ctypes.c_float()
        err = self._lib.w2v_timer_elapsed_ms(self._h, ctypes.byref(ms))
        if err:
            raise W2VLibraryError("w2v_timer_elapsed_ms: " + error_string(err))
        return float(ms.value)

    def close(self):
        if self._h:
            self._lib.w2v_timer_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def synchronize():
    err = load_library().w2v_synchronize()
    if err:
        raise W2VLibraryError("w2v_synchronize: " + error_string(err))
