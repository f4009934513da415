"""Builds the HIP shared library in-tree with hipcc for gfx950.

    python -m bidmach_amd.build

Objects go to bidmach_amd/csrc/_obj/, the library to bidmach_amd/lib/.  The library name follows
the reference's artefact naming (jni/src/Makefile:11-21: libbidmachcuda-linux-x86_64.so).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "_obj")
LIB_DIR = os.path.join(HERE, "lib")
LIB_NAME = "libbidmachhip-linux-x86_64.so"
LIB_PATH = os.path.join(LIB_DIR, LIB_NAME)
# The name the reference's Java side asks its loader for (CUMACH.java:9 loads "bidmachcuda";
# artefact libbidmachcuda-linux-x86_64.so, jni/src/Makefile:20-21): a link to the JNI glue where a
# JDK let jni/Makefile build it (the glue is linked against the HIP library), else to the HIP
# library itself, so a BIDMach installation finds the operators under the name it already uses.
ALIAS_NAME = "libbidmachcuda-linux-x86_64.so"
ALIAS_PATH = os.path.join(LIB_DIR, ALIAS_NAME)
JNI_NAME = "libbidmachcuda-jni-linux-x86_64.so"
JNI_PATH = os.path.join(LIB_DIR, JNI_NAME)

SOURCES = ["w2v_pos.hip", "w2v_neg.hip", "w2v_neg_wide.hip", "w2v_neg_rows.hip", "w2v_any_shape.hip", "w2v_slice.hip", "w2v_wordmats.hip", "w2v_lz4.hip",
           "w2v_bf16_pos.hip", "w2v_bf16_pos_chain.hip", "w2v_bf16_neg.hip", "w2v_bf16_neg_rows.hip", "w2v_bf16_neg_rows_unaligned.hip", "w2v_api.hip"]

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    "-munsafe-fp-atomics",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    # an unroll pragma that the optimizer does not honour in one large instance is not an error
    "-Wno-pass-failed",
]


def _hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _compile(src, extra):
    out = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", out]
    # the host pass warns that it does not know the packed-fp32 target feature: harmless noise
    res = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if err.strip():
        sys.stderr.write(err + "\n")
    if res.returncode != 0:
        raise subprocess.CalledProcessError(res.returncode, cmd)
    return out


def build(extra_flags=(), verbose=True, out=None):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    extra = list(extra_flags)
    out = out or LIB_PATH
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(lambda s: _compile(s, extra), SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs
    subprocess.check_call(cmd)
    if verbose:
        print("built", out)
    if out == LIB_PATH:
        link_alias(build_jni_glue())
    return out


def build_jni_glue():
    """Runs jni/Makefile (it builds only where it finds jni.h).  True if the glue library is there
    afterwards.  A missing `make` or a failed glue build does not fail the HIP build."""
    try:
        subprocess.check_call(["make", "-s", "-C", os.path.join(os.path.dirname(HERE), "jni")])
    except (OSError, subprocess.CalledProcessError) as e:
        sys.stderr.write("JNI glue not built: %s\n" % e)
        return False
    return os.path.isfile(JNI_PATH)


def link_alias(to_jni):
    if os.path.lexists(ALIAS_PATH):
        os.remove(ALIAS_PATH)
    os.symlink(JNI_NAME if to_jni else LIB_NAME, ALIAS_PATH)


if __name__ == "__main__":
    build(sys.argv[1:])
