"""The C-ABI library loads and exports every function include/bidmach_w2v.h declares (no GPU)."""
import os
import re
import subprocess

import pytest

from bidmach_amd import cumach

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bidmach_w2v.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//.*", "", text)
    return sorted(set(re.findall(r"\b(word2vec\w+|w2v_\w+)\s*\(", text)))


def test_header_declares_the_four_reference_entry_points():
    names = declared_functions()
    for n in ("word2vecPos", "word2vecNeg", "word2vecEvalPos", "word2vecEvalNeg"):
        assert n in names


def test_library_exports_every_declared_symbol():
    if not os.path.exists(cumach.lib_path()):
        pytest.fail("HIP library not built: run `python -m bidmach_amd.build`")
    lib = cumach.load_library()
    names = declared_functions()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n
    out = subprocess.check_output(["nm", "-D", "--defined-only", cumach.lib_path()], text=True)
    exported = set(line.split()[-1] for line in out.splitlines() if " T " in line)
    for n in names:
        assert n in exported, n


def test_python_binding_covers_the_header():
    assert sorted(cumach.SYMBOLS) == declared_functions()


def test_header_compiles_as_c():
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c",
                           HEADER])


def test_limits_and_floor_without_gpu():
    lib = cumach.load_library()
    assert lib.w2v_max_rows() == 1280
    assert lib.w2v_max_nwb() == 64
    assert lib.w2v_get_eval_floor() == 1.0e-40
    lib.w2v_set_eval_floor(1.0e-20)
    assert lib.w2v_get_eval_floor() == 1.0e-20
    lib.w2v_set_eval_floor(1.0e-40)


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(cumach.W2VLibraryError):
        cumach.load_library(str(tmp_path / "nope.so"))


def test_jni_glue_binds_the_reference_natives_to_declared_functions():
    """jni/cumach_w2v_jni.cpp (built only where a JDK is installed) defines one
    Java_edu_berkeley_bid_CUMACH_<name> per native the reference's Java class declares for this
    path (CUMACH.java:90,92,94,96,98) and forwards each to the C function of the same name."""
    text = open(os.path.join(ROOT, "jni", "cumach_w2v_jni.cpp")).read()
    declared = declared_functions()
    for n in ("word2vecPos", "word2vecNeg", "word2vecNegFilt", "word2vecEvalPos",
              "word2vecEvalNeg"):
        assert re.search(r"Java_edu_berkeley_bid_CUMACH_%s\(" % n, text), n
        assert re.search(r"return %s\(" % n, text), n
        assert n in declared
    assert "JNI_OnLoad" in text and "nativePointer" in text and "byteOffset" in text


def test_release_thread_without_scratch_is_a_no_op():
    assert cumach.load_library().w2v_release_thread() == 0


def test_jni_makefile_rebuilds_the_glue_and_the_alias_follows_it(tmp_path):
    """jni/Makefile builds the glue into a regular file of its own, so make's time-stamp test
    works (a target that is a symbolic link to the HIP library would always look up to date), and
    bidmach_amd/build.py points the reference's artefact name at the glue only where it exists.
    Dry run against a JAVA_HOME that holds an (empty) include/jni.h: nothing is compiled."""
    import shutil
    import subprocess
    if shutil.which("make") is None:
        pytest.skip("no make")
    from bidmach_amd import build
    (tmp_path / "include").mkdir()
    (tmp_path / "include" / "jni.h").write_text("")
    out = subprocess.run(["make", "-n", "-C", os.path.join(ROOT, "jni"), "JAVA_HOME=%s" % tmp_path],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert out.returncode == 0, out.stdout
    if not os.path.exists(build.JNI_PATH):
        assert "cumach_w2v_jni.cpp" in out.stdout and build.JNI_NAME in out.stdout, out.stdout
    assert build.JNI_NAME != build.ALIAS_NAME
    none = subprocess.run(["make", "-n", "-C", os.path.join(ROOT, "jni"), "JAVA_HOME=/nonexistent"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert none.returncode == 0 and "not built" in none.stdout
    if os.path.lexists(build.ALIAS_PATH):
        want = build.JNI_NAME if os.path.isfile(build.JNI_PATH) else build.LIB_NAME
        assert os.readlink(build.ALIAS_PATH) == want
