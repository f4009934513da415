"""Google word2vec file reader/writer in the reference's dialect (Word2Vec.scala:1332-1394)."""
import struct

import numpy as np
import pytest

from bidmach_amd.modelio import java_g, readGoogleW2V, saveGoogleW2V


@pytest.fixture
def model():
    rng = np.random.default_rng(2)
    words = ["the", "of", "and", "naïve", "x-ray", "zebra"]
    mod = rng.standard_normal((6, 5)).astype(np.float32)
    return words, mod


def test_binary_layout_is_big_endian_like_java(tmp_path, model):
    words, mod = model
    p = tmp_path / "m.bin"
    saveGoogleW2V(words, mod, str(p), binary=True)
    raw = p.read_bytes()
    assert raw.startswith(b"6 5\nthe ")
    first = raw[len(b"6 5\nthe "):len(b"6 5\nthe ") + 20]
    assert first == struct.pack(">5f", *mod[0])          # DataOutputStream.writeFloat order
    assert raw[len(b"6 5\nthe ") + 20:len(b"6 5\nthe ") + 21] == b"\n"


@pytest.mark.parametrize("binary", [False, True])
def test_round_trip(tmp_path, model, binary):
    words, mod = model
    p = tmp_path / "m"
    saveGoogleW2V(words, mod, str(p), binary=binary)
    d = {w: i for i, w in enumerate(words)}
    got = readGoogleW2V(str(p), d, 6, binary=binary)
    if binary:
        assert np.array_equal(got, mod)
    else:
        np.testing.assert_allclose(got, mod, rtol=1e-5)      # "%g" keeps 6 significant digits


def test_reader_skips_unknown_and_out_of_range_words(tmp_path, model):
    words, mod = model
    p = tmp_path / "m.txt"
    saveGoogleW2V(words, mod, str(p))
    d = {"of": 0, "zebra": 1, "and": 7}                       # "and" maps beyond n
    got = readGoogleW2V(str(p), d, 3)
    np.testing.assert_allclose(got[0], mod[1], rtol=1e-5)
    np.testing.assert_allclose(got[1], mod[5], rtol=1e-5)
    assert np.all(got[2] == 0)


def test_writer_truncates_to_the_shorter_of_dictionary_and_model(tmp_path, model):
    words, mod = model
    p = tmp_path / "m.txt"
    saveGoogleW2V(words[:4], mod, str(p))
    assert p.read_text(encoding="utf-8").splitlines()[0] == "4 5"
    saveGoogleW2V(words, mod[:3], str(p))
    assert p.read_text(encoding="utf-8").splitlines()[0] == "3 5"


def test_little_endian_option_reads_google_native_files(tmp_path, model):
    words, mod = model
    p = tmp_path / "g.bin"
    with open(p, "wb") as f:                                   # as Google's C tool writes
        f.write(b"6 5\n")
        for w, v in zip(words, mod):
            f.write(w.encode("utf-8") + b" " + v.astype("<f4").tobytes() + b"\n")
    got = readGoogleW2V(str(p), {w: i for i, w in enumerate(words)}, 6, binary=True, byteorder="<")
    assert np.array_equal(got, mod)


# Strings derived by hand from the rules of java.util.Formatter's %g (general scientific,
# default precision 6: six significant digits, half up; plain decimal for rounded magnitudes in
# [1e-4, 1e6) with trailing zeros kept, d.ddddde+xx with at least two exponent digits otherwise),
# which is what the reference's `"%g " format x` prints (Word2Vec.scala:1385).  No JVM is
# available here, so these rules and strings are the pin.
JAVA_G = [
    (0.1, "0.100000"), (1e-5, "1.00000e-05"), (123456789.0, "1.23457e+08"), (1.0, "1.00000"),
    (-2.5, "-2.50000"), (100000.0, "100000"), (123456.7, "123457"), (999999.4, "999999"),
    (999999.5, "1.00000e+06"), (1e-4, "0.000100000"), (0.00012345678, "0.000123457"),
    (0.000099999949, "9.99999e-05"), (12.345678, "12.3457"), (1e10, "1.00000e+10"),
    (-3.0e-12, "-3.00000e-12"), (0.0, "0.00000"),
    # exact ties go up (half up), where C's printf rounds to even
    (1024.125, "1024.13"), (1234565.0, "1.23457e+06"), (0.5, "0.500000"), (2.0 ** -20, "9.53674e-07"),
    (float("nan"), "NaN"), (float("inf"), "Infinity"), (float("-inf"), "-Infinity"),
]


@pytest.mark.parametrize("value,text", JAVA_G)
def test_java_g_hand_derived_strings(value, text):
    assert java_g(value) == text


def test_java_g_formats_the_float_widened_to_double():
    # the reference passes a Float, which Formatter widens: float32(0.1) = 0.100000001490116...
    assert java_g(np.float32(0.1)) == "0.100000"
    assert java_g(np.float32(16777216.0)) == "1.67772e+07"
    assert java_g(np.float32(1.0e-3)) == "0.00100000"


def test_java_g_equals_c_alternate_form_away_from_ties():
    """C's "%#g" follows the same rules (trailing zeros kept, same switch between the two forms)
    except that it keeps a bare decimal point and rounds exact ties to even: an independent
    library routine for everything but those two points."""
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(20000) * 10.0 ** rng.integers(-9, 10, 20000)).astype(np.float32)
    ties = 0
    for v in x:
        mine, c = java_g(v), "%#g" % float(v)
        c = c[:-1] if c.endswith(".") else c
        if mine != c:
            # only at exact ties, one unit in the last printed digit, away from zero
            tail = ("%.16e" % abs(float(v))).split("e")[0].replace(".", "")[6:]
            assert tail[0] == "5" and not tail[1:].strip("0"), (v, mine, c)
            assert abs(float(mine)) > abs(float(c))
            ties += 1
    assert ties < 200


def test_text_file_bytes_and_reader_round_trip(tmp_path):
    words = ["a", "b"]
    mod = np.array([[0.1, 1e-5, -123456789.0], [0.0, 2.5, 1024.125]], dtype=np.float32)
    p = tmp_path / "m.txt"
    saveGoogleW2V(words, mod, str(p))
    assert p.read_bytes() == (b"2 3\na 0.100000 1.00000e-05 -1.23457e+08 \n"
                              b"b 0.00000 2.50000 1024.13 \n")
    got = readGoogleW2V(str(p), {"a": 0, "b": 1}, 2)
    np.testing.assert_allclose(got, mod, rtol=5e-6)
