"""Google word2vec file reader/writer in the reference's dialect (Word2Vec.scala:1332-1394)."""
import struct

import numpy as np
import pytest

from bidmach_amd.modelio import readGoogleW2V, saveGoogleW2V


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
