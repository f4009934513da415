"""BIDMat dense-matrix files and the LZ4 block stream around them (bidmach_amd/matio.py), and the
checkpoint layout of the Word2Vec mirror.

Pins: the stream framing (magic, token, lengths, xxHash32 seed and mask, end marker) against a file
BIDMat itself wrote, kept as tests/golden/bidmat_written_stream.fmat.lz4 (a copy of the data file
scripts/networks/modelmat_test.fmat.lz4 of the reference: a 3x11x11x96 float tensor, not a word2vec
model; only its stream layer is used); the LZ4 block codec against pyarrow's `lz4_raw` codec in both
directions; the matrix header against the byte layout the reference's tokenizer writes
(src/main/C/newparse/utils.cpp:350-365), spelled out here by hand.
"""
import io
import os
import struct

import numpy as np
import pytest

from bidmach_amd import matio

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                      "bidmat_written_stream.fmat.lz4")


def test_stream_written_by_bidmat_is_read_and_verified():
    with open(GOLDEN, "rb") as f:
        raw = matio.lz4_stream_read(f, verify=True)      # raises on any checksum mismatch
    assert len(raw) == 24 + 4 * 3 * 11 * 11 * 96
    assert struct.unpack("<6i", raw[:24]) == (730, 3, 11, 11, 96, 0)
    x = np.frombuffer(raw, dtype="<f4", offset=24)
    assert np.isfinite(x).all() and 0.005 < float(x.std()) < 0.05


def test_stream_writer_reproduces_the_bidmat_file_byte_for_byte():
    """Same payload, same 64 KiB blocks, incompressible floats stored raw: the writer must emit
    exactly the bytes BIDMat wrote (tokens, lengths, checksums, end marker)."""
    with open(GOLDEN, "rb") as f:
        original = f.read()
    raw = matio.lz4_stream_read(io.BytesIO(original))
    out = io.BytesIO()
    matio.lz4_stream_write(out, raw)
    assert out.getvalue() == original


def test_corrupt_streams_are_rejected():
    with open(GOLDEN, "rb") as f:
        original = bytearray(f.read())
    bad = bytearray(original)
    bad[100] ^= 1                                     # payload bit flip: checksum mismatch
    with pytest.raises(matio.MatFileError):
        matio.lz4_stream_read(io.BytesIO(bytes(bad)))
    with pytest.raises(matio.MatFileError):
        matio.lz4_stream_read(io.BytesIO(bytes(original[:5000])))     # truncated
    with pytest.raises(matio.MatFileError):
        matio.lz4_stream_read(io.BytesIO(b"LZ5Block" + bytes(original[8:])))


@pytest.mark.parametrize("n", [0, 1, 11, 12, 13, 64, 1000, 65536, 200001])
@pytest.mark.parametrize("kind", ["zeros", "text", "ids", "noise"])
def test_block_codec_against_pyarrow(n, kind):
    import pyarrow as pa
    codec = pa.Codec("lz4_raw")
    rng = np.random.default_rng(n)
    if kind == "zeros":
        data = bytes(n)
    elif kind == "text":
        data = (b"the quick brown fox jumps over the lazy dog " * (n // 40 + 1))[:n]
    elif kind == "ids":                                   # what an .imat word file looks like
        data = np.minimum(rng.zipf(1.3, n // 4 + 1), 99999).astype("<i4").tobytes()[:n]
    else:
        data = rng.integers(0, 256, n, dtype=np.uint8).tobytes()
    mine = matio.lz4_block_compress(data)
    assert len(mine) <= n + n // 255 + 16
    if n:
        assert codec.decompress(mine, decompressed_size=n).to_pybytes() == data
        theirs = codec.compress(data).to_pybytes()
        assert matio.lz4_block_decompress(theirs, n) == data
        if kind in ("zeros", "text") and n >= 1000:
            assert len(mine) < n // 4                     # it does compress
    assert matio.lz4_block_decompress(mine, n) == data


def test_malformed_blocks_are_rejected():
    data = b"abcdefgh" * 100
    comp = matio.lz4_block_compress(data)
    with pytest.raises(matio.MatFileError):
        matio.lz4_block_decompress(comp[:-3], len(data))
    with pytest.raises(matio.MatFileError):
        matio.lz4_block_decompress(comp, len(data) - 1)           # output too small
    with pytest.raises(matio.MatFileError):
        matio.lz4_block_decompress(b"\x00\x01\x00", 10)            # match before any output


def test_matrix_header_layout_is_the_tokenizers(tmp_path):
    """fmt, nrows, ncols, nnz as little-endian int32, then the elements column by column."""
    m = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.int32)          # 2 x 3: (word, sentence) rows
    p = str(tmp_path / "w.imat")
    matio.saveIMat(p, m)
    raw = open(p, "rb").read()
    assert raw == struct.pack("<4i", 110, 2, 3, 0) + struct.pack("<6i", 1, 4, 2, 5, 3, 6)
    # a file as the tokenizer writes it for an int vector (nnz = nrows, utils.cpp:350-365)
    q = str(tmp_path / "v.imat")
    open(q, "wb").write(struct.pack("<4i", 110, 4, 1, 4) + struct.pack("<4i", 9, 8, 7, 6))
    assert matio.loadIMat(q).tolist() == [[9], [8], [7], [6]]
    f = str(tmp_path / "x.fmat")
    open(f, "wb").write(struct.pack("<4i", 130, 1, 2, 0) + struct.pack("<2f", 0.5, -2.0))
    assert matio.loadFMat(f).tolist() == [[0.5, -2.0]]
    with pytest.raises(matio.MatFileError):
        matio.loadIMat(f)


@pytest.mark.parametrize("suffix", ["", ".gz", ".lz4"])
@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
def test_round_trip(tmp_path, suffix, dtype):
    rng = np.random.default_rng(3)
    m = (rng.standard_normal((5, 40000)) * 100).astype(dtype)
    p = str(tmp_path / ("m.mat" + suffix))
    matio.saveMat(p, m)
    back = matio.loadMat(p)
    assert back.dtype == np.dtype(dtype) and back.shape == m.shape and np.array_equal(back, m)
    assert back.flags.f_contiguous


def test_word_file_compresses_and_feeds_the_model(tmp_path):
    """A 2 x N (word id, sentence id) file as the Word2Vec learner reads it."""
    from bidmach_amd import corpus
    n = 300000
    words = corpus.zipf_stream(n, 5000, 1.0, seed=1)
    sent = np.cumsum(np.random.default_rng(2).random(n) < 0.04).astype(np.int32)
    mats = np.stack([words, sent]).astype(np.int32)
    p = str(tmp_path / "words.imat.lz4")
    matio.saveIMat(p, mats)
    assert os.path.getsize(p) < 0.8 * mats.nbytes
    back = matio.loadIMat(p)
    assert back.shape == (2, n) and np.array_equal(back, mats)


def test_checkpoint_layout_round_trip(tmp_path):
    """Model.save / Model.load layout: options.json + modelmat%02d.lz4, dim x columns each."""
    from bidmach_amd.word2vec import Options, Word2Vec
    o = Options(vocabSize=900, dim=16, nSlices=2, iSlice=1, nHeadTerms=50, maxArraySize=16 * 200,
                lrate=0.3, seed=5)
    m = Word2Vec(o, device="cpu")
    m.init()
    m.modelmats[1].normal_(0.0, 0.1)
    prefix = str(tmp_path / "ckpt") + os.sep
    m.save(prefix)
    names = sorted(os.listdir(prefix))
    assert names == ["modelmat%02d.lz4" % i for i in range(len(m.modelmats))] + ["options.json"]
    first = matio.loadFMat(prefix + "modelmat00.lz4")
    assert first.shape == (16, 200)                       # BIDMat's shape: dim x columns
    m2 = Word2Vec(Options(dim=16), device="cpu")
    m2.load(prefix)
    assert m2.opts.nSlices == 2 and m2.opts.nHeadTerms == 50 and m2.opts.lrate == 0.3
    assert len(m2.modelmats) == len(m.modelmats)
    for a, b in zip(m.modelmats, m2.modelmats):
        assert a.shape == b.shape and bool((a == b).all())
