"""BIDMat dense-matrix files, as BIDMach reads its word2vec input and writes its checkpoints.

What is mirrored:
  layout        a 16-byte header of four little-endian int32 (type code, nrows, ncols, nnz)
                followed by the elements in column-major order.  Type codes: 110 int32, 120 int64,
                130 float32, 140 float64.  This is what the reference's tokenizer writes for the
                (word id, sentence id) files the Word2Vec learner consumes
                (src/main/C/newparse/utils.cpp:350-365, :423-438, :484-510 of the reference) and what
                BIDMat's saveMat/loadMat use for `modelmat%02d.lz4` (models/Model.scala:259-262,
                :284-292).  nnz is not used for dense matrices (the tokenizer writes nrows or 0).
  compression   chosen by the file name: `.gz` is gzip (utils.cpp:283-340), `.lz4` is the block
                stream of the lz4-java library that BIDMat uses (neither is in the reference tree;
                the framing below is pinned by the one such file the reference ships,
                scripts/networks/modelmat_test.fmat.lz4): per block the 8-byte magic "LZ4Block", a
                token byte (0x10 raw or 0x20 LZ4-compressed, plus log2(block size) - 10), the
                compressed and the original length (int32 LE), the xxHash32 of the original bytes
                (seed 0x9747b28c, low 28 bits), then the block; a block of length 0 ends the stream.

Matrices are numpy arrays of BIDMat's shape (nrows, ncols); files hold them column-major, so
`loadMat` returns a Fortran-ordered array.  A model table kept as (vocab, dim) in C order, as the
rest of this package does, is the transpose view: saveMat(path, table.T) writes it without a copy
and loadMat(path).T gives it back.

The LZ4 block codec is the HIP library's host-side one (w2v_lz4_*); the checksum comes from the
`xxhash` module.
"""
import ctypes
import gzip
import io
import struct

import numpy as np

TYPE_CODES = {np.dtype("<i4"): 110, np.dtype("<i8"): 120, np.dtype("<f4"): 130,
              np.dtype("<f8"): 140}
DTYPES = {v: k for k, v in TYPE_CODES.items()}

LZ4_MAGIC = b"LZ4Block"
LZ4_METHOD_RAW = 0x10
LZ4_METHOD_LZ4 = 0x20
LZ4_SEED = 0x9747B28C
LZ4_BLOCK = 1 << 16          # lz4-java's default block size; token level = log2(size) - 10 = 6


class MatFileError(ValueError):
    pass


def _checksum(data):
    import xxhash
    return xxhash.xxh32(data, seed=LZ4_SEED).intdigest() & 0x0FFFFFFF


def _codec():
    from .cumach import load_library
    return load_library()


def lz4_block_compress(data):
    """One LZ4 block (raw format, no framing)."""
    lib = _codec()
    data = bytes(data)
    cap = lib.w2v_lz4_compress_bound(len(data))
    out = ctypes.create_string_buffer(cap)
    n = lib.w2v_lz4_compress(data, len(data), out, cap)
    if n < 0:
        raise MatFileError("LZ4 compression failed")
    return out.raw[:n]


def lz4_block_decompress(data, original_length):
    lib = _codec()
    data = bytes(data)
    out = ctypes.create_string_buffer(max(original_length, 1))
    n = lib.w2v_lz4_decompress(data, len(data), out, original_length)
    if n != original_length:
        raise MatFileError("malformed LZ4 block")
    return out.raw[:original_length]


class LZ4BlockWriter:
    """File-like writer of an lz4-java block stream: bytes written are cut into blocks of
    `block_size`; a block that does not shrink is stored raw; close() writes the end marker."""

    def __init__(self, f, block_size=LZ4_BLOCK):
        self.f = f
        self.block_size = block_size
        self.level = max(0, int(block_size).bit_length() - 1 - 10)
        self.pending = bytearray()

    def _emit(self, chunk):
        comp = lz4_block_compress(chunk)
        if len(comp) >= len(chunk):
            method, body = LZ4_METHOD_RAW, chunk
        else:
            method, body = LZ4_METHOD_LZ4, comp
        self.f.write(LZ4_MAGIC + struct.pack("<BiiI", method | self.level, len(body), len(chunk),
                                             _checksum(chunk)))
        self.f.write(body)

    def write(self, data):
        view = memoryview(data).cast("B")
        pos = 0
        if self.pending:
            take = min(self.block_size - len(self.pending), len(view))
            self.pending += view[:take]
            pos = take
            if len(self.pending) == self.block_size:
                self._emit(bytes(self.pending))
                self.pending = bytearray()
        while len(view) - pos >= self.block_size:
            self._emit(bytes(view[pos:pos + self.block_size]))
            pos += self.block_size
        if pos < len(view):
            self.pending += view[pos:]

    def close(self):
        if self.pending:
            self._emit(bytes(self.pending))
            self.pending = bytearray()
        self.f.write(LZ4_MAGIC + struct.pack("<BiiI", LZ4_METHOD_RAW | self.level, 0, 0, 0))


def lz4_stream_write(f, payload, block_size=LZ4_BLOCK):
    """Writes `payload` (bytes-like) as an lz4-java block stream."""
    w = LZ4BlockWriter(f, block_size)
    w.write(payload)
    w.close()


def lz4_stream_read(f, verify=True):
    """Reads an lz4-java block stream to its end marker (or end of file); returns the bytes as a
    writable buffer."""
    out = io.BytesIO()
    while True:
        head = f.read(21)
        if len(head) == 0:
            break
        if len(head) != 21 or head[:8] != LZ4_MAGIC:
            raise MatFileError("not an LZ4Block stream")
        token, clen, olen, check = struct.unpack("<BiiI", head[8:])
        method = token & 0xF0
        if clen < 0 or olen < 0 or (olen == 0) != (clen == 0):
            raise MatFileError("corrupt LZ4Block header")
        if olen == 0:
            if check != 0:
                raise MatFileError("corrupt LZ4Block end marker")
            break
        body = f.read(clen)
        if len(body) != clen:
            raise MatFileError("truncated LZ4Block stream")
        if method == LZ4_METHOD_RAW:
            if clen != olen:
                raise MatFileError("corrupt raw block")
            chunk = body
        elif method == LZ4_METHOD_LZ4:
            chunk = lz4_block_decompress(body, olen)
        else:
            raise MatFileError("unknown LZ4Block method 0x%02x" % method)
        if verify and _checksum(chunk) != check:
            raise MatFileError("LZ4Block checksum mismatch")
        out.write(chunk)
    return out.getbuffer()


def _encode(m):
    m = np.asarray(m)
    if m.ndim == 1:
        m = m.reshape(-1, 1)
    if m.ndim != 2:
        raise MatFileError("only dense 2-D matrices are supported")
    dt = m.dtype.newbyteorder("<") if m.dtype.byteorder == ">" else m.dtype
    if np.dtype(dt) not in TYPE_CODES:
        raise MatFileError("unsupported element type %s" % m.dtype)
    body = np.asfortranarray(m.astype(dt, copy=False))
    header = struct.pack("<4i", TYPE_CODES[np.dtype(dt)], m.shape[0], m.shape[1], 0)
    return header, body


def _decode(raw):
    if len(raw) < 16:
        raise MatFileError("file shorter than a matrix header")
    code, nrows, ncols, _nnz = struct.unpack("<4i", raw[:16])
    if code not in DTYPES:
        raise MatFileError("unsupported matrix type code %d" % code)
    dt = DTYPES[code]
    need = nrows * ncols * dt.itemsize
    if nrows < 0 or ncols < 0 or len(raw) - 16 < need:
        raise MatFileError("matrix body shorter than its header says")
    flat = np.frombuffer(raw, dtype=dt, count=nrows * ncols, offset=16)
    return flat.reshape((nrows, ncols), order="F")


def saveMat(path, m):
    """Writes matrix `m` (shape nrows x ncols) to `path`; `.lz4` / `.gz` suffixes compress."""
    header, body = _encode(m)
    # body is Fortran-ordered: its transpose is C-contiguous, so this is the column-major byte run
    data = memoryview(body.T.reshape(-1)).cast("B") if body.size else b""
    if path.endswith(".lz4"):
        with open(path, "wb") as f:
            w = LZ4BlockWriter(f)
            w.write(header)
            w.write(data)
            w.close()
    elif path.endswith(".gz"):
        with gzip.open(path, "wb") as f:
            f.write(header)
            f.write(data)
    else:
        with open(path, "wb") as f:
            f.write(header)
            f.write(data)


def loadMat(path):
    """Reads a dense matrix file; returns a writable, Fortran-ordered (nrows, ncols) array."""
    if path.endswith(".lz4"):
        with open(path, "rb") as f:
            raw = lz4_stream_read(f)
    elif path.endswith(".gz"):
        with gzip.open(path, "rb") as f:
            raw = bytearray(f.read())
    else:
        with open(path, "rb") as f:
            raw = bytearray(f.read())
    return _decode(raw)


# BIDMat's typed entry points, as the reference's scripts call them (e.g. scripts/buildcriteo.ssc:12)
def loadIMat(path):
    m = loadMat(path)
    if m.dtype != np.dtype("<i4"):
        raise MatFileError("%s holds %s, not int32" % (path, m.dtype))
    return m


def loadFMat(path):
    m = loadMat(path)
    if m.dtype != np.dtype("<f4"):
        raise MatFileError("%s holds %s, not float32" % (path, m.dtype))
    return m


def saveIMat(path, m):
    saveMat(path, np.asarray(m, dtype=np.int32))


def saveFMat(path, m):
    saveMat(path, np.asarray(m, dtype=np.float32))
