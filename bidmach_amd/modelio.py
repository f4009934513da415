"""Google word2vec model files, as BIDMach.networks.Word2Vec reads and writes them
(src/main/scala/BIDMach/networks/Word2Vec.scala:1332-1394 of the reference).

Layout: a header line "<nwords> <dim>\\n", then per word its string, one space, `dim` values and a
newline.  Text files print each value with "%g " (:1385); binary files hold raw IEEE floats.  The
reference writes binary values through java.io.DataOutputStream.writeFloat (:1383) and reads them
with DataInputStream.readFloat (:1350), i.e. BIG-endian, whereas Google's own tool writes
little-endian; `byteorder` selects which (default: the reference's).

A model matrix here is the (vocab, dim) C-order array the operators use (word w's vector is row
w), which is the reference's dim x vocab column-major FMat.
"""
import numpy as np


def saveGoogleW2V(words, mod, fname, binary=False, byteorder=">"):
    """words: sequence of strings (the dictionary, id order); mod: (vocab, dim) float32."""
    mod = np.asarray(mod, dtype=np.float32)
    nwords = min(mod.shape[0], len(words))      # the reference warns and truncates (:1369-1374)
    dim = mod.shape[1]
    with open(fname, "wb") as f:
        f.write(("%d %d\n" % (nwords, dim)).encode())
        for i in range(nwords):
            f.write(words[i].encode("utf-8") + b" ")
            if binary:
                f.write(mod[i].astype(byteorder + "f4").tobytes())
            else:
                f.write("".join("%g " % v for v in mod[i]).encode())
            f.write(b"\n")


def readGoogleW2V(fname, dictionary, n, binary=False, byteorder=">"):
    """dictionary: dict word -> id.  Returns an (n, dim) float32 matrix holding the vectors of
    the words whose id is in [0, n); other words are skipped, missing ones stay zero (:1344-1356)."""
    with open(fname, "rb") as f:
        header = f.readline().split()
        nr, dim = int(header[0]), int(header[1])
        model = np.zeros((n, dim), dtype=np.float32)
        for _ in range(nr):
            if binary:
                word = bytearray()
                while True:
                    c = f.read(1)
                    if not c:
                        raise EOFError("truncated word2vec file %s" % fname)
                    if c == b" ":
                        break
                    if c != b"\n" or word:          # tolerate the newline that ends a record
                        word += c
                vec = np.frombuffer(f.read(4 * dim), dtype=byteorder + "f4")
                if vec.shape[0] != dim:
                    raise EOFError("truncated word2vec file %s" % fname)
                tail = f.read(1)
                if tail not in (b"\n", b""):
                    f.seek(-1, 1)
                word = word.decode("utf-8")
            else:
                parts = f.readline().split()
                if len(parts) != dim + 1:
                    raise ValueError("bad record in word2vec text file %s" % fname)
                word = parts[0].decode("utf-8")
                vec = np.array([float(x) for x in parts[1:]], dtype=np.float32)
            icol = dictionary.get(word, -1)
            if 0 <= icol < n:
                model[icol] = vec
        return model
