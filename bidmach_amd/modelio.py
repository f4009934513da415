"""Google word2vec model files, as BIDMach.networks.Word2Vec reads and writes them
(src/main/scala/BIDMach/networks/Word2Vec.scala:1332-1394 of the reference).

Layout: a header line "<nwords> <dim>\\n", then per word its string, one space, `dim` values and a
newline.  Text files print each value with Java's "%g " (:1385; java_g below); binary files hold raw IEEE floats.  The
reference writes binary values through java.io.DataOutputStream.writeFloat (:1383) and reads them
with DataInputStream.readFloat (:1350), i.e. BIG-endian, whereas Google's own tool writes
little-endian; `byteorder` selects which (default: the reference's).

A model matrix here is the (vocab, dim) C-order array the operators use (word w's vector is row
w), which is the reference's dim x vocab column-major FMat.
"""
import math
from decimal import Decimal

import numpy as np


def java_g(v):
    """One value as the reference's writer prints it: Scala's `"%g " format x`
    (Word2Vec.scala:1385) is java.util.Formatter's general-scientific conversion with the default
    precision 6, applied to the float widened to double.  Its rules: round to 6 significant
    digits, half up on the decimal digits; if the rounded magnitude is in [1e-4, 1e6) print it as
    a plain decimal with 6 significant digits in all, trailing zeros kept and no decimal point
    when no fraction digit is left ("0.100000", "12.3457", "123457"); otherwise as d.ddddde+xx
    with a sign and at least two exponent digits ("1.00000e-05", "1.23457e+08").  Zero prints as
    "0.00000", not-a-number as "NaN", the infinities as "Infinity" / "-Infinity".  Unlike C's and
    Python's %g nothing is stripped."""
    x = float(v)
    if math.isnan(x):
        return "NaN"
    if math.isinf(x):
        return "Infinity" if x > 0 else "-Infinity"
    sign = "-" if math.copysign(1.0, x) < 0 else ""
    x = abs(x)
    if x == 0.0:
        return sign + "0.00000"
    # the shortest decimal digits that identify the double, which is what Java rounds
    t = Decimal(repr(x)).as_tuple()
    all_digits = "".join(map(str, t.digits)).lstrip("0")
    exp10 = len(t.digits) + t.exponent - 1 - (len(t.digits) - len(all_digits))
    digits = (all_digits + "000000")[:6]
    if len(all_digits) > 6 and all_digits[6] >= "5":      # half up
        n = int(digits) + 1
        if n == 1000000:
            n, exp10 = 100000, exp10 + 1
        digits = "%06d" % n
    if -4 <= exp10 < 6:
        if exp10 >= 0:
            whole, frac = digits[:exp10 + 1], digits[exp10 + 1:]
            return sign + whole + ("." + frac if frac else "")
        return sign + "0." + "0" * (-exp10 - 1) + digits
    return "%s%s.%se%s%02d" % (sign, digits[0], digits[1:], "-" if exp10 < 0 else "+", abs(exp10))


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
                f.write("".join(java_g(v) + " " for v in mod[i]).encode())
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
