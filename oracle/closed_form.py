"""float64 numpy statement of the SGNS mathematics (TEST INFRASTRUCTURE).

This is not a transcription of the C oracle: it states skip-gram negative sampling the way a
textbook does, over the whole minibatch at once, with every dot product taken from the
pre-call snapshot of the tables ("snapshot semantics"):

    positives   L+ = sum over valid (centre i, context p) of log s(A[w_i] . B[w_p])
                dA[w_i] += ascale_i * lr * (1 - s) * B[w_p]
                dB[w_p] += bscale_p * lr * (1 - s) * A[w_i]
    negatives   L- = sum over groups g, k < nwb, j < nwa of log(1 - s(A[wa_gj] . B[wb_gk]))
                dA[wa_gj] += ascale * (-lr * s) * B[wb_gk]
                dB[wb_gk] += bscale * (-lr * s) * A[wa_gj]

with s the saturating logistic function of the reference (exactly 1 above 16, exactly 0 below
-16; jni/src/BIDMach_CPUMACH.c:48-55) and scale = (1 + id) ** vexp (:33,42,215,222).
On a collision-free minibatch (every column touched by one work unit only) the sequential
CPU result equals these sums, which is what pins the C oracle in tests/test_oracle.py.
The valid-pair rule is the reference's: W[i] >= 0, LB[i] <= j <= UB[i], j != 0,
0 <= i+j < ncols, W[i+j] >= 0 (:30-41).
"""
import numpy as np


def sat_sigmoid(s):
    s = np.asarray(s, dtype=np.float64)
    out = 1.0 / (1.0 + np.exp(-np.clip(s, -40.0, 40.0)))
    out = np.where(s > 16.0, 1.0, out)
    out = np.where(s < -16.0, 0.0, out)
    return out


def valid_pairs(W, LB, UB):
    """(centre position, context position) of every valid pair, in centre-major order."""
    W = np.asarray(W)
    n = W.shape[0]
    if n == 0:
        return np.zeros(0, np.int64), np.zeros(0, np.int64)
    lo = int(min(LB.min(), 0))
    hi = int(max(UB.max(), 0))
    ci, pi = [], []
    idx = np.arange(n, dtype=np.int64)
    for j in range(lo, hi + 1):
        if j == 0:
            continue
        p = idx + j
        ok = (W >= 0) & (LB <= j) & (j <= UB) & (p >= 0) & (p < n)
        ok[ok] &= W[p[ok]] >= 0
        ci.append(idx[ok])
        pi.append(p[ok])
    ci = np.concatenate(ci)
    pi = np.concatenate(pi)
    order = np.lexsort((pi, ci))
    return ci[order], pi[order]


def scale(ids, vexp):
    return (1.0 + np.asarray(ids, dtype=np.float64)) ** float(vexp)


def eval_pos(W, LB, UB, A, B, floor=1.0e-40):
    ci, pi = valid_pairs(W, LB, UB)
    A64 = A.astype(np.float64)
    B64 = B.astype(np.float64)
    s = np.einsum("ij,ij->i", A64[W[ci]], B64[W[pi]])
    return float(np.log(np.maximum(sat_sigmoid(s), floor)).sum())


def eval_neg(nwa, nwb, WA, WB, A, B, floor=1.0e-40):
    WA = np.asarray(WA).reshape(-1, nwa)   # group-major
    WB = np.asarray(WB).reshape(-1, nwb)
    A64 = A.astype(np.float64)
    B64 = B.astype(np.float64)
    s = np.einsum("gjd,gkd->gjk", A64[WA], B64[WB])
    return float(np.log(np.maximum(1.0 - sat_sigmoid(s), floor)).sum())


def pos_update(W, LB, UB, A, B, lrate, vexp):
    """Returns (A_new, B_new) in float64 under snapshot semantics."""
    ci, pi = valid_pairs(W, LB, UB)
    A64 = A.astype(np.float64)
    B64 = B.astype(np.float64)
    wa, wb = W[ci], W[pi]
    s = np.einsum("ij,ij->i", A64[wa], B64[wb])
    g = float(lrate) * (1.0 - sat_sigmoid(s))
    dA = np.zeros_like(A64)
    dB = np.zeros_like(B64)
    np.add.at(dA, wa, (scale(wa, vexp) * g)[:, None] * B64[wb])
    np.add.at(dB, wb, (scale(wb, vexp) * g)[:, None] * A64[wa])
    return A64 + dA, B64 + dB


def neg_update(nwa, nwb, WA, WB, A, B, lrate, vexp):
    WA = np.asarray(WA).reshape(-1, nwa)
    WB = np.asarray(WB).reshape(-1, nwb)
    A64 = A.astype(np.float64)
    B64 = B.astype(np.float64)
    a = A64[WA]                                   # g x nwa x d
    b = B64[WB]                                   # g x nwb x d
    s = np.einsum("gjd,gkd->gjk", a, b)
    g = -float(lrate) * sat_sigmoid(s)            # g x nwa x nwb
    da = scale(WA, vexp)[:, :, None] * np.einsum("gjk,gkd->gjd", g, b)
    db = scale(WB, vexp)[:, :, None] * np.einsum("gjk,gjd->gkd", g, a)
    dA = np.zeros_like(A64)
    dB = np.zeros_like(B64)
    np.add.at(dA, WA.reshape(-1), da.reshape(-1, A.shape[1]))
    np.add.at(dB, WB.reshape(-1), db.reshape(-1, B.shape[1]))
    return A64 + dA, B64 + dB


# ---- sliced, multi-part models ---------------------------------------------------------------
# The reference can split the vocabulary over nslices workers (jni/src/BIDMach_CPUMACH.c:80-88):
# ids below nhead ("head") live on every worker, the others ("tail") on worker id % nslices.
# A worker packs its resident words densely, head first then its tail words in id order, and
# cuts the packed table into parts of maxcols columns.  The functions below state the sliced
# passes on the *logical* full-vocabulary tables with masks, so they share no index arithmetic
# with the C oracle; pack_parts / unpack_parts move between the logical tables and the parts
# one worker holds.

def slice_flags(ids, islice, nslices, nhead):
    ids = np.asarray(ids)
    head = ids < nhead
    mine = (~head) & (ids % nslices == islice)
    return mine, head


def resident_words(vocab, islice, nslices, nhead):
    """Word ids stored by worker islice, in packed-column order."""
    ids = np.arange(vocab)
    mine, head = slice_flags(ids, islice, nslices, nhead)
    return np.concatenate([ids[head], ids[mine]])


def pack_parts(full, islice, nslices, nhead, maxcols):
    """List of (columns, d) arrays: the parts worker islice holds of a logical (vocab, d) table."""
    words = resident_words(full.shape[0], islice, nslices, nhead)
    packed = full[words]
    return [np.ascontiguousarray(packed[s:s + maxcols]) for s in range(0, len(words), maxcols)]


def unpack_parts(parts, full, islice, nslices, nhead):
    """Copy of `full` with the resident words' rows replaced by the parts' contents."""
    words = resident_words(full.shape[0], islice, nslices, nhead)
    out = np.array(full, copy=True)
    out[words] = np.concatenate(parts)[: len(words)]
    return out


def _trained(am, ah, bm, bh, dohead):
    return ((dohead > 1) & ah & bh) | (am & bh) | (bm & ah) | (am & bm)


def pos_update_slice(W, LB, UB, A, B, lrate, vexp, islice, nslices, nhead, dohead):
    """Snapshot-semantics positive pass of one worker on logical tables (:90-184): a pair is
    trained iff both words are resident and at least one is the worker's own (or both are head
    and dohead > 1); a column is written iff it is the worker's own, or head and dohead > 0."""
    ci, pi = valid_pairs(W, LB, UB)
    A64 = A.astype(np.float64)
    B64 = B.astype(np.float64)
    wa, wb = W[ci], W[pi]
    am, ah = slice_flags(wa, islice, nslices, nhead)
    bm, bh = slice_flags(wb, islice, nslices, nhead)
    keep = _trained(am, ah, bm, bh, dohead)
    wa, wb, am, ah, bm, bh = (x[keep] for x in (wa, wb, am, ah, bm, bh))
    s = np.einsum("ij,ij->i", A64[wa], B64[wb])
    g = float(lrate) * (1.0 - sat_sigmoid(s))
    dA = np.zeros_like(A64)
    dB = np.zeros_like(B64)
    wr_a = am | (ah & (dohead > 0))
    wr_b = bm | (bh & (dohead > 0))
    np.add.at(dA, wa[wr_a], ((scale(wa, vexp) * g)[:, None] * B64[wb])[wr_a])
    np.add.at(dB, wb[wr_b], ((scale(wb, vexp) * g)[:, None] * A64[wa])[wr_b])
    return A64 + dA, B64 + dB


def neg_update_slice(nwa, nwb, WA, WB, A, B, lrate, vexp, islice, nslices, nhead, dohead):
    WA = np.asarray(WA).reshape(-1, nwa)
    WB = np.asarray(WB).reshape(-1, nwb)
    A64 = A.astype(np.float64)
    B64 = B.astype(np.float64)
    a = A64[WA]
    b = B64[WB]
    am, ah = slice_flags(WA, islice, nslices, nhead)
    bm, bh = slice_flags(WB, islice, nslices, nhead)
    keep = _trained(am[:, :, None], ah[:, :, None], bm[:, None, :], bh[:, None, :], dohead)
    s = np.einsum("gjd,gkd->gjk", a, b)
    g = np.where(keep, -float(lrate) * sat_sigmoid(s), 0.0)
    da = scale(WA, vexp)[:, :, None] * np.einsum("gjk,gkd->gjd", g, b)
    db = scale(WB, vexp)[:, :, None] * np.einsum("gjk,gjd->gkd", g, a)
    da[~(am | (ah & (dohead > 0)))] = 0.0
    db[~(bm | (bh & (dohead > 0)))] = 0.0
    dA = np.zeros_like(A64)
    dB = np.zeros_like(B64)
    np.add.at(dA, WA.reshape(-1), da.reshape(-1, A.shape[1]))
    np.add.at(dB, WB.reshape(-1), db.reshape(-1, B.shape[1]))
    return A64 + dA, B64 + dB


def eval_pos_slice(W, LB, UB, A, B, islice, nslices, nhead, floor=1.0e-20):
    """Forward score of one worker: pairs whose two words are both resident
    (Word2Vec.scala:1007-1069)."""
    ci, pi = valid_pairs(W, LB, UB)
    wa, wb = W[ci], W[pi]
    am, ah = slice_flags(wa, islice, nslices, nhead)
    bm, bh = slice_flags(wb, islice, nslices, nhead)
    keep = (am | ah) & (bm | bh)
    s = np.einsum("ij,ij->i", A.astype(np.float64)[wa[keep]], B.astype(np.float64)[wb[keep]])
    return float(np.log(np.maximum(sat_sigmoid(s), floor)).sum())


def eval_neg_slice(nwa, nwb, WA, WB, A, B, islice, nslices, nhead, floor=1.0e-20):
    WA = np.asarray(WA).reshape(-1, nwa)
    WB = np.asarray(WB).reshape(-1, nwb)
    am, ah = slice_flags(WA, islice, nslices, nhead)
    bm, bh = slice_flags(WB, islice, nslices, nhead)
    keep = (am | ah)[:, :, None] & (bm | bh)[:, None, :]
    s = np.einsum("gjd,gkd->gjk", A.astype(np.float64)[WA], B.astype(np.float64)[WB])
    return float(np.where(keep, np.log(np.maximum(1.0 - sat_sigmoid(s), floor)), 0.0).sum())
