"""Writes tests/golden/sgns_small.npz and tests/golden/sgns_slice_small.npz: small seeded inputs of
the SGNS operators (single-table, and sliced multi-part) with their expected outputs.

The reference holds no golden vector, known-answer test or fixture for its word2vec functions, and
its C implementation cannot be built in this image (it needs jni.h), so these vectors are NOT
reference outputs: they are the outputs of oracle/w2v_oracle.c (single thread), stored together with
the float64 closed-form results of oracle/closed_form.py that pin it.  They guard the oracle and the
HIP library against regressions on fixed inputs, collision-free for the updates.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from bidmach_amd import corpus  # noqa: E402
from oracle import closed_form as cf  # noqa: E402
from oracle.cpumach import CPUMACH  # noqa: E402


def main():
    rng = np.random.default_rng(20240607)
    d, V, skip, nwa, nwb = 20, 256, 3, 4, 3
    A = (rng.standard_normal((V, d)) * 0.4).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.4).astype(np.float32)
    out = dict(d=d, V=V, skip=skip, nwa=nwa, nwb=nwb, A=A, B=B, lrate=np.float32(0.05),
               vexp=np.float32(0.5))

    # forward-only scoring on a colliding, ragged minibatch
    n = 400
    W = corpus.zipf_stream(n, V, 1.0, seed=7)
    W[rng.random(n) < 0.1] = -1
    sent = np.cumsum(rng.random(n) < 0.05)
    LB, UB = corpus.window_bounds(n, skip, rng, sentence=sent)
    WA = rng.integers(0, V, 30 * nwa).astype(np.int32)
    WB = corpus.zipf_stream(30 * nwb, V, 1.0, seed=8)
    out.update(eW=W, eLB=LB, eUB=UB, eWA=WA, eWB=WB,
               evalpos=CPUMACH.word2vecEvalPos(d, n, skip, W, LB, UB, A, B, 1),
               evalneg=CPUMACH.word2vecEvalNeg(d, 30, nwa, nwb, WA, WB, A, B, 1),
               evalpos_closed=cf.eval_pos(W, LB, UB, A, B),
               evalneg_closed=cf.eval_neg(nwa, nwb, WA, WB, A, B))

    # updates on collision-free minibatches
    W, LB, UB = corpus.collision_free_pos(30, skip, V, rng)
    W[rng.random(W.shape[0]) < 0.05] = -1
    Ap, Bp = A.copy(), B.copy()
    CPUMACH.word2vecPos(d, W.shape[0], skip, W, LB, UB, Ap, Bp, 0.05, 0.5, 1)
    Ac, Bc = cf.pos_update(W, LB, UB, A, B, 0.05, 0.5)
    out.update(pW=W, pLB=LB, pUB=UB, posA=Ap, posB=Bp, posA_closed=Ac, posB_closed=Bc)

    WA, WB = corpus.collision_free_neg(30, nwa, nwb, V, rng)
    An, Bn = A.copy(), B.copy()
    CPUMACH.word2vecNeg(d, 30, nwa, nwb, WA, WB, An, Bn, 0.05, 0.5, 1)
    Ac, Bc = cf.neg_update(nwa, nwb, WA, WB, A, B, 0.05, 0.5)
    out.update(nWA=WA, nWB=WB, negA=An, negB=Bn, negA_closed=Ac, negB_closed=Bc)

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sgns_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")
    slice_fixture()


def slice_fixture():
    """One worker (islice 1 of 3, 10 head words, parts of 40 columns, head columns written) of a
    sliced model.  Tables are stored in their logical full-vocabulary form; the parts the worker
    holds are cut from them with closed_form.pack_parts."""
    rng = np.random.default_rng(20240608)
    d, V, skip, nwa, nwb = 12, 256, 2, 3, 2
    islice, nslices, nhead, maxcols, dohead = 1, 3, 10, 40, 1
    sl = (islice, nslices, maxcols, nhead, 0)
    A = (rng.standard_normal((V, d)) * 0.4).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.4).astype(np.float32)
    out = dict(d=d, V=V, skip=skip, nwa=nwa, nwb=nwb, A=A, B=B, lrate=np.float32(0.05),
               vexp=np.float32(0.5), islice=islice, nslices=nslices, nhead=nhead, maxcols=maxcols,
               dohead=dohead)

    def parts(X):
        return cf.pack_parts(X, islice, nslices, nhead, maxcols)

    def mm(bp, ap):
        return [m for pair in zip(bp, ap) for m in pair]

    n = 300
    W = corpus.zipf_stream(n, V, 1.0, seed=17)
    W[rng.random(n) < 0.1] = -1
    LB, UB = corpus.window_bounds(n, skip, rng, sentence=np.cumsum(rng.random(n) < 0.05))
    WA = rng.integers(0, V, 40 * nwa).astype(np.int32)
    WB = corpus.zipf_stream(40 * nwb, V, 1.0, seed=18)
    m = mm(parts(B), parts(A))
    out.update(eW=W, eLB=LB, eUB=UB, eWA=WA, eWB=WB,
               evalpos=CPUMACH.word2vecEvalPosSlice(d, n, skip, W, LB, UB, m, 1, *sl),
               evalneg=CPUMACH.word2vecEvalNegSlice(d, 40, nwa, nwb, WA, WB, m, 1, *sl),
               evalpos_closed=cf.eval_pos_slice(W, LB, UB, A, B, islice, nslices, nhead),
               evalneg_closed=cf.eval_neg_slice(nwa, nwb, WA, WB, A, B, islice, nslices, nhead))

    W, LB, UB = corpus.collision_free_pos(50, skip, V, rng)
    ap, bp = parts(A), parts(B)
    CPUMACH.word2vecPosSlice(d, W.shape[0], skip, W, LB, UB, mm(bp, ap), 0.05, 0.5, 1, *sl, dohead)
    Ac, Bc = cf.pos_update_slice(W, LB, UB, A, B, 0.05, 0.5, islice, nslices, nhead, dohead)
    out.update(pW=W, pLB=LB, pUB=UB, posA=cf.unpack_parts(ap, A, islice, nslices, nhead),
               posB=cf.unpack_parts(bp, B, islice, nslices, nhead), posA_closed=Ac, posB_closed=Bc)

    WA, WB = corpus.collision_free_neg(50, nwa, nwb, V, rng)
    ap, bp = parts(A), parts(B)
    CPUMACH.word2vecNegSlice(d, 50, nwa, nwb, WA, WB, mm(bp, ap), 0.05, 0.5, 1, *sl, dohead)
    Ac, Bc = cf.neg_update_slice(nwa, nwb, WA, WB, A, B, 0.05, 0.5, islice, nslices, nhead, dohead)
    out.update(nWA=WA, nWB=WB, negA=cf.unpack_parts(ap, A, islice, nslices, nhead),
               negB=cf.unpack_parts(bp, B, islice, nslices, nhead), negA_closed=Ac, negB_closed=Bc)

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sgns_slice_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
