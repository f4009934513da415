"""Pins the sliced, multi-part functions of the C oracle (oracle/w2v_oracle.c) without running
any reference code.

Three independent anchors: (1) with one worker and one part the sliced functions must reproduce
the plain ones bit for bit (the plain ones are pinned in test_oracle.py); (2) cutting the same
table into several parts must not change a bit; (3) on collision-free minibatches the result,
moved back to the logical full-vocabulary tables, must equal a float64 closed form that states
the reference's rules (jni/src/BIDMach_CPUMACH.c:80-88,137-157,315-349) with boolean masks and
shares no index arithmetic with the C code.  A wrong packed column, a wrong owner test, a
dropped or extra clause of the pair rule, or a write to a column the worker may not write fails
one of them.
"""
import math

import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import closed_form as cf


def rand_tables(rng, vocab, d, scale=0.3):
    A = (rng.standard_normal((vocab, d)) * scale).astype(np.float32)
    B = (rng.standard_normal((vocab, d)) * scale).astype(np.float32)
    return A, B


def interleave(bparts, aparts, dual=False):
    """Model-matrix list of the reference: B of part m at 2m, A at 2m+1; with dualMode one more
    pair in front (Word2Vec.scala:118-131)."""
    mm = []
    if dual:
        mm += [np.full_like(bparts[0], 7.0), np.full_like(aparts[0], 7.0)]
    for b, a in zip(bparts, aparts):
        mm += [b, a]
    return mm


def zipf_minibatch(rng, n, vocab):
    W = corpus.zipf_stream(n, vocab, 1.0, seed=int(rng.integers(1 << 30)))
    W[rng.random(n) < 0.05] = -1
    ub = rng.integers(1, 4, n).astype(np.int32)
    return W.astype(np.int32), (-ub).astype(np.int32), ub


# ---- (1) one worker, one part: the plain functions ---------------------------------------------

@pytest.mark.parametrize("nhead,dohead", [(0, 0), (0, 1), (50, 2)])
def test_one_worker_one_part_equals_plain(oracle, nhead, dohead):
    rng = np.random.default_rng(1)
    V, d, n = 50, 12, 400
    A, B = rand_tables(rng, V, d)
    W, LB, UB = zipf_minibatch(rng, n, V)
    WA = rng.integers(0, V, 60 * 3).astype(np.int32)
    WB = rng.integers(0, V, 60 * 2).astype(np.int32)
    A1, B1, A2, B2 = A.copy(), B.copy(), A.copy(), B.copy()
    oracle.word2vecPos(d, n, 3, W, LB, UB, A1, B1, 0.05, 0.5, 1)
    oracle.word2vecNeg(d, 60, 3, 2, WA, WB, A1, B1, 0.02, 0.5, 1)
    oracle.word2vecPosSlice(d, n, 3, W, LB, UB, [B2, A2], 0.05, 0.5, 1, 0, 1, V, nhead, 0, dohead)
    oracle.word2vecNegSlice(d, 60, 3, 2, WA, WB, [B2, A2], 0.02, 0.5, 1, 0, 1, V, nhead, 0, dohead)
    assert np.array_equal(A1, A2) and np.array_equal(B1, B2)
    e1 = oracle.word2vecEvalPos(d, n, 3, W, LB, UB, A1, B1, 1, floor=1e-20)
    e2 = oracle.word2vecEvalPosSlice(d, n, 3, W, LB, UB, [B2, A2], 1, 0, 1, V, nhead, 0)
    assert e1 == e2
    e1 = oracle.word2vecEvalNeg(d, 60, 3, 2, WA, WB, A1, B1, 1, floor=1e-20)
    e2 = oracle.word2vecEvalNegSlice(d, 60, 3, 2, WA, WB, [B2, A2], 1, 0, 1, V, nhead, 0)
    assert e1 == e2


def test_all_head_without_head_training_is_a_noop(oracle):
    """Head-head pairs are trained only when doHead > 1 (:137)."""
    rng = np.random.default_rng(2)
    V, d, n = 40, 8, 200
    A, B = rand_tables(rng, V, d)
    W, LB, UB = zipf_minibatch(rng, n, V)
    for dohead in (0, 1):
        A2, B2 = A.copy(), B.copy()
        oracle.word2vecPosSlice(d, n, 3, W, LB, UB, [B2, A2], 0.05, 0.0, 1, 0, 2, V, V, 0, dohead)
        assert np.array_equal(A, A2) and np.array_equal(B, B2)


# ---- (2) several parts, dual mode ---------------------------------------------------------------

@pytest.mark.parametrize("maxcols", [7, 16, 49])
@pytest.mark.parametrize("dual", [False, True])
def test_cutting_into_parts_changes_nothing(oracle, maxcols, dual):
    rng = np.random.default_rng(3)
    V, d, n = 50, 10, 300
    A, B = rand_tables(rng, V, d)
    W, LB, UB = zipf_minibatch(rng, n, V)
    WA = rng.integers(0, V, 40 * 4).astype(np.int32)
    WB = rng.integers(0, V, 40 * 3).astype(np.int32)
    A1, B1 = A.copy(), B.copy()
    oracle.word2vecPos(d, n, 3, W, LB, UB, A1, B1, 0.05, 0.5, 1)
    oracle.word2vecNeg(d, 40, 4, 3, WA, WB, A1, B1, 0.02, 0.5, 1)
    ap = cf.pack_parts(A, 0, 1, 0, maxcols)
    bp = cf.pack_parts(B, 0, 1, 0, maxcols)
    assert len(ap) == math.ceil(V / maxcols)
    mm = interleave(bp, ap, dual)
    oracle.word2vecPosSlice(d, n, 3, W, LB, UB, mm, 0.05, 0.5, 1, 0, 1, maxcols, 0, dual, 0)
    oracle.word2vecNegSlice(d, 40, 4, 3, WA, WB, mm, 0.02, 0.5, 1, 0, 1, maxcols, 0, dual, 0)
    assert np.array_equal(np.concatenate(ap), A1) and np.array_equal(np.concatenate(bp), B1)
    if dual:       # the leading pair belongs to the device half of a dual-mode model: untouched
        assert np.all(mm[0] == 7.0) and np.all(mm[1] == 7.0)
    e1 = oracle.word2vecEvalPos(d, n, 3, W, LB, UB, A1, B1, 1, floor=1e-20)
    assert e1 == oracle.word2vecEvalPosSlice(d, n, 3, W, LB, UB, mm, 1, 0, 1, maxcols, 0, dual)
    e1 = oracle.word2vecEvalNeg(d, 40, 4, 3, WA, WB, A1, B1, 1, floor=1e-20)
    assert e1 == oracle.word2vecEvalNegSlice(d, 40, 4, 3, WA, WB, mm, 1, 0, 1, maxcols, 0, dual)


# ---- (3) closed forms on the logical tables -----------------------------------------------------

SLICINGS = [  # islice, nslices, nhead, maxcols, dohead
    (0, 3, 7, 1000, 0),
    (2, 3, 7, 1000, 1),
    (1, 3, 7, 23, 2),
    (0, 2, 0, 40, 1),
    (3, 4, 64, 50, 2),
]


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead", SLICINGS)
@pytest.mark.parametrize("vexp", [0.0, 0.5])
def test_pos_slice_closed_form(oracle, islice, nslices, nhead, maxcols, dohead, vexp):
    rng = np.random.default_rng(10 + islice)
    V, d, skip = 330, 9, 2
    A, B = rand_tables(rng, V, d)
    W, LB, UB = corpus.collision_free_pos(60, skip, V, rng)
    ap = cf.pack_parts(A, islice, nslices, nhead, maxcols)
    bp = cf.pack_parts(B, islice, nslices, nhead, maxcols)
    mm = interleave(bp, ap)
    oracle.word2vecPosSlice(d, len(W), skip, W, LB, UB, mm, 0.1, vexp, 1, islice, nslices, maxcols,
                            nhead, 0, dohead)
    gotA = cf.unpack_parts(ap, A, islice, nslices, nhead)
    gotB = cf.unpack_parts(bp, B, islice, nslices, nhead)
    wantA, wantB = cf.pos_update_slice(W, LB, UB, A, B, 0.1, vexp, islice, nslices, nhead, dohead)
    assert np.abs(wantA - A).max() > 1e-3 or np.abs(wantB - B).max() > 1e-3   # something trained
    assert np.abs(gotA - wantA).max() < 2e-5 * (1 + V) ** vexp
    assert np.abs(gotB - wantB).max() < 2e-5 * (1 + V) ** vexp


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead", SLICINGS)
@pytest.mark.parametrize("vexp", [0.0, 0.5])
def test_neg_slice_closed_form(oracle, islice, nslices, nhead, maxcols, dohead, vexp):
    rng = np.random.default_rng(20 + islice)
    V, d, nwa, nwb, G = 330, 9, 4, 3, 45
    A, B = rand_tables(rng, V, d)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    ap = cf.pack_parts(A, islice, nslices, nhead, maxcols)
    bp = cf.pack_parts(B, islice, nslices, nhead, maxcols)
    mm = interleave(bp, ap)
    oracle.word2vecNegSlice(d, G, nwa, nwb, WA, WB, mm, 0.1, vexp, 1, islice, nslices, maxcols,
                            nhead, 0, dohead)
    gotA = cf.unpack_parts(ap, A, islice, nslices, nhead)
    gotB = cf.unpack_parts(bp, B, islice, nslices, nhead)
    wantA, wantB = cf.neg_update_slice(nwa, nwb, WA, WB, A, B, 0.1, vexp, islice, nslices, nhead,
                                       dohead)
    assert np.abs(wantA - A).max() > 1e-3 or np.abs(wantB - B).max() > 1e-3
    assert np.abs(gotA - wantA).max() < 2e-5 * (1 + V) ** vexp
    assert np.abs(gotB - wantB).max() < 2e-5 * (1 + V) ** vexp


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead", SLICINGS)
def test_eval_slice_closed_form(oracle, islice, nslices, nhead, maxcols, dohead):
    rng = np.random.default_rng(30 + islice)
    V, d, n = 330, 9, 500
    A, B = rand_tables(rng, V, d, 0.5)
    W, LB, UB = zipf_minibatch(rng, n, V)
    WA = rng.integers(0, V, 80 * 4).astype(np.int32)
    WB = rng.integers(0, V, 80 * 3).astype(np.int32)
    mm = interleave(cf.pack_parts(B, islice, nslices, nhead, maxcols),
                    cf.pack_parts(A, islice, nslices, nhead, maxcols))
    got = oracle.word2vecEvalPosSlice(d, n, 3, W, LB, UB, mm, 1, islice, nslices, maxcols, nhead, 0)
    want = cf.eval_pos_slice(W, LB, UB, A, B, islice, nslices, nhead)
    assert want < -1.0 and got == pytest.approx(want, rel=1e-6)
    got = oracle.word2vecEvalNegSlice(d, 80, 4, 3, WA, WB, mm, 1, islice, nslices, maxcols, nhead, 0)
    want = cf.eval_neg_slice(4, 3, WA, WB, A, B, islice, nslices, nhead)
    assert want < -1.0 and got == pytest.approx(want, rel=1e-6)


def test_eval_slice_brute_force_tiny(oracle):
    """The residency rule spelled out pair by pair, on one part."""
    rng = np.random.default_rng(5)
    V, d, n, nslices, islice, nhead = 12, 4, 10, 3, 1, 3
    A, B = rand_tables(rng, V, d, 1.0)
    W = rng.integers(-1, V, n).astype(np.int32)
    LB = -rng.integers(0, 3, n).astype(np.int32)
    UB = rng.integers(0, 3, n).astype(np.int32)

    def resident(w):
        return w < nhead or w % nslices == islice

    want = 0.0
    for i in range(n):
        for p in range(n):
            j = p - i
            if W[i] < 0 or W[p] < 0 or j == 0 or j < LB[i] or j > UB[i]:
                continue
            if resident(W[i]) and resident(W[p]):
                s = float(np.dot(A[W[i]].astype(np.float64), B[W[p]].astype(np.float64)))
                want += math.log(1.0 / (1.0 + math.exp(-s)))
    mm = interleave(cf.pack_parts(B, islice, nslices, nhead, 100),
                    cf.pack_parts(A, islice, nslices, nhead, 100))
    got = oracle.word2vecEvalPosSlice(d, n, 2, W, LB, UB, mm, 1, islice, nslices, 100, nhead, 0)
    assert got == pytest.approx(want, rel=1e-6, abs=1e-6)


def test_workers_together_train_every_pair_once(oracle):
    """With doHead = 2 on worker 0 only, every pair with at most one tail owner is trained by
    exactly one worker: the head-head pairs by worker 0 and a (tail, head) pair by the tail's
    owner; (tail, tail) pairs of two different owners are trained by nobody.  Summed over the
    workers, the trained-pair count must match that rule."""
    rng = np.random.default_rng(6)
    V, nslices, nhead = 60, 3, 10
    a = rng.integers(0, V, 4000)
    b = rng.integers(0, V, 4000)
    count = np.zeros(4000, np.int64)
    for s in range(nslices):
        am, ah = cf.slice_flags(a, s, nslices, nhead)
        bm, bh = cf.slice_flags(b, s, nslices, nhead)
        count += cf._trained(am, ah, bm, bh, 2 if s == 0 else 0)
    tail_a, tail_b = a >= nhead, b >= nhead
    foreign = tail_a & tail_b & (a % nslices != b % nslices)
    assert np.all(count[foreign] == 0) and np.all(count[~foreign] == 1)
