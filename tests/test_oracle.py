"""Pins the C oracle (oracle/w2v_oracle.c) without running any reference code.

The reference holds no test, fixture or golden vector for the word2vec functions, and its C file
cannot be built in this image (it includes <jni.h>).  Each check below is chosen so that a
plausible mistake in the restatement fails it: float64 closed forms on collision-free
minibatches (dropped term, wrong sign, transposed operand, wrong scale), brute-force enumeration
of the pair rule on tiny inputs (window/validity logic), exact special cases of the clamps and
the floor, no-op invariants, and two-pair analytic cases that depend on the update order
(B immediately, A after the window; jni/src/BIDMach_CPUMACH.c:57-67, 239-254).
"""
import math

import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import closed_form as cf

C_FLOOR = 1.0e-40
LOG_FLOOR = math.log(1.0e-40)


def rand_tables(rng, vocab, d, scale=0.3):
    A = (rng.standard_normal((vocab, d)) * scale).astype(np.float32)
    B = (rng.standard_normal((vocab, d)) * scale).astype(np.float32)
    return A, B


def brute_pairs(W, LB, UB):
    """The pair rule spelled out position by position."""
    n = len(W)
    out = []
    for i in range(n):
        if W[i] < 0:
            continue
        for p in range(n):
            j = p - i
            if j == 0 or j < LB[i] or j > UB[i] or W[p] < 0:
                continue
            out.append((i, p))
    return out


# ---------------------------------------------------------------------------------------------
# Eval functions
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("seed", [0, 1, 2])
def test_eval_pos_brute_force_tiny(oracle, seed):
    rng = np.random.default_rng(seed)
    d, V, N = 4, 8, 6
    A, B = rand_tables(rng, V, d, 1.0)
    W = rng.integers(-1, V, N).astype(np.int32)
    LB = -rng.integers(0, 4, N).astype(np.int32)
    UB = rng.integers(0, 4, N).astype(np.int32)
    want = 0.0
    for i, p in brute_pairs(W, LB, UB):
        s = float(np.dot(A[W[i]].astype(np.float64), B[W[p]].astype(np.float64)))
        want += math.log(1.0 / (1.0 + math.exp(-s)))
    got = oracle.word2vecEvalPos(d, N, 3, W, LB, UB, A, B, 1)
    assert got == pytest.approx(want, rel=1e-6, abs=1e-6)
    assert cf.eval_pos(W, LB, UB, A, B) == pytest.approx(want, rel=1e-12, abs=1e-12)


def test_eval_neg_brute_force_tiny(oracle):
    rng = np.random.default_rng(3)
    d, V, G, nwa, nwb = 4, 8, 3, 3, 2
    A, B = rand_tables(rng, V, d, 1.0)
    WA = rng.integers(0, V, G * nwa).astype(np.int32)
    WB = rng.integers(0, V, G * nwb).astype(np.int32)
    want = 0.0
    for g in range(G):
        for k in range(nwb):
            for j in range(nwa):
                s = float(np.dot(A[WA[g * nwa + j]].astype(np.float64),
                                 B[WB[g * nwb + k]].astype(np.float64)))
                want += math.log(1.0 - 1.0 / (1.0 + math.exp(-s)))
    got = oracle.word2vecEvalNeg(d, G, nwa, nwb, WA, WB, A, B, 1)
    assert got == pytest.approx(want, rel=1e-6)
    assert cf.eval_neg(nwa, nwb, WA, WB, A, B) == pytest.approx(want, rel=1e-12)


@pytest.mark.parametrize("d,V,N,skip", [(100, 500, 4000, 5), (300, 200, 1000, 10), (7, 50, 300, 3)])
def test_eval_closed_form_random(oracle, d, V, N, skip):
    rng = np.random.default_rng(d)
    A, B = rand_tables(rng, V, d, 0.2)
    W = corpus.zipf_stream(N, V, 1.0, seed=5)
    W[rng.random(N) < 0.1] = -1
    sent = np.cumsum(rng.random(N) < 0.05)
    LB, UB = corpus.window_bounds(N, skip, rng, sentence=sent)
    got = oracle.word2vecEvalPos(d, N, skip, W, LB, UB, A, B, 3)
    assert got == pytest.approx(cf.eval_pos(W, LB, UB, A, B), rel=2e-6)
    WA, WB, G = corpus.negative_groups(W, LB, UB, 5, 5, rng, vocab=V)
    got = oracle.word2vecEvalNeg(d, G, 5, 5, WA, WB, A, B, 3)
    assert got == pytest.approx(cf.eval_neg(5, 5, WA, WB, A, B), rel=2e-6)


def test_eval_zero_tables_is_pairs_log_half(oracle):
    rng = np.random.default_rng(0)
    d, V, N = 16, 40, 200
    A = np.zeros((V, d), np.float32)
    B = np.zeros((V, d), np.float32)
    W = rng.integers(-1, V, N).astype(np.int32)
    LB, UB = corpus.window_bounds(N, 4, rng)
    npairs, _ = corpus.count_pairs(W, LB, UB)
    assert npairs == len(brute_pairs(W, LB, UB))
    got = oracle.word2vecEvalPos(d, N, 4, W, LB, UB, A, B, 2)
    assert got == pytest.approx(npairs * math.log(0.5), rel=1e-12)
    WA = rng.integers(0, V, 30).astype(np.int32)
    WB = rng.integers(0, V, 20).astype(np.int32)
    got = oracle.word2vecEvalNeg(d, 10, 3, 2, WA, WB, A, B, 2)
    assert got == pytest.approx(60 * math.log(0.5), rel=1e-12)


@pytest.mark.parametrize("s,pos_want,neg_want,neg_abs", [
    (16.5, 0.0, LOG_FLOOR, 1e-9),                 # above the clamp: sigma is exactly 1
    (-16.5, LOG_FLOOR, 0.0, 1e-9),                # below the clamp: sigma is exactly 0
    # on the clamp the smooth branch still applies; sigma = 1 - 2 ulp as a float, so
    # log(1 - sigma) is only near -16 (and far from the floor's -92.1)
    (16.0, -math.log1p(math.exp(-16.0)), -16.0, 0.1),
    (-16.0, -16.0 - math.log1p(math.exp(-16.0)), -math.log1p(math.exp(-16.0)), 2e-7),
])
def test_sigmoid_clamps_and_floor(oracle, s, pos_want, neg_want, neg_abs):
    A = np.array([[1.0], [0.0]], np.float32)
    B = np.array([[0.0], [s]], np.float32)
    W = np.array([0, 1], np.int32)         # centre word 0, context word 1
    LB = np.array([0, 0], np.int32)
    UB = np.array([1, 0], np.int32)
    got = oracle.word2vecEvalPos(1, 2, 1, W, LB, UB, A, B, 1)
    assert got == pytest.approx(pos_want, rel=1e-6, abs=2e-7)
    WA = np.array([0], np.int32)
    WB = np.array([1], np.int32)
    got = oracle.word2vecEvalNeg(1, 1, 1, 1, WA, WB, A, B, 1)
    assert got == pytest.approx(neg_want, rel=1e-6, abs=neg_abs)


def test_eval_floor_parameter(oracle):
    A = np.array([[1.0], [0.0]], np.float32)
    B = np.array([[0.0], [-20.0]], np.float32)
    W = np.array([0, 1], np.int32)
    LB = np.array([0, 0], np.int32)
    UB = np.array([1, 0], np.int32)
    assert oracle.word2vecEvalPos(1, 2, 1, W, LB, UB, A, B, 1, floor=1e-20) == \
        pytest.approx(math.log(1e-20), rel=1e-12)
    assert oracle.word2vecEvalPos(1, 2, 1, W, LB, UB, A, B, 1) == \
        pytest.approx(math.log(1e-40), rel=1e-12)


# ---------------------------------------------------------------------------------------------
# Update functions: closed forms on collision-free minibatches
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("vexp", [0.0, 0.5, 1.0, 0.3])
@pytest.mark.parametrize("d,skip", [(100, 5), (33, 2)])
def test_pos_update_closed_form(oracle, vexp, d, skip):
    rng = np.random.default_rng(11)
    V = 2000
    A, B = rand_tables(rng, V, d, 0.3)
    W, LB, UB = corpus.collision_free_pos(40, skip, V, rng)
    W[rng.random(W.shape[0]) < 0.1] = -1
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPos(d, W.shape[0], skip, W, LB, UB, A2, B2, 0.05, vexp, 1)
    Aw, Bw = cf.pos_update(W, LB, UB, A, B, 0.05, vexp)
    tol = 2e-6 * max(1.0, (1 + V) ** vexp)
    np.testing.assert_allclose(A2, Aw, rtol=0, atol=tol)
    np.testing.assert_allclose(B2, Bw, rtol=0, atol=tol)
    assert np.abs(A2 - A).max() > 1e-4 and np.abs(B2 - B).max() > 1e-4


@pytest.mark.parametrize("vexp", [0.0, 0.5, 1.0, 0.3])
@pytest.mark.parametrize("d,nwa,nwb", [(100, 5, 5), (20, 15, 5), (9, 1, 3)])
def test_neg_update_closed_form(oracle, vexp, d, nwa, nwb):
    rng = np.random.default_rng(12)
    V, G = 3000, 50
    A, B = rand_tables(rng, V, d, 0.3)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, A2, B2, 0.05, vexp, 1)
    Aw, Bw = cf.neg_update(nwa, nwb, WA, WB, A, B, 0.05, vexp)
    tol = 2e-6 * max(1.0, (1 + V) ** vexp)
    np.testing.assert_allclose(A2, Aw, rtol=0, atol=tol)
    np.testing.assert_allclose(B2, Bw, rtol=0, atol=tol)
    assert np.abs(A2 - A).max() > 1e-4 and np.abs(B2 - B).max() > 1e-4


def test_neg_filt_drops_pairs_with_filtered_ids(oracle):
    """word2vecNegFilt: ids >= nwords take no part (DNN127.cu:690-711).  On a collision-free
    minibatch the result is the closed form over the surviving ids of each group."""
    rng = np.random.default_rng(14)
    d, V, G, nwa, nwb, nwords = 16, 3000, 60, 5, 4, 2000
    A, B = rand_tables(rng, V, d, 0.3)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    assert (WA >= nwords).any() and (WB >= nwords).any()
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecNegFilt(d, G, nwords, nwa, nwb, WA, WB, A2, B2, 0.05, 0.5, 1)
    Aw, Bw = A.astype(np.float64), B.astype(np.float64)
    for g in range(G):
        wa = WA[g * nwa:(g + 1) * nwa]
        wb = WB[g * nwb:(g + 1) * nwb]
        wa, wb = wa[wa < nwords], wb[wb < nwords]
        if len(wa) and len(wb):
            Ag, Bg = cf.neg_update(len(wa), len(wb), wa, wb, A, B, 0.05, 0.5)
            Aw[wa], Bw[wb] = Ag[wa], Bg[wb]
    np.testing.assert_allclose(A2, Aw, rtol=0, atol=2e-4)
    np.testing.assert_allclose(B2, Bw, rtol=0, atol=2e-4)
    assert np.array_equal(A2[nwords:], A[nwords:]) and np.array_equal(B2[nwords:], B[nwords:])
    # with nwords beyond every id it is word2vecNeg
    A3, B3, A4, B4 = A.copy(), B.copy(), A.copy(), B.copy()
    oracle.word2vecNegFilt(d, G, V, nwa, nwb, WA, WB, A3, B3, 0.05, 0.5, 1)
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, A4, B4, 0.05, 0.5, 1)
    assert np.array_equal(A3, A4) and np.array_equal(B3, B4)


def test_first_minibatch_identity(oracle):
    """A == 0 (the model's start, Word2Vec.scala:117): dB = 0 and dA = ascale*lr*0.5*sum(B_ctx)."""
    rng = np.random.default_rng(5)
    d, V, skip, vexp, lr = 24, 400, 3, 0.5, 0.1
    B = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    A = np.zeros((V, d), np.float32)
    W, LB, UB = corpus.collision_free_pos(20, skip, V, rng)
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPos(d, W.shape[0], skip, W, LB, UB, A2, B2, lr, vexp, 1)
    assert np.array_equal(B2, B)
    for c in np.flatnonzero(UB > 0):
        ctx = [W[c + j] for j in range(-skip, skip + 1) if j != 0]
        want = math.sqrt(1 + W[c]) * lr * 0.5 * B[ctx].astype(np.float64).sum(0)
        np.testing.assert_allclose(A2[W[c]], want, rtol=1e-5, atol=1e-7)


def test_noop_invariants(oracle):
    rng = np.random.default_rng(6)
    d, V, N = 12, 100, 300
    A, B = rand_tables(rng, V, d)
    W = rng.integers(0, V, N).astype(np.int32)
    LB, UB = corpus.window_bounds(N, 5, rng)
    WA = rng.integers(0, V, 50).astype(np.int32)
    WB = rng.integers(0, V, 50).astype(np.int32)
    # lrate = 0
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPos(d, N, 5, W, LB, UB, A2, B2, 0.0, 0.5, 2)
    oracle.word2vecNeg(d, 10, 5, 5, WA, WB, A2, B2, 0.0, 0.5, 2)
    assert np.array_equal(A2, A) and np.array_equal(B2, B)
    # every word dropped
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPos(d, N, 5, np.full(N, -1, np.int32), LB, UB, A2, B2, 0.1, 0.5, 2)
    assert np.array_equal(A2, A) and np.array_equal(B2, B)
    # empty windows
    Z = np.zeros(N, np.int32)
    oracle.word2vecPos(d, N, 5, W, Z, Z, A2, B2, 0.1, 0.5, 2)
    assert np.array_equal(A2, A) and np.array_equal(B2, B)
    assert oracle.word2vecEvalPos(d, N, 5, W, Z, Z, A, B, 2) == 0.0
    # empty minibatch
    E = np.zeros(0, np.int32)
    oracle.word2vecPos(d, 0, 5, E, E, E, A2, B2, 0.1, 0.5, 2)
    oracle.word2vecNeg(d, 0, 5, 5, E, E, A2, B2, 0.1, 0.5, 2)
    assert np.array_equal(A2, A) and np.array_equal(B2, B)
    assert oracle.word2vecEvalNeg(d, 0, 5, 5, E, E, A, B, 2) == 0.0


def test_window_clipped_at_minibatch_edges(oracle):
    """Offsets that leave [0, ncols) are skipped, not wrapped (BIDMach_CPUMACH.c:38)."""
    rng = np.random.default_rng(8)
    d, V, N = 8, 50, 6
    A, B = rand_tables(rng, V, d, 1.0)
    W = rng.permutation(V)[:N].astype(np.int32)
    LB = np.full(N, -10, np.int32)
    UB = np.full(N, 10, np.int32)
    want = 0.0
    for i in range(N):
        for p in range(N):
            if p != i:
                s = float(np.dot(A[W[i]].astype(np.float64), B[W[p]].astype(np.float64)))
                want += -math.log1p(math.exp(-s))
    assert oracle.word2vecEvalPos(d, N, 10, W, LB, UB, A, B, 1) == pytest.approx(want, rel=1e-6)


def test_thread_count_independent_on_collision_free(oracle):
    rng = np.random.default_rng(9)
    d, V, skip = 50, 3000, 4
    A, B = rand_tables(rng, V, d)
    W, LB, UB = corpus.collision_free_pos(60, skip, V, rng)
    outs = []
    for nt in (1, 3, 8):
        A2, B2 = A.copy(), B.copy()
        oracle.word2vecPos(d, W.shape[0], skip, W, LB, UB, A2, B2, 0.05, 0.5, nt)
        outs.append((A2, B2))
    for A2, B2 in outs[1:]:
        assert np.array_equal(A2, outs[0][0]) and np.array_equal(B2, outs[0][1])
    WA, WB = corpus.collision_free_neg(40, 5, 5, V, rng)
    outs = []
    for nt in (1, 3, 8):
        A2, B2 = A.copy(), B.copy()
        oracle.word2vecNeg(d, 40, 5, 5, WA, WB, A2, B2, 0.05, 0.5, nt)
        outs.append((A2, B2))
    for A2, B2 in outs[1:]:
        assert np.array_equal(A2, outs[0][0]) and np.array_equal(B2, outs[0][1])


# ---------------------------------------------------------------------------------------------
# Update order on colliding input (sequential semantics), derived by hand
# ---------------------------------------------------------------------------------------------

def _sig(s):
    return 1.0 / (1.0 + math.exp(-s))


def test_pos_order_b_immediate_a_deferred(oracle):
    """One centre whose two context positions hold the same word x.  The second pair must see
    B[x] already updated by the first, while A[c] stays at its old value until the window ends."""
    rng = np.random.default_rng(21)
    d, lr, vexp = 6, 0.5, 0.5
    A, B = rand_tables(rng, 4, d, 0.8)
    c, x = 2, 1
    W = np.array([c, x, x], np.int32)
    LB = np.zeros(3, np.int32)
    UB = np.array([2, 0, 0], np.int32)
    a = A[c].astype(np.float64)
    b = B[x].astype(np.float64)
    asc, bsc = math.sqrt(1 + c), math.sqrt(1 + x)
    g1 = lr * (1 - _sig(a @ b))
    daa = asc * g1 * b
    b1 = b + bsc * g1 * a
    g2 = lr * (1 - _sig(a @ b1))          # uses the updated B column and the old A column
    daa = daa + asc * g2 * b1
    b2 = b1 + bsc * g2 * a
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPos(d, 3, 2, W, LB, UB, A2, B2, lr, vexp, 1)
    np.testing.assert_allclose(B2[x], b2, rtol=2e-6, atol=2e-6)
    np.testing.assert_allclose(A2[c], a + daa, rtol=2e-6, atol=2e-6)
    # the order matters at this step size: the order-free (snapshot) result is measurably different
    As, Bs = cf.pos_update(W, LB, UB, A, B, lr, vexp)
    assert np.abs(Bs[x] - b2).max() > 1e-3
    others = [w for w in range(4) if w != c]
    assert np.array_equal(A2[others], A[others])
    assert np.array_equal(B2[[0, 2, 3]], B[[0, 2, 3]])


def test_neg_order_b_after_inner_loop_a_after_group(oracle):
    """One group with WB = [x, x] and WA = [p, q]: the second k sees B[x] updated by the first k;
    A columns are written only after both (BIDMach_CPUMACH.c:244-254)."""
    rng = np.random.default_rng(22)
    d, lr, vexp = 5, 0.7, 1.0
    A, B = rand_tables(rng, 5, d, 0.8)
    p, q, x = 0, 3, 2
    WA = np.array([p, q], np.int32)
    WB = np.array([x, x], np.int32)
    ap, aq = A[p].astype(np.float64), A[q].astype(np.float64)
    b = B[x].astype(np.float64)
    sp, sq, sx = 1.0 + p, 1.0 + q, 1.0 + x
    dap = np.zeros(d)
    daq = np.zeros(d)
    for _ in range(2):
        gp = -lr * _sig(ap @ b)
        gq = -lr * _sig(aq @ b)
        dbb = sx * gp * ap + sx * gq * aq
        dap += sp * gp * b
        daq += sq * gq * b
        b = b + dbb
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecNeg(d, 1, 2, 2, WA, WB, A2, B2, lr, vexp, 1)
    np.testing.assert_allclose(B2[x], b, rtol=3e-6, atol=3e-6)
    np.testing.assert_allclose(A2[p], ap + dap, rtol=3e-6, atol=3e-6)
    np.testing.assert_allclose(A2[q], aq + daq, rtol=3e-6, atol=3e-6)
    As, Bs = cf.neg_update(2, 2, WA, WB, A, B, lr, vexp)
    assert np.abs(Bs[x] - b).max() > 1e-3


def test_neg_sign_pushes_scores_down_and_pos_up(oracle):
    """Direction of the step: a positive pair's score rises, a negative pair's falls."""
    rng = np.random.default_rng(23)
    d = 10
    A, B = rand_tables(rng, 4, d, 0.5)
    W = np.array([0, 1], np.int32)
    LB = np.zeros(2, np.int32)
    UB = np.array([1, 0], np.int32)
    before = float(A[0] @ B[1])
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPos(d, 2, 1, W, LB, UB, A2, B2, 0.1, 0.0, 1)
    assert float(A2[0] @ B2[1]) > before
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecNeg(d, 1, 1, 1, np.array([0], np.int32), np.array([1], np.int32), A2, B2,
                       0.1, 0.0, 1)
    assert float(A2[0] @ B2[1]) < before
