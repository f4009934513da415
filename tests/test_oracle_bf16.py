"""Pins of the bfloat16-storage oracle (oracle/w2v_oracle_bf16.c); CPU only.

The reference has no reduced-precision variant, so nothing of its own can pin this oracle.  What
pins it: the fp32 oracle (itself pinned by closed forms in test_oracle.py), the definition of
stochastic rounding (the result is one of the two bfloat16 neighbours of the fp32 value, the upper
one with probability equal to the dropped fraction), and exactness where nothing is dropped.
"""
import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import cpumach

C_FLOOR = cpumach.C_FLOOR


def tables16(rng, vocab, d, scale):
    A = cpumach.bf16_truncate((rng.standard_normal((vocab, d)) * scale).astype(np.float32))
    B = cpumach.bf16_truncate((rng.standard_normal((vocab, d)) * scale).astype(np.float32))
    return A, B


def neighbours_ok(got16, want32):
    """Every stored value is the truncation of the fp32 value or the next bf16 away from zero."""
    lo = cpumach.bf16_truncate(want32).astype(np.int64)
    g = got16.astype(np.int64)
    exact = (np.ascontiguousarray(want32, np.float32).view(np.uint32) & 0xFFFF) == 0
    ok = (g == lo) | ((g == lo + 1) & ~exact)
    return bool(ok.all())


def test_narrow_gives_a_neighbour_and_is_exact_on_representable_values(oracle):
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(300) * 0.01, rng.standard_normal(100) * 100,
                         [0.0, -0.0, 1.0, -1.0, 0.5, 3.0e-39, -3.0e-39]]).astype(np.float32)
    for t, x in enumerate(xs):
        key = cpumach.bf16_key(7, t, 3)
        h = cpumach.bf16_narrow(x, key, t)
        assert neighbours_ok(np.array([h], np.uint16), np.array([x], np.float32))
    rep = cpumach.bf16_widen(cpumach.bf16_truncate(xs))
    for t, x in enumerate(rep):
        h = cpumach.bf16_narrow(x, cpumach.bf16_key(1, t, 0), 5)
        assert cpumach.bf16_widen(np.array([h], np.uint16))[0] == x or (x == 0 and h in (0, 0x8000))
    # infinities and NaN keep their class
    inf = cpumach.bf16_narrow(np.float32(np.inf), 123, 4)
    assert np.isinf(cpumach.bf16_widen(np.array([inf], np.uint16))[0])
    nan = cpumach.bf16_narrow(np.float32(np.nan), 123, 4)
    assert np.isnan(cpumach.bf16_widen(np.array([nan], np.uint16))[0])


@pytest.mark.parametrize("frac", [0.0, 0.1, 0.5, 0.9, 0.999])
def test_narrow_is_unbiased(oracle, frac):
    # x sits `frac` of the way from one bf16 value to the next: the upper one must be chosen with
    # probability frac, over rows and over keys alike
    base = np.array([0x3C23], np.uint16)  # about 0.00995
    u = (base.astype(np.uint32) << 16) + np.uint32(round(frac * 65536))
    x = u.view(np.float32)[0]
    n = 20000
    up_rows = sum(cpumach.bf16_narrow(x, 0xABCDEF01, r) != int(base[0]) for r in range(n))
    up_keys = sum(cpumach.bf16_narrow(x, cpumach.bf16_key(99, t, 1), 17) != int(base[0])
                  for t in range(n))
    sigma = max(np.sqrt(frac * (1 - frac) / n), 1e-9)
    assert abs(up_rows / n - frac) <= 5 * sigma + 1e-4
    assert abs(up_keys / n - frac) <= 5 * sigma + 1e-4


def test_keys_differ_between_units_slots_and_seeds(oracle):
    keys = {cpumach.bf16_key(s, u, sl) for s in (1, 2) for u in range(50) for sl in
            (0, 1, 2, 0xFFFFFFFF, 0x10000, 0x10001)}
    assert len(keys) == 2 * 50 * 6


@pytest.mark.parametrize("d,V,N,skip", [(100, 500, 4000, 5), (65, 200, 1500, 3), (1, 10, 100, 2)])
def test_eval_equals_fp32_oracle_on_widened_tables(oracle, d, V, N, skip):
    rng = np.random.default_rng(d)
    A, B = tables16(rng, V, d, 0.4 / d ** 0.25)
    W = corpus.zipf_stream(N, V, 1.0, seed=d)
    W[rng.random(N) < 0.05] = -1
    LB, UB = corpus.window_bounds(N, skip, rng)
    A32, B32 = cpumach.bf16_widen(A), cpumach.bf16_widen(B)
    assert oracle.word2vecEvalPosBf16(d, N, skip, W, LB, UB, A, B) == \
        oracle.word2vecEvalPos(d, N, skip, W, LB, UB, A32, B32, 1)
    G, nwa, nwb = N // 10, 5, 4
    WA = rng.integers(0, V, G * nwa).astype(np.int32)
    WB = rng.integers(0, V, G * nwb).astype(np.int32)
    assert oracle.word2vecEvalNegBf16(d, G, nwa, nwb, WA, WB, A, B) == \
        oracle.word2vecEvalNeg(d, G, nwa, nwb, WA, WB, A32, B32, 1)


@pytest.mark.parametrize("hot", [0, 1500])
@pytest.mark.parametrize("vexp", [0.0, 0.5, 0.75])
@pytest.mark.parametrize("d,skip,ncentres", [(100, 5, 60), (33, 3, 40), (1, 2, 20)])
def test_pos_update_is_a_rounding_of_the_fp32_oracle(oracle, vexp, d, skip, ncentres, hot):
    # collision-free: every column is written once, so every stored element must be one of the
    # two bf16 neighbours of what the fp32 oracle computes from the widened tables
    rng = np.random.default_rng(d + skip)
    V = 4000
    A, B = tables16(rng, V, d, 0.5 / d ** 0.25)
    W, LB, UB = corpus.collision_free_pos(ncentres, skip, V, rng)
    W[rng.random(W.shape[0]) < 0.05] = -1
    A32, B32 = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    oracle.word2vecPos(d, W.shape[0], skip, W, LB, UB, A32, B32, 0.025, vexp, 1)
    A16, B16 = A.copy(), B.copy()
    oracle.word2vecPosBf16(d, W.shape[0], skip, W, LB, UB, A16, B16, 0.025, vexp, 11, hot)
    assert neighbours_ok(A16, A32) and neighbours_ok(B16, B32)
    changed = (A16 != A).any(axis=1).sum() + (B16 != B).any(axis=1).sum()
    assert changed > ncentres
    # columns no unit touches keep their bits
    untouched = np.setdiff1d(np.arange(V), W[W >= 0])
    assert (A16[untouched] == A[untouched]).all() and (B16[untouched] == B[untouched]).all()
    # same seed, same bits; another seed, other roundings
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPosBf16(d, W.shape[0], skip, W, LB, UB, A2, B2, 0.025, vexp, 11, hot)
    assert (A2 == A16).all() and (B2 == B16).all()
    if d > 1:
        oracle.word2vecPosBf16(d, W.shape[0], skip, W, LB, UB, A2, B2, 0.025, vexp, 12, hot)
        assert (B2 != B16).any()


@pytest.mark.parametrize("hot", [0, 1500])
@pytest.mark.parametrize("vexp", [0.0, 0.5, 0.75])
@pytest.mark.parametrize("d,nwa,nwb,G", [(100, 5, 5, 60), (33, 7, 8, 30), (1, 1, 1, 20),
                                         (20, 15, 3, 20)])
def test_neg_update_is_a_rounding_of_the_fp32_oracle(oracle, vexp, d, nwa, nwb, G, hot):
    rng = np.random.default_rng(d + nwa)
    V = 4000
    A, B = tables16(rng, V, d, 0.5 / d ** 0.25)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    A32, B32 = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, A32, B32, 0.025, vexp, 1)
    A16, B16 = A.copy(), B.copy()
    oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, A16, B16, 0.025, vexp, 5, hot)
    assert neighbours_ok(A16, A32) and neighbours_ok(B16, B32)
    assert (A16 != A).any() and (B16 != B).any()


@pytest.mark.parametrize("hot", [0, 1500])
def test_neg_skips_pairs_with_a_dropped_word(oracle, hot):
    # ids below zero (the positive stream's mark for a dropped word) skip every pair they take
    # part in: pinned against the fp32 oracle's filtered negative pass, which drops them too
    rng = np.random.default_rng(77)
    d, V, G, nwa, nwb = 40, 4000, 80, 6, 5
    A, B = tables16(rng, V, d, 0.5 / d ** 0.25)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    WA[rng.random(WA.shape[0]) < 0.2] = -1
    WB[rng.random(WB.shape[0]) < 0.2] = -1
    WA[:nwa] = -1                      # a group without A words
    WB[nwb:2 * nwb] = -1               # a group without B words
    A32, B32 = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    oracle.word2vecNegFilt(d, G, V, nwa, nwb, WA, WB, A32, B32, 0.025, 0.5, 1)
    A16, B16 = A.copy(), B.copy()
    oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, A16, B16, 0.025, 0.5, 5, hot)
    assert neighbours_ok(A16, A32) and neighbours_ok(B16, B32)
    assert (A16 != A).any() and (B16 != B).any()
    # columns of words whose every partner was dropped, and unused columns, keep their bits
    same_a = (A32 == cpumach.bf16_widen(A)).all(axis=1)
    same_b = (B32 == cpumach.bf16_widen(B)).all(axis=1)
    assert (A16[same_a] == A[same_a]).all() and (B16[same_b] == B[same_b]).all()
    want = oracle.word2vecEvalNeg(d, G, nwa, nwb, np.where(WA < 0, 0, WA).astype(np.int32),
                                  np.where(WB < 0, 0, WB).astype(np.int32),
                                  cpumach.bf16_widen(A), cpumach.bf16_widen(B), 1)
    got = oracle.word2vecEvalNegBf16(d, G, nwa, nwb, WA, WB, A, B)
    assert got > want                  # fewer (negative) terms than with the ids patched to 0
    # forward sum over the kept pairs only: brute force
    a32, b32 = cpumach.bf16_widen(A).astype(np.float64), cpumach.bf16_widen(B).astype(np.float64)
    tot = 0.0
    for i in range(G):
        for k in range(nwb):
            for j in range(nwa):
                wa, wb = WA[i * nwa + j], WB[i * nwb + k]
                if wa >= 0 and wb >= 0:
                    s = float(a32[wa] @ b32[wb])
                    tot += np.log(max(1.0 - 1.0 / (1.0 + np.exp(-s)), 1e-40))
    assert got == pytest.approx(tot, rel=1e-6)


def test_mean_over_seeds_approaches_the_fp32_result(oracle):
    # the expectation of the stored value is the fp32 value: averaged over many seeds the bf16
    # result comes far closer to the fp32 oracle than one bf16 step
    rng = np.random.default_rng(3)
    d, V, G, nwa, nwb = 16, 400, 10, 3, 2
    A, B = tables16(rng, V, d, 0.3)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    A32, B32 = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, A32, B32, 0.05, 0.0, 1)
    nseed = 400
    accA = np.zeros_like(A32, dtype=np.float64)
    for s in range(nseed):
        A16, B16 = A.copy(), B.copy()
        oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, A16, B16, 0.05, 0.0, 1000 + s)
        accA += cpumach.bf16_widen(A16)
    rows = np.unique(WA)
    step = np.abs(A32[rows]) * 2.0 ** -7  # at least one bf16 step of each value
    err = np.abs(accA[rows] / nseed - A32[rows])
    assert (err <= 5 * step / np.sqrt(nseed) + 1e-12).all()
    assert np.abs(cpumach.bf16_widen(A16)[rows] - A32[rows]).max() > err.max()


def test_side_buffers_follow_the_sequential_fp32_run_on_colliding_minibatches(oracle):
    # with every word routed through the fp32 side buffers nothing is rounded to bf16 inside a
    # call, so even on a Zipf minibatch, where later units read what earlier ones wrote, the
    # result is the sequential fp32 oracle's (on the widened tables) narrowed once: within one
    # bf16 step, plus a few fp32 ulps for the different association of the sums
    rng = np.random.default_rng(21)
    d, V, N, skip, nwa, nwb = 24, 300, 3000, 4, 5, 4
    A, B = tables16(rng, V, d, 0.3)
    W = corpus.zipf_stream(N, V, 1.0, seed=4)
    W[rng.random(N) < 0.05] = -1
    LB, UB = corpus.window_bounds(N, skip, rng)
    G = 400
    WA = rng.integers(0, V, G * nwa).astype(np.int32)
    WB = corpus.zipf_stream(G * nwb, V, 1.0, seed=5)

    def close(got16, want32):
        step = np.abs(want32) * 2.0 ** -7
        slack = np.abs(want32).max() * 2.0 ** -17
        return bool((np.abs(cpumach.bf16_widen(got16) - want32) <= step + slack).all())

    A32, B32 = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    oracle.word2vecPos(d, N, skip, W, LB, UB, A32, B32, 0.025, 0.5, 1)
    A16, B16 = A.copy(), B.copy()
    oracle.word2vecPosBf16(d, N, skip, W, LB, UB, A16, B16, 0.025, 0.5, 8, V)
    assert close(A16, A32) and close(B16, B32)
    assert np.abs(A32 - cpumach.bf16_widen(A)).max() > 0.05      # many updates piled up

    A32, B32 = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, A32, B32, 0.025, 0.5, 1)
    A16, B16 = A.copy(), B.copy()
    oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, A16, B16, 0.025, 0.5, 9, V)
    assert close(A16, A32) and close(B16, B32)
    # words the call never touched keep their bits
    untouched = np.setdiff1d(np.arange(V), np.concatenate([WA, WB]))
    assert (A16[untouched] == A[untouched]).all() and (B16[untouched] == B[untouched]).all()
