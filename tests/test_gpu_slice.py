"""Parity of the sliced, multi-part HIP operators with the CPU oracle, through the C ABI (needs an
MI355X).  Same tolerances as the single-table operators: forward sums within 1e-5 relative,
updates within 1e-4 absolute per element on collision-free minibatches.  Every part of the model
is a separate device allocation, as in the reference's list of model matrices.
"""
import math

import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

EVAL_RTOL = 1e-5
UPDATE_ATOL = 1e-4

SLICINGS = [  # islice, nslices, nhead, maxcols, dohead, dual
    (0, 1, 0, 1 << 20, 0, False),      # one worker, one part: the plain operators
    (0, 3, 40, 1 << 20, 0, False),
    (2, 3, 40, 1 << 20, 1, False),
    (1, 3, 40, 397, 2, False),         # several parts
    (3, 4, 0, 164, 1, True),           # no head, dual-mode list
    (0, 2, 500, 333, 2, True),
]


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    from bidmach_amd.cumach import CUMACH, load_library
    load_library()
    return torch, CUMACH


def dev(torch, x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def rand_tables(rng, vocab, d, scale=0.3):
    A = (rng.standard_normal((vocab, d)) * scale).astype(np.float32)
    B = (rng.standard_normal((vocab, d)) * scale).astype(np.float32)
    return A, B


def model_lists(torch, A, B, islice, nslices, nhead, maxcols, dual):
    """(host list for the oracle, device list for the library) of one worker's model matrices."""
    ap = cf.pack_parts(A, islice, nslices, nhead, maxcols)
    bp = cf.pack_parts(B, islice, nslices, nhead, maxcols)
    host = []
    if dual:
        host += [np.full_like(bp[0], 3.0), np.full_like(ap[0], 3.0)]
    for b, a in zip(bp, ap):
        host += [b, a]
    return host, [dev(torch, m) for m in host]


def assert_lists_close(devlist, hostlist, atol):
    worst = 0.0
    for k, (g, h) in enumerate(zip(devlist, hostlist)):
        worst = max(worst, float(np.abs(g.cpu().numpy() - h).max()))
    assert worst < atol, worst
    return worst


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead,dual", SLICINGS)
@pytest.mark.parametrize("d,vexp", [(100, 0.0), (300, 0.5), (65, 1.0)])
def test_pos_slice_matches_oracle(gpu, oracle, islice, nslices, nhead, maxcols, dohead, dual, d,
                                  vexp, skip=3):
    torch, CUMACH = gpu
    rng = np.random.default_rng(7 * d + islice)
    V = 2200
    A, B = rand_tables(rng, V, d, 0.5 / math.sqrt(d) ** 0.5)
    W, LB, UB = corpus.collision_free_pos(300 if skip <= 3 else 30, skip, V, rng)
    W[rng.random(len(W)) < 0.03] = -1
    host, devl = model_lists(torch, A, B, islice, nslices, nhead, maxcols, dual)
    before = [h.copy() for h in host]
    lr = 0.05 / (1 + V) ** vexp
    oracle.word2vecPosSlice(d, len(W), skip, W, LB, UB, host, lr, vexp, 1, islice, nslices,
                            maxcols, nhead, dual, dohead)
    err = CUMACH.word2vecPosSlice(d, len(W), skip, dev(torch, W), dev(torch, LB), dev(torch, UB),
                                  devl, lr, vexp, islice, nslices, maxcols, nhead, dual, dohead)
    assert err == 0
    assert max(np.abs(h - b).max() for h, b in zip(host, before)) > 1e-4   # something trained
    assert_lists_close(devl, host, UPDATE_ATOL)
    # columns the oracle left alone are bit-identical on the device too
    for g, h, b in zip(devl, host, before):
        same = np.all(h == b, axis=1)
        assert np.array_equal(g.cpu().numpy()[same], b[same])


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead,dual", SLICINGS)
@pytest.mark.parametrize("d,nwa,nwb,vexp", [(100, 5, 5, 0.0), (300, 15, 5, 0.5), (130, 3, 8, 0.5),
                                            (64, 70, 2, 0.0),
                                            # more B words than a wave holds at once
                                            (300, 5, 10, 0.5), (100, 4, 21, 0.0)])
def test_neg_slice_matches_oracle(gpu, oracle, islice, nslices, nhead, maxcols, dohead, dual, d,
                                  nwa, nwb, vexp):
    torch, CUMACH = gpu
    rng = np.random.default_rng(11 * d + islice)
    G = 120
    V = G * (nwa + nwb) + 600
    A, B = rand_tables(rng, V, d, 0.5 / math.sqrt(d) ** 0.5)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    host, devl = model_lists(torch, A, B, islice, nslices, nhead, maxcols, dual)
    before = [h.copy() for h in host]
    lr = 0.05 / (1 + V) ** vexp
    oracle.word2vecNegSlice(d, G, nwa, nwb, WA, WB, host, lr, vexp, 1, islice, nslices, maxcols,
                            nhead, dual, dohead)
    err = CUMACH.word2vecNegSlice(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB), devl, lr, vexp,
                                  islice, nslices, maxcols, nhead, dual, dohead)
    assert err == 0
    assert max(np.abs(h - b).max() for h, b in zip(host, before)) > 1e-5
    assert_lists_close(devl, host, UPDATE_ATOL)
    for g, h, b in zip(devl, host, before):
        same = np.all(h == b, axis=1)
        assert np.array_equal(g.cpu().numpy()[same], b[same])


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead,dual", SLICINGS)
@pytest.mark.parametrize("d", [100, 300])
def test_eval_slice_matches_oracle(gpu, oracle, islice, nslices, nhead, maxcols, dohead, dual, d):
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(13 * d + islice)
    V, N, skip, nwa, G = 3000, 20000, 5, 5, 4000
    nwb = 5 if d == 100 else 10
    A, B = rand_tables(rng, V, d, 0.6 / math.sqrt(d) ** 0.5)
    W = corpus.zipf_stream(N, V, 1.0, seed=d + islice)
    W[rng.random(N) < 0.05] = -1
    LB, UB = corpus.window_bounds(N, skip, rng, sentence=np.cumsum(rng.random(N) < 0.03))
    WA = rng.integers(0, V, G * nwa).astype(np.int32)
    WB = corpus.zipf_stream(G * nwb, V, 1.0, seed=d)
    host, devl = model_lists(torch, A, B, islice, nslices, nhead, maxcols, dual)
    floor = 1.0e-20                                   # the Scala twins' floor
    old = lib.w2v_get_eval_floor()
    lib.w2v_set_eval_floor(floor)
    try:
        ret = torch.zeros(2, dtype=torch.float64, device="cuda")
        err = CUMACH.word2vecEvalPosSlice(d, N, skip, dev(torch, W), dev(torch, LB), dev(torch, UB),
                                          devl, islice, nslices, maxcols, nhead, dual, ret[0:1])
        assert err == 0
        err = CUMACH.word2vecEvalNegSlice(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB), devl,
                                          islice, nslices, maxcols, nhead, dual, ret[1:2])
        assert err == 0
    finally:
        lib.w2v_set_eval_floor(old)
    wpos = oracle.word2vecEvalPosSlice(d, N, skip, W, LB, UB, host, 4, islice, nslices, maxcols,
                                       nhead, dual, floor=floor)
    wneg = oracle.word2vecEvalNegSlice(d, G, nwa, nwb, WA, WB, host, 4, islice, nslices, maxcols,
                                       nhead, dual, floor=floor)
    got = ret.cpu().numpy()
    assert wpos < -10.0 and wneg < -10.0
    assert got[0] == pytest.approx(wpos, rel=EVAL_RTOL)
    assert got[1] == pytest.approx(wneg, rel=EVAL_RTOL)


@pytest.mark.parametrize("shift", [0, 1, 40])
def test_pos_slice_result_does_not_depend_on_shift(gpu, oracle, shift):
    """`shift` only sizes the halo staged on chip: 0 takes the per-centre kernel, 1 leaves most of
    the window to the gather path of the tiled kernel, 40 is clamped."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(17)
    V, d, skip = 2600, 100, 4
    islice, nslices, nhead, maxcols, dohead = 1, 2, 200, 500, 1
    A, B = rand_tables(rng, V, d, 0.15)
    W, LB, UB = corpus.collision_free_pos(280, skip, V, rng)
    host, devl = model_lists(torch, A, B, islice, nslices, nhead, maxcols, False)
    oracle.word2vecPosSlice(d, len(W), skip, W, LB, UB, host, 0.05, 0.0, 1, islice, nslices,
                            maxcols, nhead, 0, dohead)
    err = CUMACH.word2vecPosSlice(d, len(W), shift, dev(torch, W), dev(torch, LB), dev(torch, UB),
                                  devl, 0.05, 0.0, islice, nslices, maxcols, nhead, 0, dohead)
    assert err == 0
    assert_lists_close(devl, host, UPDATE_ATOL)


def test_colliding_minibatch_stays_close_to_sequential_oracle(gpu, oracle):
    """A Zipf minibatch on a three-part, two-worker model with a small step: the Hogwild result
    differs from the single-thread oracle only in second order."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(5)
    V, d, N, skip, nwa, nwb = 3000, 128, 30000, 5, 5, 5
    islice, nslices, nhead, maxcols, dohead = 1, 2, 300, 700, 1
    A, B = rand_tables(rng, V, d, 0.05)
    W = corpus.zipf_stream(N, V, 1.0, seed=9)
    LB, UB = corpus.window_bounds(N, skip, rng)
    WA, WB, G = corpus.negative_groups(W, LB, UB, nwa, nwb, rng, vocab=V)
    host, devl = model_lists(torch, A, B, islice, nslices, nhead, maxcols, False)
    before = [h.copy() for h in host]
    lr = 3e-5
    oracle.word2vecPosSlice(d, N, skip, W, LB, UB, host, lr, 0.0, 1, islice, nslices, maxcols,
                            nhead, 0, dohead)
    oracle.word2vecNegSlice(d, G, nwa, nwb, WA, WB, host, lr / nwa, 0.0, 1, islice, nslices,
                            maxcols, nhead, 0, dohead)
    assert CUMACH.word2vecPosSlice(d, N, skip, dev(torch, W), dev(torch, LB), dev(torch, UB), devl,
                                   lr, 0.0, islice, nslices, maxcols, nhead, 0, dohead) == 0
    assert CUMACH.word2vecNegSlice(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB), devl, lr / nwa,
                                   0.0, islice, nslices, maxcols, nhead, 0, dohead) == 0
    moved = max(np.abs(h - b).max() for h, b in zip(host, before))
    worst = max(float(np.abs(g.cpu().numpy() - h).max()) for g, h in zip(devl, host))
    print("\nlargest update %.3e, largest GPU-oracle distance %.3e" % (moved, worst))
    assert moved > 1e-5 and worst < 0.05 * moved


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead,dual", SLICINGS[1:4])
def test_pos_slice_shape_that_fits_no_tile(gpu, oracle, islice, nslices, nhead, maxcols, dohead,
                                           dual):
    """dim 1000 with a window of +-25: not even 8 tokens and their halo fit in a CU's LDS, so the
    wave-per-centre kernel runs."""
    test_pos_slice_matches_oracle(gpu, oracle, islice, nslices, nhead, maxcols, dohead, dual, 1000,
                                  0.5, skip=25)


def test_bad_slice_arguments_are_rejected(gpu):
    torch, CUMACH = gpu
    d, n = 32, 64
    W = torch.zeros(n, dtype=torch.int32, device="cuda")
    t = [torch.zeros(10, d, device="cuda") for _ in range(4)]
    ret = torch.zeros(1, dtype=torch.float64, device="cuda")

    def pos(mm, islice=0, nslices=1, maxcols=10, nhead=0, dual=0, dohead=0):
        return CUMACH.word2vecPosSlice(d, n, 2, W, W, W, mm, 0.1, 0.0, islice, nslices, maxcols,
                                       nhead, dual, dohead)

    assert pos(t) == 0
    assert pos(t[:3]) != 0                       # odd number of matrices
    assert pos(t[:2], dual=1) != 0               # dual mode needs a second pair
    assert pos(t, islice=2, nslices=2) != 0
    assert pos(t, nslices=0) != 0
    assert pos(t, maxcols=0) != 0
    assert pos([t[0], None]) != 0
    from bidmach_amd.cumach import load_library
    too_many = 2 * (load_library().w2v_max_slice_parts() + 1)
    assert pos([t[0]] * too_many) != 0
    assert CUMACH.word2vecEvalPosSlice(d, n, 2, W, W, W, t, 0, 1, 10, 0, 0, None) != 0
    assert CUMACH.word2vecEvalPosSlice(d, n, 2, W, W, W, t, 0, 1, 10, 0, 0, ret) == 0
    assert CUMACH.word2vecNegSlice(d, 4, 2, 65, W, W, t, 0.1, 0.0, 0, 1, 10, 0, 0, 0) != 0  # nwb > 64
