"""The ordered form of the update operators (w2v_set_ordered_mode in include/bidmach_w2v.h): the
kernels that walk tokens / groups in the reference's order on a bounded number of workers, taken
by default for launches full of frequent words.  (needs an MI355X)

Forced on, they must pass the same oracle checks as the throughput kernels.  What sets them apart
is checked on minibatches made of a handful of words, where every update collides with the ones
before it: a launch small enough for one worker must then reproduce the oracle's SEQUENTIAL
result (jni/src/BIDMach_CPUMACH.c:26-68, :210-254 at one thread), which no kernel that works
from a snapshot of its columns can.
"""
import numpy as np
import pytest

from bidmach_amd import corpus
from tests import test_gpu_parity as parity

pytestmark = pytest.mark.gpu

gpu = parity.gpu


@pytest.fixture
def ordered():
    from bidmach_amd.cumach import load_library
    lib = load_library()
    assert lib.w2v_get_ordered_mode() == -1
    lib.w2v_set_ordered_mode(1)
    yield lib
    lib.w2v_set_ordered_mode(-1)


@pytest.mark.parametrize("vexp", [0.0, 0.5, 0.75])
@pytest.mark.parametrize("d,skip,ncentres", [(100, 5, 300), (300, 5, 300), (512, 10, 100),
                                             (1, 2, 50), (65, 3, 100), (1280, 5, 40),
                                             (24, 40, 30), (1000, 25, 30)])
def test_pos_update_forced_ordered(gpu, oracle, ordered, vexp, d, skip, ncentres):
    parity.test_pos_update_matches_oracle(gpu, oracle, vexp, d, skip, ncentres)


@pytest.mark.parametrize("vexp", [0.0, 0.5, 0.75])
@pytest.mark.parametrize("d,nwa,nwb,G", [(100, 5, 5, 400), (300, 5, 5, 400), (512, 15, 5, 100),
                                         (1, 1, 1, 50), (65, 7, 8, 100), (1280, 5, 5, 30),
                                         (40, 70, 3, 40), (300, 6, 2, 100), (640, 16, 4, 50),
                                         (700, 6, 5, 50),
                                         # more than 8 B words (the reference's GPU launcher
                                         # runs 5 x 10, DNN127.cu:1434)
                                         (300, 5, 10, 200), (100, 4, 21, 100), (64, 3, 64, 40),
                                         (512, 16, 9, 40)])
def test_neg_update_forced_ordered(gpu, oracle, ordered, vexp, d, nwa, nwb, G):
    # (40, 70, 3) and (700, 6, 5) have no row-by-row instance: the group-at-a-time kernel on a
    # few workgroups stands in
    parity.test_neg_update_matches_oracle(gpu, oracle, vexp, d, nwa, nwb, G)


def test_other_checks_forced_ordered(gpu, oracle, ordered):
    parity.test_pos_update_ragged_windows_and_tile_edges(gpu, oracle)
    parity.test_neg_filt_matches_oracle(gpu, oracle, 100, 10, 5)
    parity.test_neg_filt_matches_oracle(gpu, oracle, 300, 5, 5)
    parity.test_heavy_collisions_lose_no_contribution(gpu)
    parity.test_noop_invariants_on_gpu(gpu)
    for shift in (0, 2, 100):
        parity.test_pos_update_any_shift_argument(gpu, oracle, shift)


def tiny_colliding(rng, d, V, n, skip):
    A = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    W = rng.integers(0, V, n).astype(np.int32)
    W[rng.random(n) < 0.1] = -1
    LB, UB = corpus.window_bounds(n, skip, rng)
    return A, B, W, LB, UB


@pytest.mark.parametrize("d,skip", [(100, 5), (300, 3), (64, 12)])
def test_one_worker_reproduces_the_sequential_positive_pass(gpu, oracle, d, skip):
    """60 tokens over 6 words: every pair updates columns the pairs before it updated.  The
    launch holds only frequent words (ids below 16), so the default takes the ordered form, and
    60 tokens are one worker's range: the result is the oracle's one-thread result up to the
    rounding of the dot products.  The throughput kernel (ordered form off) works from one
    snapshot per tile and lands visibly elsewhere."""
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(d)
    A, B, W, LB, UB = tiny_colliding(rng, d, 6, 60, skip)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecPos(d, 60, skip, W, LB, UB, Ao, Bo, 0.05, 0.5, 1)
    Ag, Bg = parity.gpu_pos(gpu, d, skip, W, LB, UB, A, B, 0.05, 0.5)
    err = max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max())
    assert err <= 2e-5, err
    lib.w2v_set_ordered_mode(0)
    try:
        At, Bt = parity.gpu_pos(gpu, d, skip, W, LB, UB, A, B, 0.05, 0.5)
    finally:
        lib.w2v_set_ordered_mode(-1)
    assert max(np.abs(At - Ao).max(), np.abs(Bt - Bo).max()) > 50 * err + 1e-3


def comes_back_stream(rng, n, skip, fixed):
    """Distinct words, except that word 3 stands at every (2 skip + 1)-th position: it leaves
    a token's window at one end just as the next token's window reaches its next occurrence at
    the other end, which inside a team of wavefronts is another wave's position."""
    W = (16 + rng.permutation(n)).astype(np.int32)
    W[7::2 * skip + 1] = 3
    if fixed:
        LB = np.full(n, -skip, np.int32)
        UB = np.full(n, skip, np.int32)
    else:
        LB, UB = corpus.window_bounds(n, skip, rng)
    return W, LB, UB


@pytest.mark.parametrize("fixed", [True, False])
@pytest.mark.parametrize("d,skip", [(100, 5), (300, 5), (64, 3)])
def test_one_team_hands_a_column_from_wave_to_wave_in_order(gpu, oracle, d, skip, fixed):
    """One worker (a team of four wavefronts) on a stream whose only repeated word comes back one
    position beyond the window each time: the wave that reads its column for the next token is
    not the wave that has just added to it, and must still see that add (the sequential oracle's
    result, up to the rounding of the dot products; a missed add is 1e-3 and more)."""
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(d + skip)
    n = 600
    V = n + 16
    A = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    W, LB, UB = comes_back_stream(rng, n, skip, fixed)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecPos(d, n, skip, W, LB, UB, Ao, Bo, 0.05, 0.0, 1)
    lib.w2v_set_ordered_mode(1)
    lib.w2v_set_ordered_workers(1, 1)
    try:
        Ag, Bg = parity.gpu_pos(gpu, d, skip, W, LB, UB, A, B, 0.05, 0.0)
    finally:
        lib.w2v_set_ordered_mode(-1)
        lib.w2v_set_ordered_workers(0, 0)
    err = max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max())
    assert np.abs(Bo[3] - B[3]).max() > 0.05     # the word's column did move, many times
    assert err <= 2e-5, err


@pytest.mark.parametrize("d,nwa,nwb", [(100, 5, 5), (300, 5, 5), (200, 12, 3), (300, 5, 10),
                                       (100, 3, 14)])
def test_one_worker_reproduces_the_sequential_negative_pass(gpu, oracle, d, nwa, nwb):
    """16 groups over 8 words (distinct inside a group's B words and inside its A words, as the
    group-level order of the reference matters only there): B columns change from row to row and
    from group to group, A columns from group to group."""
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(d + nwa)
    V, G = 14, 16
    A = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    WA = np.concatenate([rng.permutation(V)[:nwa] for _ in range(G)]).astype(np.int32)
    WB = np.concatenate([rng.permutation(V)[:nwb] for _ in range(G)]).astype(np.int32)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.05, 0.5, 1)
    Ag, Bg = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.05, 0.5)
    err = max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max())
    assert err <= 2e-5, err
    lib.w2v_set_ordered_mode(0)
    try:
        At, Bt = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.05, 0.5)
    finally:
        lib.w2v_set_ordered_mode(-1)
    if nwb <= 8:   # (the kernel for wider groups walks 16 groups on one wave, in order as well)
        assert max(np.abs(At - Ao).max(), np.abs(Bt - Bo).max()) > 50 * err + 1e-3


def test_a_word_twice_among_a_groups_b_words_sees_its_first_update(gpu, oracle):
    """The reference writes a B column back before it turns to the next B word (:244-246), so a
    word that is a group's B word twice is dotted the second time with its first delta in it."""
    rng = np.random.default_rng(11)
    d, V, G, nwa, nwb = 100, 14, 8, 5, 5
    A = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    WA = np.concatenate([rng.permutation(V)[:nwa] for _ in range(G)]).astype(np.int32)
    WB = np.concatenate([rng.permutation(V)[:nwb] for _ in range(G)]).astype(np.int32)
    WB[1::nwb] = WB[0::nwb]          # rows 0 and 1 of every group are the same word
    WB[4::nwb] = WB[2::nwb]          # and rows 2 and 4
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.05, 0.0, 1)
    Ag, Bg = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.05, 0.0)
    assert max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max()) <= 2e-5


def test_the_decision_does_not_depend_on_how_the_vocabulary_is_numbered(gpu, oracle):
    """The decision is made on the device from how often the words of the launch occur, not from
    their ids: the same heavy collisions on ids 100..105 (no id below 16) take the ordered form
    by default and reproduce the sequential result."""
    rng = np.random.default_rng(5)
    d, skip = 100, 5
    A, B, W, LB, UB = tiny_colliding(rng, d, 6, 60, skip)
    big = np.zeros((200, d), np.float32)
    A2, B2 = big.copy(), big.copy()
    A2[100:106], B2[100:106] = A, B
    W2 = np.where(W >= 0, W + 100, -1).astype(np.int32)
    Ao, Bo = A2.copy(), B2.copy()
    oracle.word2vecPos(d, 60, skip, W2, LB, UB, Ao, Bo, 0.05, 0.0, 1)
    Ag, Bg = parity.gpu_pos(gpu, d, skip, W2, LB, UB, A2, B2, 0.05, 0.0)
    assert max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max()) <= 2e-5
    G, nwa, nwb = 16, 3, 3
    WA = np.concatenate([100 + rng.permutation(6)[:nwa] for _ in range(G)]).astype(np.int32)
    WB = np.concatenate([100 + rng.permutation(6)[:nwb] for _ in range(G)]).astype(np.int32)
    Ao, Bo = A2.copy(), B2.copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.05, 0.0, 1)
    Ag, Bg = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A2, B2, 0.05, 0.0)
    assert max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max()) <= 2e-5


def test_launches_without_frequent_words_keep_the_throughput_kernels(gpu, oracle):
    """2000 tokens, every word once: no word is frequent, so the default is the tiled kernel,
    whose tiles of 16 adjacent tokens work from one snapshot of their columns: at a large step its
    result is visibly not the sequential one (adjacent windows share their context positions),
    while the ordered form, forced onto one worker, is."""
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(6)
    d, skip, n = 100, 5, 2000
    A = (rng.standard_normal((n, d)) * 0.3).astype(np.float32)
    B = (rng.standard_normal((n, d)) * 0.3).astype(np.float32)
    W = rng.permutation(n).astype(np.int32)
    LB, UB = corpus.window_bounds(n, skip, rng)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecPos(d, n, skip, W, LB, UB, Ao, Bo, 0.3, 0.0, 1)
    Ag, Bg = parity.gpu_pos(gpu, d, skip, W, LB, UB, A, B, 0.3, 0.0)
    assert max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max()) > 1e-3
    lib.w2v_set_ordered_mode(1)
    lib.w2v_set_ordered_workers(1, 1)       # one worker: the sequential order itself
    try:
        Ag, Bg = parity.gpu_pos(gpu, d, skip, W, LB, UB, A, B, 0.3, 0.0)
    finally:
        lib.w2v_set_ordered_mode(-1)
        lib.w2v_set_ordered_workers(0, 0)
    assert max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max()) <= 2e-5


def test_a_b_word_of_two_tiles_of_a_wide_group_sees_its_first_update(gpu, oracle):
    """Groups with more than 8 B words pass their B columns through registers in tiles of 8; a
    word that is a B word in two tiles is read for the second one as the first one's adds left it
    (BIDMach_CPUMACH.c:219-246 walks the rows one after the other).  The ids are spread over a
    large vocabulary so that no word of the launch is frequent and the throughput kernel runs."""
    rng = np.random.default_rng(12)
    d, V, G, nwa, nwb = 100, 40000, 300, 4, 10
    A = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    ids = rng.permutation(V)[:G * (nwa + nwb)].astype(np.int32)
    WA = ids[:G * nwa].copy()
    WB = ids[G * nwa:].copy()
    WB[8::nwb] = WB[0::nwb]          # row 8 (second tile) repeats row 0 (first tile)
    WB[9::nwb] = WB[5::nwb]          # and row 9 repeats row 5
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.05, 0.0, 1)
    Ag, Bg = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.05, 0.0)
    assert max(np.abs(Ag - Ao).max(), np.abs(Bg - Bo).max()) <= 2e-5


def test_ordered_launch_of_a_shape_without_a_row_by_row_instance(gpu, oracle):
    """17 A words per group fit no instance of the row-by-row kernel: an ordered launch then runs
    the group-at-a-time kernels on a few workgroups, for the single-table, the wide and the sliced
    operator alike.  On colliding words that order is not the sequential one, so the check is the
    collision-free parity with the ordered form forced."""
    from bidmach_amd.cumach import load_library
    lib = load_library()
    lib.w2v_set_ordered_mode(1)
    try:
        parity.test_neg_update_matches_oracle(gpu, oracle, 0.5, 200, 17, 5, 60)
        parity.test_neg_update_matches_oracle(gpu, oracle, 0.5, 200, 17, 12, 60)
        islice, nslices, nhead, maxcols, dohead, dual = sliced_slicings()[1]
        sliced_mod().test_neg_slice_matches_oracle(gpu, oracle, islice, nslices, nhead, maxcols,
                                                   dohead, dual, 200, 17, 5, 0.5)
        sliced_mod().test_neg_slice_matches_oracle(gpu, oracle, islice, nslices, nhead, maxcols,
                                                   dohead, dual, 200, 17, 12, 0.5)
    finally:
        lib.w2v_set_ordered_mode(-1)


def sliced_mod():
    from tests import test_gpu_slice
    return test_gpu_slice


def sliced_slicings():
    return sliced_mod().SLICINGS


# ---- sliced, multi-part models (word2vecPosSlice / word2vecNegSlice) ---------------------------

from tests import test_gpu_slice as sliced   # noqa: E402


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead,dual", sliced.SLICINGS)
def test_slice_updates_forced_ordered(gpu, oracle, ordered, islice, nslices, nhead, maxcols, dohead,
                                      dual):
    g = gpu   # (torch, CUMACH), as the sliced tests' own fixture
    for d, vexp in ((100, 0.0), (300, 0.5)):
        sliced.test_pos_slice_matches_oracle(g, oracle, islice, nslices, nhead, maxcols, dohead,
                                             dual, d, vexp)
    sliced.test_pos_slice_matches_oracle(g, oracle, islice, nslices, nhead, maxcols, dohead, dual,
                                         1000, 0.5, skip=25)   # a shape that fits no tile
    for d, nwa, nwb, vexp in ((100, 5, 5, 0.0), (300, 15, 5, 0.5), (130, 3, 8, 0.5)):
        sliced.test_neg_slice_matches_oracle(g, oracle, islice, nslices, nhead, maxcols, dohead,
                                             dual, d, nwa, nwb, vexp)


SMALL_SLICINGS = [  # islice, nslices, nhead, maxcols, dohead: 14 words, all of them "frequent"
    (0, 1, 0, 1 << 20, 0),
    (1, 2, 4, 5, 0),       # head read-only, three parts
    (0, 2, 4, 5, 1),       # head written
    (1, 3, 6, 4, 2),       # head-head pairs trained too
]


@pytest.mark.parametrize("islice,nslices,nhead,maxcols,dohead", SMALL_SLICINGS)
def test_one_worker_reproduces_the_sequential_sliced_passes(gpu, oracle, islice, nslices, nhead,
                                                            maxcols, dohead):
    """The sliced operators on minibatches where every update collides with the ones before it
    (14 words, all with ids below 16, so the default takes the ordered form; one worker's range):
    the result is the oracle's one-thread result (BIDMach_CPUMACH.c:80-184, :267-366), with the
    rules for which pairs are trained and which columns written; with the ordered form switched
    off the throughput kernels land visibly elsewhere."""
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(100 * nslices + dohead)
    d, V, n, skip, G, nwa, nwb = 100, 14, 60, 4, 16, 5, 5
    A = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.3).astype(np.float32)
    W = rng.integers(0, V, n).astype(np.int32)
    W[rng.random(n) < 0.1] = -1
    LB, UB = corpus.window_bounds(n, skip, rng)
    WA = np.concatenate([rng.permutation(V)[:nwa] for _ in range(G)]).astype(np.int32)
    WB = np.concatenate([rng.permutation(V)[:nwb] for _ in range(G)]).astype(np.int32)

    def run(mode):
        host, devl = sliced.model_lists(torch, A, B, islice, nslices, nhead, maxcols, False)
        lib.w2v_set_ordered_mode(mode)
        try:
            assert CUMACH.word2vecPosSlice(d, n, skip, sliced.dev(torch, W), sliced.dev(torch, LB),
                                           sliced.dev(torch, UB), devl, 0.05, 0.5, islice, nslices,
                                           maxcols, nhead, False, dohead) == 0
            assert CUMACH.word2vecNegSlice(d, G, nwa, nwb, sliced.dev(torch, WA),
                                           sliced.dev(torch, WB), devl, 0.05, 0.5, islice, nslices,
                                           maxcols, nhead, False, dohead) == 0
        finally:
            lib.w2v_set_ordered_mode(-1)
        return host, [m.cpu().numpy() for m in devl]

    host, got = run(-1)
    before = [h.copy() for h in host]
    oracle.word2vecPosSlice(d, n, skip, W, LB, UB, host, 0.05, 0.5, 1, islice, nslices, maxcols,
                            nhead, False, dohead)
    oracle.word2vecNegSlice(d, G, nwa, nwb, WA, WB, host, 0.05, 0.5, 1, islice, nslices, maxcols,
                            nhead, False, dohead)
    assert max(np.abs(h - b).max() for h, b in zip(host, before)) > 1e-2
    err = max(np.abs(g - h).max() for g, h in zip(got, host))
    assert err <= 2e-5, err
    _, loose = run(0)
    assert max(np.abs(g - h).max() for g, h in zip(loose, host)) > 50 * err + 1e-3


def test_last_launch_form_reports_what_the_device_decided(gpu, oracle):
    """w2v_last_launch_form reads back the counts that the kernels of the thread's last update
    call looked at: a launch over a handful of words took the ordered form, a launch of distinct
    words the throughput kernels, and forcing either way is reported as forced."""
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(5)
    d, skip, n = 64, 3, 4000
    LB, UB = corpus.window_bounds(n, skip, rng)
    A = (rng.standard_normal((n + 16, d)) * 0.1).astype(np.float32)
    B = (rng.standard_normal((n + 16, d)) * 0.1).astype(np.float32)
    few = rng.integers(0, 6, n).astype(np.int32)
    distinct = (16 + rng.permutation(n)).astype(np.int32)
    parity.gpu_pos(gpu, d, skip, few, LB, UB, A, B, 0.01, 0.0)
    assert lib.w2v_last_launch_form() == 1
    parity.gpu_pos(gpu, d, skip, distinct, LB, UB, A, B, 0.01, 0.0)
    assert lib.w2v_last_launch_form() == 0
    G = n // 5
    parity.gpu_neg(gpu, d, G, 5, 5, few[:5 * G], distinct[:5 * G], A, B, 0.01, 0.0)
    assert lib.w2v_last_launch_form() == 1          # the A words are the frequent ones here
    parity.gpu_neg(gpu, d, G, 5, 5, distinct[:5 * G], distinct[::-1][:5 * G].copy(), A, B, 0.01, 0.0)
    assert lib.w2v_last_launch_form() == 0
    lib.w2v_set_ordered_mode(1)
    try:
        parity.gpu_pos(gpu, d, skip, distinct, LB, UB, A, B, 0.01, 0.0)
        assert lib.w2v_last_launch_form() == 1
    finally:
        lib.w2v_set_ordered_mode(-1)
    lib.w2v_set_ordered_mode(0)
    try:
        parity.gpu_pos(gpu, d, skip, few, LB, UB, A, B, 0.01, 0.0)
        assert lib.w2v_last_launch_form() == 0
    finally:
        lib.w2v_set_ordered_mode(-1)

