"""The ordered form of the bfloat16 update operators (w2v_set_ordered_mode in
include/bidmach_w2v.h), taken by default for launches full of frequent words: a bounded number
of workers, each walking its tokens / groups in the reference's order with device-scope reads.
(needs an MI355X)

Forced on, it must pass the oracle checks of the throughput kernels (same roundings: every write
uses the same random bits whichever kernel makes it).  On minibatches made of a handful of words,
where every update collides with the ones before it, one worker must land on the bfloat16
oracle's SEQUENTIAL result (loop nests of jni/src/BIDMach_CPUMACH.c:26-68, :210-254 at one
thread) up to the occasional rounding that falls the other way.
"""
import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import cpumach
from tests import test_gpu_bf16 as b16

pytestmark = pytest.mark.gpu

gpu = b16.gpu


@pytest.fixture
def ordered():
    from bidmach_amd.cumach import load_library
    lib = load_library()
    assert lib.w2v_get_ordered_mode() == -1
    lib.w2v_set_ordered_mode(1)
    yield lib
    lib.w2v_set_ordered_mode(-1)


@pytest.fixture(params=[0, 1024])
def hot(request):
    from bidmach_amd.cumach import load_library
    lib = load_library()
    old = lib.w2v_get_bf16_hot_words()
    assert lib.w2v_set_bf16_hot_words(request.param) == 0
    yield request.param
    lib.w2v_set_bf16_hot_words(old)


@pytest.mark.parametrize("vexp", [0.0, 0.5])
@pytest.mark.parametrize("d,skip,ncentres", [(100, 5, 300), (300, 5, 300), (512, 10, 100),
                                             (1, 2, 50), (65, 3, 100), (1280, 5, 40),
                                             (24, 40, 30)])
def test_pos_update_bf16_forced_ordered(gpu, oracle, ordered, hot, vexp, d, skip, ncentres):
    b16.test_pos_update_bf16(gpu, oracle, hot, vexp, d, skip, ncentres)


@pytest.mark.parametrize("vexp", [0.0, 0.5])
@pytest.mark.parametrize("d,nwa,nwb,G", [(100, 5, 5, 400), (300, 5, 5, 400), (512, 15, 5, 100),
                                         (1, 1, 1, 50), (65, 7, 8, 100), (1280, 5, 5, 30),
                                         (40, 70, 3, 40), (640, 6, 2, 100), (130, 4, 6, 100)])
def test_neg_update_bf16_forced_ordered(gpu, oracle, ordered, hot, vexp, d, nwa, nwb, G):
    # (40, 70, 3) and (640, 6, 2) have no row-by-row instance: the group-at-a-time kernel on a
    # few waves stands in
    b16.test_neg_update_bf16(gpu, oracle, hot, vexp, d, nwa, nwb, G)


def test_other_checks_bf16_forced_ordered(gpu, oracle, ordered, hot):
    b16.test_neg_bf16_skips_pairs_with_a_dropped_word(gpu, oracle, hot)
    b16.test_unaligned_tables_take_the_halfword_path(gpu, oracle, hot)


def steps_apart(got, want):
    """Largest distance between two bf16 arrays in units of the bf16 step at the larger value."""
    g, w = cpumach.bf16_widen(got), cpumach.bf16_widen(want)
    step = np.maximum(np.abs(g), np.abs(w)) * 2.0 ** -7 + 1e-30
    return float((np.abs(g - w) / step).max())


@pytest.mark.parametrize("d,skip", [(100, 5), (300, 3), (64, 12)])
def test_one_worker_lands_on_the_sequential_positive_pass(gpu, oracle, hot, d, skip):
    """60 tokens over 6 words, all with ids below 16, so the default takes the ordered form; 60
    tokens are one worker's range.  With the words' updates going through fp32 side buffers
    (hot = 1024) the only roundings are those of the final narrowing; without (hot = 0) every
    write rounds, with the oracle's bits, and a rounding that falls the other way (the dot is
    summed in another order) moves what follows by a fraction of a step."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(d)
    V, n = 6, 60
    A, B = b16.tables16(rng, V, d, 0.3)
    W = rng.integers(0, V, n).astype(np.int32)
    W[rng.random(n) < 0.1] = -1
    LB, UB = corpus.window_bounds(n, skip, rng)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecPosBf16(d, n, skip, W, LB, UB, Ao, Bo, 0.05, 0.5, 77, hot)
    Ad, Bd = b16.dev16(torch, A), b16.dev16(torch, B)
    assert CUMACH.word2vecPosBf16(d, n, skip, b16.dev(torch, W), b16.dev(torch, LB),
                                  b16.dev(torch, UB), Ad, Bd, 0.05, 0.5, 77) == 0
    apart = max(steps_apart(b16.host16(Ad), Ao), steps_apart(b16.host16(Bd), Bo))
    moved = max(steps_apart(Ao, A), steps_apart(Bo, B))
    print("\npositive pass, d %d, %d frequent words: %.2f bf16 steps from the sequential oracle "
          "(the pass moved the tables by %.0f steps)" % (d, hot, apart, moved))
    assert moved > 20.0
    assert apart <= (1.01 if hot else 3.0), apart


@pytest.mark.parametrize("fixed", [True, False])
@pytest.mark.parametrize("d,skip", [(100, 5), (300, 5)])
def test_one_team_hands_a_column_from_wave_to_wave_in_order_bf16(gpu, oracle, ordered, hot, d,
                                                                 skip, fixed):
    """One worker on a stream whose only repeated word comes back one position beyond the window
    each time (tests/test_gpu_ordered.py, comes_back_stream): inside a team of wavefronts the
    wave that reads the word's column for the next token is not the wave that has just written
    it, and must still see that write."""
    torch, CUMACH = gpu
    from tests.test_gpu_ordered import comes_back_stream
    rng = np.random.default_rng(d + skip)
    n = 600
    V = n + 16
    A, B = b16.tables16(rng, V, d, 0.3)
    W, LB, UB = comes_back_stream(rng, n, skip, fixed)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecPosBf16(d, n, skip, W, LB, UB, Ao, Bo, 0.05, 0.0, 78, hot)
    Ad, Bd = b16.dev16(torch, A), b16.dev16(torch, B)
    ordered.w2v_set_ordered_workers(1, 1)
    try:
        assert CUMACH.word2vecPosBf16(d, n, skip, b16.dev(torch, W), b16.dev(torch, LB),
                                      b16.dev(torch, UB), Ad, Bd, 0.05, 0.0, 78) == 0
    finally:
        ordered.w2v_set_ordered_workers(0, 0)
    # In steps of the larger of the values before and after (an element that the pass takes
    # through zero keeps the rounding of the size it had).  With the side buffers the only
    # roundings are those of the final narrowing.  Without them every write rounds, and where the
    # team's order of summing the centre's delta makes one rounding fall the other way, the
    # difference travels on through word 3's column (seen: 2 elements in 10^5 beyond 3 steps,
    # 0.4 % of the column's movement); one missed write per occurrence would be a tenth of it.
    def steps(got, want, before):
        g, w, b = (cpumach.bf16_widen(x) for x in (got, want, before))
        step = np.maximum(np.maximum(np.abs(g), np.abs(w)), np.abs(b)) * 2.0 ** -7 + 1e-30
        return np.abs(g - w) / step
    assert steps_apart(Bo[3], B[3]) > 20.0
    sa, sb = steps(b16.host16(Ad), Ao, A), steps(b16.host16(Bd), Bo, B)
    if hot:
        assert max(sa.max(), sb.max()) <= 1.01, (sa.max(), sb.max())
    else:
        assert max((sa > 3.0).mean(), (sb > 3.0).mean()) <= 1e-3
        g, w, b = (cpumach.bf16_widen(x[3]) for x in (b16.host16(Bd), Bo, B))
        assert np.abs(g - w).mean() <= 0.02 * np.abs(w - b).mean()


@pytest.mark.parametrize("d,nwa,nwb", [(100, 5, 5), (300, 5, 5), (200, 12, 3)])
def test_one_worker_lands_on_the_sequential_negative_pass(gpu, oracle, hot, d, nwa, nwb):
    """16 groups over 14 words: B columns change from row to row and from group to group, A
    columns from group to group."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(d + nwa)
    V, G = 14, 16
    A, B = b16.tables16(rng, V, d, 0.3)
    WA = np.concatenate([rng.permutation(V)[:nwa] for _ in range(G)]).astype(np.int32)
    WB = np.concatenate([rng.permutation(V)[:nwb] for _ in range(G)]).astype(np.int32)
    WB[1] = WB[0]                        # one group with the same B word in rows 0 and 1
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.05, 0.5, 78, hot)
    Ad, Bd = b16.dev16(torch, A), b16.dev16(torch, B)
    assert CUMACH.word2vecNegBf16(d, G, nwa, nwb, b16.dev(torch, WA), b16.dev(torch, WB), Ad, Bd,
                                  0.05, 0.5, 78) == 0
    apart = max(steps_apart(b16.host16(Ad), Ao), steps_apart(b16.host16(Bd), Bo))
    moved = max(steps_apart(Ao, A), steps_apart(Bo, B))
    print("\nnegative pass, d %d, %d frequent words: %.2f bf16 steps from the sequential oracle "
          "(the pass moved the tables by %.0f steps)" % (d, hot, apart, moved))
    assert moved > 20.0
    assert apart <= (1.01 if hot else 3.0), apart


def test_ordered_bf16_under_a_bound_on_workgroups(gpu, oracle, ordered, hot):
    """w2v_set_max_workgroups bounds the ordered kernels' workers as well (one workgroup: four
    workers, which then walk longer ranges)."""
    ordered.w2v_set_max_workgroups(1)
    try:
        b16.test_pos_update_bf16(gpu, oracle, hot, 0.5, 300, 5, 300)
        b16.test_neg_update_bf16(gpu, oracle, hot, 0.5, 300, 5, 5, 400)
        b16.test_neg_update_bf16(gpu, oracle, hot, 0.0, 40, 70, 3, 40)   # the few-waves stand-in
    finally:
        ordered.w2v_set_max_workgroups(0)


@pytest.fixture
def rare_stores():
    """Every word outside the side buffers counts as rare within the launch (forced threshold:
    up to 64 occurrences), so the ordered kernels write it back with plain stores instead of
    compare-and-swap exchanges (store_col16 in w2v_bf16.h)."""
    from bidmach_amd.cumach import load_library
    lib = load_library()
    assert lib.w2v_get_rare_update_mode() == -1
    lib.w2v_set_rare_update_mode(64)
    yield lib
    lib.w2v_set_rare_update_mode(-1)


@pytest.mark.parametrize("d,skip,ncentres", [(100, 5, 300), (300, 5, 300), (65, 3, 100)])
def test_pos_update_bf16_ordered_with_plain_stores(gpu, oracle, ordered, rare_stores, hot, d, skip,
                                                   ncentres):
    """Without overlapping updates a plain store leaves the bits the exchange would."""
    b16.test_pos_update_bf16(gpu, oracle, hot, 0.5, d, skip, ncentres)


@pytest.mark.parametrize("d,nwa,nwb,G", [(100, 5, 5, 400), (300, 5, 5, 400), (65, 7, 8, 100),
                                         (512, 15, 5, 100)])
def test_neg_update_bf16_ordered_with_plain_stores(gpu, oracle, ordered, rare_stores, hot, d, nwa,
                                                   nwb, G):
    b16.test_neg_update_bf16(gpu, oracle, hot, 0.5, d, nwa, nwb, G)
