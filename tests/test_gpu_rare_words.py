"""word2vecNeg's plain read-modify-write for words that are rare within a call (see
w2v_set_rare_update_mode in include/bidmach_w2v.h).  The default applies it only to calls with tens
of thousands of groups, so the parity tests never reach it; here the threshold is forced.
(needs an MI355X)
"""
import numpy as np
import pytest

from bidmach_amd import corpus
from tests import test_gpu_parity as parity
from tests import test_gpu_slice as sliced

pytestmark = pytest.mark.gpu

gpu = parity.gpu


@pytest.fixture(params=[2, 64], ids=["upto2", "upto64"])
def rare_mode(request):
    from bidmach_amd.cumach import load_library
    lib = load_library()
    assert lib.w2v_get_rare_update_mode() == -1
    lib.w2v_set_rare_update_mode(request.param)
    assert lib.w2v_get_rare_update_mode() == request.param
    yield request.param
    lib.w2v_set_rare_update_mode(-1)
    assert lib.w2v_get_rare_update_mode() == -1


def test_collision_free_updates_match_oracle(gpu, oracle, rare_mode):
    """Every word occurs once, so every column beyond the 16 lowest ids takes the plain path."""
    for vexp in (0.0, 0.5):
        parity.test_neg_update_matches_oracle(gpu, oracle, vexp, 300, 5, 5, 400)
        parity.test_neg_update_matches_oracle(gpu, oracle, vexp, 65, 7, 8, 100)
        parity.test_neg_update_matches_oracle(gpu, oracle, vexp, 1280, 5, 5, 30)
        parity.test_neg_update_matches_oracle(gpu, oracle, vexp, 40, 70, 3, 40)
    parity.test_neg_filt_matches_oracle(gpu, oracle, 100, 10, 5)


def test_sliced_model_matches_oracle(gpu, oracle, rare_mode):
    """Collision-free groups against a sliced, multi-part model: columns that are not written
    (read-only head words, words of other workers) must stay bit-identical too."""
    for slicing in sliced.SLICINGS:
        sliced.test_neg_slice_matches_oracle(gpu, oracle, *slicing, 100, 5, 5, 0.0)
        sliced.test_neg_slice_matches_oracle(gpu, oracle, *slicing, 130, 3, 8, 0.5)
        sliced.test_neg_slice_matches_oracle(gpu, oracle, *slicing, 64, 70, 2, 0.0)


def test_plain_path_is_bit_identical_to_atomics_without_collisions(gpu, rare_mode):
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(11)
    d, V, G, nwa, nwb = 300, 50000, 2000, 5, 5
    A, B = parity.rand_tables(rng, V, d, 0.2)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    got = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.025, 0.5)
    lib.w2v_set_rare_update_mode(0)
    want = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.025, 0.5)
    lib.w2v_set_rare_update_mode(rare_mode)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    assert not np.array_equal(got[0], A)


def test_frequent_words_stay_atomic_and_exact(gpu, rare_mode):
    """64 words with thousands of occurrences each next to 40,000 words that occur at most twice:
    the frequent ones must still receive every contribution (A is zero, so each A delta is
    -lr/2 times a sum of B columns whatever the interleaving), the rare ones take the plain path."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(12)
    d, V, G, nwa, nwb = 128, 50000, 20000, 5, 5
    A = np.zeros((V, d), np.float32)
    B = (rng.standard_normal((V, d)) * 0.1).astype(np.float32)
    WA = rng.integers(100, 164, G * nwa).astype(np.int32)          # frequent
    rare = rng.permutation(np.arange(1000, V))[:G * nwa // 5]
    WA[::5] = rare                                                  # one rare word per group
    WB = rng.integers(100, 164, G * nwb).astype(np.int32)
    lr = 1e-6
    Ad, Bd = parity.dev(torch, A), parity.dev(torch, B)
    assert CUMACH.word2vecNeg(d, G, nwa, nwb, parity.dev(torch, WA), parity.dev(torch, WB), Ad, Bd,
                              lr, 0.0) == 0
    wa, wb = WA.reshape(G, nwa), WB.reshape(G, nwb)
    sumB = B.astype(np.float64)[wb].sum(axis=1)
    want = np.zeros((V, d))
    np.add.at(want, wa.reshape(-1), np.repeat(-lr * 0.5 * sumB, nwa, axis=0))
    got = Ad.cpu().numpy().astype(np.float64)
    scale = np.abs(want[100:164]).max()
    assert scale > 1e-4
    assert np.abs(got[100:164] - want[100:164]).max() < 5e-3 * scale
    # each rare word occurs once: its column holds exactly its one contribution
    rscale = np.abs(want[rare]).max()
    assert np.abs(got[rare] - want[rare]).max() < 5e-3 * rscale
    untouched = np.setdiff1d(np.arange(V), np.concatenate([rare, np.arange(100, 164)]))
    assert not got[untouched].any()


def test_small_tables_are_updated_coherently_across_the_device(gpu, oracle, rare_mode):
    """A table small enough to stay in every L2 slice of the device, trained with all words
    treated as rare as far as the threshold allows: the result must stay as close to the
    sequential oracle as the all-atomic run does (an update path that kept XCD-local copies of the
    columns would lose most of the updates)."""
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(13)
    d, V, G, nwa, nwb = 100, 4000, 40000, 5, 5
    A, B = parity.rand_tables(rng, V, d, 0.2)
    WA = rng.integers(16, V, G * nwa).astype(np.int32)    # ~50 occurrences per word
    WB = rng.integers(16, V, G * nwb).astype(np.int32)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNeg(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.01, 0.0, 1)
    try:
        # one workgroup per XCD: 32 groups in flight, so that two updates of one word rarely
        # overlap and what is measured is whether the XCDs see each other's stores
        lib.w2v_set_max_workgroups(8)
        got = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.01, 0.0)
        lib.w2v_set_rare_update_mode(0)
        ref = parity.gpu_neg(gpu, d, G, nwa, nwb, WA, WB, A, B, 0.01, 0.0)
    finally:
        lib.w2v_set_max_workgroups(0)
        lib.w2v_set_rare_update_mode(rare_mode)
    moved = np.abs(Ao - A).mean() + np.abs(Bo - B).mean()
    dist_ref = np.abs(ref[0] - Ao).mean() + np.abs(ref[1] - Bo).mean()
    dist_got = np.abs(got[0] - Ao).mean() + np.abs(got[1] - Bo).mean()
    print("\nmean |update| %.3e; distance from the sequential oracle: atomics %.3e, rare mode %d %.3e"
          % (moved, dist_ref, rare_mode, dist_got))
    assert dist_ref < 0.1 * moved
    assert dist_got < 2.0 * dist_ref + 0.01 * moved
