"""The two ways the library updates the most frequent words (exact and combining, see
w2v_set_hot_update_mode in include/bidmach_w2v.h), each forced in turn, against the same oracle
checks as the default.  The default picks per launch and takes the exact mode for the small launches
of the parity tests, so without forcing it the combining mode would only be exercised by the
full-size tests.  (needs an MI355X)
"""
import numpy as np
import pytest

from bidmach_amd import corpus
from tests import test_gpu_parity as parity
from tests import test_gpu_slice as sliced

pytestmark = pytest.mark.gpu

gpu = parity.gpu


@pytest.fixture(params=[0, 1, 2], ids=["exact", "combining", "off"])
def hot_mode(request):
    from bidmach_amd.cumach import load_library
    lib = load_library()
    assert lib.w2v_get_hot_update_mode() == -1
    lib.w2v_set_hot_update_mode(request.param)
    assert lib.w2v_get_hot_update_mode() == request.param
    yield request.param
    lib.w2v_set_hot_update_mode(-1)


def test_collision_free_updates(gpu, oracle, hot_mode):
    """Word ids 0..15 are among the ids of these minibatches, each written once."""
    parity.test_pos_update_matches_oracle(gpu, oracle, 0.5, 300, 5, 300)
    parity.test_neg_update_matches_oracle(gpu, oracle, 0.5, 300, 5, 5, 400)
    parity.test_pos_update_ragged_windows_and_tile_edges(gpu, oracle)
    parity.test_neg_filt_matches_oracle(gpu, oracle, 100, 10, 5)


def test_heavy_collisions_lose_no_contribution(gpu, hot_mode):
    parity.test_heavy_collisions_lose_no_contribution(gpu)


def test_sliced_model(gpu, oracle, hot_mode):
    sliced.test_pos_slice_matches_oracle(gpu, oracle, 1, 3, 40, 397, 2, False, 100, 0.0)
    sliced.test_neg_slice_matches_oracle(gpu, oracle, 0, 2, 500, 333, 2, True, 100, 5, 5, 0.0)
    sliced.test_colliding_minibatch_stays_close_to_sequential_oracle(gpu, oracle)


@pytest.mark.parametrize("d", [37, 128, 300, 1280])
def test_hot_columns_receive_every_update_exactly_once(gpu, hot_mode, d):
    """Only words 0..15, tens of thousands of updates each, with the A table zero: every B delta
    is then lr * 0.5 * 0 = 0 and every A delta is the sum of -lr/2 * B columns, known exactly up
    to rounding whatever the interleaving.  Shadow copies that lost or duplicated a write, or a
    fold that dropped what it swapped out, would show as a wrong multiple."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(4)
    V, G, nwa, nwb = 64, (60000 if d <= 300 else 12000), 5, 5
    A = np.zeros((V, d), np.float32)
    B = (rng.standard_normal((V, d)) * 0.1 * (128.0 / d) ** 0.5).astype(np.float32)
    WA = rng.integers(0, 16, G * nwa).astype(np.int32)
    WB = rng.integers(0, 16, G * nwb).astype(np.int32)
    lr = 1e-6
    Ad, Bd = parity.dev(torch, A), parity.dev(torch, B)
    assert CUMACH.word2vecNeg(d, G, nwa, nwb, parity.dev(torch, WA), parity.dev(torch, WB), Ad, Bd,
                              lr, 0.0) == 0
    # dA[w] = -lr * sum over (group, j with WA = w, k) of sigmoid(A.B ~ 0) * B[WB]; A stays ~1e-2 at
    # most, so sigmoid = 0.5 to first order
    wa = WA.reshape(G, nwa)
    wb = WB.reshape(G, nwb)
    sumB = B.astype(np.float64)[wb].sum(axis=1)                    # G x d
    want = np.zeros((V, d))
    np.add.at(want, wa.reshape(-1), np.repeat(-lr * 0.5 * sumB, nwa, axis=0))
    got = Ad.cpu().numpy().astype(np.float64)
    scale = np.abs(want).max()
    assert scale > 1e-4
    assert np.abs(got - want).max() < 5e-3 * scale
    assert np.abs(Bd.cpu().numpy() - B).max() < 5e-3 * np.abs(B).max()


def test_default_mode_decides_per_table(gpu):
    """No forced mode.  The words read from table B hold no hot id at all, a twentieth of those
    read from table A are id 0 (what the reference's closed-form negative sampler does at a large
    vocabulary): table A must get its shadow copies while table B goes without, and A's column 0
    must still receive each of its 75,000 contributions exactly once (A starts at zero, so each is
    -lr/2 times a sum of B columns to first order, whatever the interleaving)."""
    torch, CUMACH = gpu
    from bidmach_amd.cumach import load_library
    assert load_library().w2v_get_hot_update_mode() == -1
    rng = np.random.default_rng(21)
    d, V, G, nwa, nwb = 64, 5000, 300000, 5, 5
    A = np.zeros((V, d), np.float32)
    B = (rng.standard_normal((V, d)) * 0.1).astype(np.float32)
    WA = rng.integers(16, V, G * nwa).astype(np.int32)
    WA[rng.random(G * nwa) < 0.05] = 0
    WB = rng.integers(16, V, G * nwb).astype(np.int32)
    lr = 1e-7
    Ad, Bd = parity.dev(torch, A), parity.dev(torch, B)
    assert CUMACH.word2vecNeg(d, G, nwa, nwb, parity.dev(torch, WA), parity.dev(torch, WB), Ad, Bd,
                              lr, 0.0) == 0
    wa, wb = WA.reshape(G, nwa), WB.reshape(G, nwb)
    sumB = B.astype(np.float64)[wb].sum(axis=1)                    # G x d
    want = np.zeros((V, d))
    np.add.at(want, wa.reshape(-1), np.repeat(-lr * 0.5 * sumB, nwa, axis=0))
    got = Ad.cpu().numpy().astype(np.float64)
    assert (wa == 0).sum() > 70000
    scale0 = np.abs(want[0]).max()
    assert np.abs(got[0] - want[0]).max() < 5e-3 * scale0
    assert np.abs(got - want).max() < 5e-3 * np.abs(want).max()


def test_mode_argument_is_normalised(gpu):
    from bidmach_amd.cumach import load_library
    lib = load_library()
    for given, kept in ((7, -1), (1, 1), (0, 0), (2, 2), (-5, -1)):
        lib.w2v_set_hot_update_mode(given)
        assert lib.w2v_get_hot_update_mode() == kept
    lib.w2v_set_hot_update_mode(-1)
