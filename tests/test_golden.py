"""Replay of the committed fixture tests/golden/sgns_small.npz (see make_fixtures.py for what it
holds and why it cannot be reference output)."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sgns_small.npz")


@pytest.fixture(scope="module")
def g():
    return np.load(GOLDEN)


def test_fixture_is_self_consistent(g):
    """Oracle outputs stored in the fixture agree with the float64 closed forms stored beside them."""
    assert float(g["evalpos"]) == pytest.approx(float(g["evalpos_closed"]), rel=2e-6)
    assert float(g["evalneg"]) == pytest.approx(float(g["evalneg_closed"]), rel=2e-6)
    for k in ("posA", "posB", "negA", "negB"):
        assert np.abs(g[k] - g[k + "_closed"]).max() < 5e-5
        assert np.abs(g[k] - g[k[-1]]).max() > 1e-3     # the update is not a no-op


def test_oracle_reproduces_fixture(g, oracle):
    d, skip, nwa, nwb = int(g["d"]), int(g["skip"]), int(g["nwa"]), int(g["nwb"])
    A, B = g["A"], g["B"]
    lr, vexp = float(g["lrate"]), float(g["vexp"])
    assert oracle.word2vecEvalPos(d, g["eW"].shape[0], skip, g["eW"], g["eLB"], g["eUB"], A, B, 1) \
        == float(g["evalpos"])
    assert oracle.word2vecEvalNeg(d, g["eWA"].shape[0] // nwa, nwa, nwb, g["eWA"], g["eWB"], A, B,
                                  1) == float(g["evalneg"])
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecPos(d, g["pW"].shape[0], skip, g["pW"], g["pLB"], g["pUB"], A2, B2, lr, vexp, 3)
    assert np.array_equal(A2, g["posA"]) and np.array_equal(B2, g["posB"])
    A2, B2 = A.copy(), B.copy()
    oracle.word2vecNeg(d, g["nWA"].shape[0] // nwa, nwa, nwb, g["nWA"], g["nWB"], A2, B2, lr, vexp,
                       3)
    assert np.array_equal(A2, g["negA"]) and np.array_equal(B2, g["negB"])


@pytest.mark.gpu
def test_hip_library_reproduces_fixture(g):
    import torch
    from bidmach_amd.cumach import CUMACH

    def dev(x):
        return torch.from_numpy(np.ascontiguousarray(x)).cuda()

    d, skip, nwa, nwb = int(g["d"]), int(g["skip"]), int(g["nwa"]), int(g["nwb"])
    lr, vexp = float(g["lrate"]), float(g["vexp"])
    ret = torch.zeros(2, dtype=torch.float64, device="cuda")
    A, B = dev(g["A"]), dev(g["B"])
    assert CUMACH.word2vecEvalPosF64(d, g["eW"].shape[0], skip, dev(g["eW"]), dev(g["eLB"]),
                                     dev(g["eUB"]), A, B, ret[0:1]) == 0
    assert CUMACH.word2vecEvalNegF64(d, g["eWA"].shape[0] // nwa, nwa, nwb, dev(g["eWA"]),
                                     dev(g["eWB"]), A, B, ret[1:2]) == 0
    r = ret.cpu().numpy()
    assert r[0] == pytest.approx(float(g["evalpos"]), rel=1e-5)
    assert r[1] == pytest.approx(float(g["evalneg"]), rel=1e-5)
    A, B = dev(g["A"]), dev(g["B"])
    assert CUMACH.word2vecPos(d, g["pW"].shape[0], skip, dev(g["pW"]), dev(g["pLB"]),
                              dev(g["pUB"]), A, B, lr, vexp) == 0
    assert np.abs(A.cpu().numpy() - g["posA"]).max() <= 1e-4
    assert np.abs(B.cpu().numpy() - g["posB"]).max() <= 1e-4
    A, B = dev(g["A"]), dev(g["B"])
    assert CUMACH.word2vecNeg(d, g["nWA"].shape[0] // nwa, nwa, nwb, dev(g["nWA"]), dev(g["nWB"]),
                              A, B, lr, vexp) == 0
    assert np.abs(A.cpu().numpy() - g["negA"]).max() <= 1e-4
    assert np.abs(B.cpu().numpy() - g["negB"]).max() <= 1e-4
