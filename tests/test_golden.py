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


# ---- sliced, multi-part model fixture ------------------------------------------------------------

SLICE_GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                            "sgns_slice_small.npz")


@pytest.fixture(scope="module")
def gs():
    return np.load(SLICE_GOLDEN)


def _slicing(gs):
    return tuple(int(gs[k]) for k in ("islice", "nslices", "nhead", "maxcols", "dohead"))


def _model_list(gs):
    from oracle import closed_form as cf
    islice, nslices, nhead, maxcols, _ = _slicing(gs)
    ap = cf.pack_parts(gs["A"], islice, nslices, nhead, maxcols)
    bp = cf.pack_parts(gs["B"], islice, nslices, nhead, maxcols)
    return ap, bp, [m for pair in zip(bp, ap) for m in pair]


def test_slice_fixture_is_self_consistent(gs):
    assert float(gs["evalpos"]) == pytest.approx(float(gs["evalpos_closed"]), rel=2e-6)
    assert float(gs["evalneg"]) == pytest.approx(float(gs["evalneg_closed"]), rel=2e-6)
    for k in ("posA", "posB", "negA", "negB"):
        assert np.abs(gs[k] - gs[k + "_closed"]).max() < 5e-5
        assert np.abs(gs[k] - gs[k[-1]]).max() > 1e-3


def test_oracle_reproduces_slice_fixture(gs, oracle):
    from oracle import closed_form as cf
    d, skip, nwa, nwb = int(gs["d"]), int(gs["skip"]), int(gs["nwa"]), int(gs["nwb"])
    islice, nslices, nhead, maxcols, dohead = _slicing(gs)
    lr, vexp = float(gs["lrate"]), float(gs["vexp"])
    sl = (islice, nslices, maxcols, nhead, 0)
    _, _, mm = _model_list(gs)
    assert oracle.word2vecEvalPosSlice(d, gs["eW"].shape[0], skip, gs["eW"], gs["eLB"], gs["eUB"],
                                       mm, 1, *sl) == float(gs["evalpos"])
    assert oracle.word2vecEvalNegSlice(d, gs["eWA"].shape[0] // nwa, nwa, nwb, gs["eWA"],
                                       gs["eWB"], mm, 1, *sl) == float(gs["evalneg"])
    ap, bp, mm = _model_list(gs)
    oracle.word2vecPosSlice(d, gs["pW"].shape[0], skip, gs["pW"], gs["pLB"], gs["pUB"], mm, lr,
                            vexp, 2, *sl, dohead)
    assert np.array_equal(cf.unpack_parts(ap, gs["A"], islice, nslices, nhead), gs["posA"])
    assert np.array_equal(cf.unpack_parts(bp, gs["B"], islice, nslices, nhead), gs["posB"])
    ap, bp, mm = _model_list(gs)
    oracle.word2vecNegSlice(d, gs["nWA"].shape[0] // nwa, nwa, nwb, gs["nWA"], gs["nWB"], mm, lr,
                            vexp, 2, *sl, dohead)
    assert np.array_equal(cf.unpack_parts(ap, gs["A"], islice, nslices, nhead), gs["negA"])
    assert np.array_equal(cf.unpack_parts(bp, gs["B"], islice, nslices, nhead), gs["negB"])


@pytest.mark.gpu
def test_hip_library_reproduces_slice_fixture(gs):
    import torch
    from bidmach_amd.cumach import CUMACH, load_library
    from oracle import closed_form as cf

    def dev(x):
        return torch.from_numpy(np.ascontiguousarray(x)).cuda()

    d, skip, nwa, nwb = int(gs["d"]), int(gs["skip"]), int(gs["nwa"]), int(gs["nwb"])
    islice, nslices, nhead, maxcols, dohead = _slicing(gs)
    lr, vexp = float(gs["lrate"]), float(gs["vexp"])
    sl = (islice, nslices, maxcols, nhead, False)
    lib = load_library()
    old = lib.w2v_get_eval_floor()
    lib.w2v_set_eval_floor(1.0e-20)
    try:
        ret = torch.zeros(2, dtype=torch.float64, device="cuda")
        mm = [dev(m) for m in _model_list(gs)[2]]
        assert CUMACH.word2vecEvalPosSlice(d, gs["eW"].shape[0], skip, dev(gs["eW"]),
                                           dev(gs["eLB"]), dev(gs["eUB"]), mm, *sl, ret[0:1]) == 0
        assert CUMACH.word2vecEvalNegSlice(d, gs["eWA"].shape[0] // nwa, nwa, nwb, dev(gs["eWA"]),
                                           dev(gs["eWB"]), mm, *sl, ret[1:2]) == 0
    finally:
        lib.w2v_set_eval_floor(old)
    r = ret.cpu().numpy()
    assert r[0] == pytest.approx(float(gs["evalpos"]), rel=1e-5)
    assert r[1] == pytest.approx(float(gs["evalneg"]), rel=1e-5)

    def logical(mm, which, full):
        parts = [m.cpu().numpy() for m in mm[which::2]]
        return cf.unpack_parts(parts, full, islice, nslices, nhead)

    mm = [dev(m) for m in _model_list(gs)[2]]
    assert CUMACH.word2vecPosSlice(d, gs["pW"].shape[0], skip, dev(gs["pW"]), dev(gs["pLB"]),
                                   dev(gs["pUB"]), mm, lr, vexp, *sl, dohead) == 0
    assert np.abs(logical(mm, 1, gs["A"]) - gs["posA"]).max() <= 1e-4
    assert np.abs(logical(mm, 0, gs["B"]) - gs["posB"]).max() <= 1e-4
    mm = [dev(m) for m in _model_list(gs)[2]]
    assert CUMACH.word2vecNegSlice(d, gs["nWA"].shape[0] // nwa, nwa, nwb, dev(gs["nWA"]),
                                   dev(gs["nWB"]), mm, lr, vexp, *sl, dohead) == 0
    assert np.abs(logical(mm, 1, gs["A"]) - gs["negA"]).max() <= 1e-4
    assert np.abs(logical(mm, 0, gs["B"]) - gs["negB"]).max() <= 1e-4
