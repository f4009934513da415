"""word2vecEvalNegNoAlloc, the entry point that allocates nothing, against word2vecEvalNeg through
the C ABI (needs an MI355X).  Two calls in a row, the second on a smaller input: both must give
the ordinary entry point's sum (and the oracle's, to 1e-5), and the device's free memory must not
move across the calls."""
import ctypes

import numpy as np
import pytest

from bidmach_amd import corpus

pytestmark = pytest.mark.gpu


def test_no_alloc_entry_point_matches_the_ordinary_one_twice_in_a_row(oracle):
    import torch
    assert torch.cuda.is_available()
    from bidmach_amd.cumach import load_library
    lib = load_library()
    rng = np.random.default_rng(12)
    d, V, nwa, nwb = 300, 20000, 5, 5
    A = (rng.standard_normal((V, d)) * 0.2).astype(np.float32)
    B = (rng.standard_normal((V, d)) * 0.2).astype(np.float32)
    Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr())

    # make sure the ordinary path's scratch (and the code object) exist before free memory is read
    big = 60000
    WA0 = rng.integers(0, V, big * nwa).astype(np.int32)
    WB0 = corpus.zipf_stream(big * nwb, V, 1.0, seed=1)
    WAd0, WBd0 = torch.from_numpy(WA0).cuda(), torch.from_numpy(WB0).cuda()
    ret = torch.zeros(4, dtype=torch.float32, device="cuda")
    assert lib.word2vecEvalNeg(d, big, nwa, nwb, ptr(WAd0), ptr(WBd0), ptr(Ad), ptr(Bd),
                               ptr(ret[0:1])) == 0
    # the first call on a device looks the array's address up, which is when the runtime may
    # materialise the code object's data segment: done here, before free memory is read
    assert lib.word2vecEvalNegNoAlloc(d, 8, nwa, nwb, ptr(WAd0), ptr(WBd0), ptr(Ad), ptr(Bd),
                                      ptr(ret[2:3])) == 0
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]

    for call, G in enumerate((big, 777)):        # the second call is the smaller one
        WA, WB = WA0[:G * nwa].copy(), WB0[:G * nwb].copy()
        WAd, WBd = torch.from_numpy(WA).cuda(), torch.from_numpy(WB).cuda()
        torch.cuda.synchronize()
        before = torch.cuda.mem_get_info()[0]
        ret.zero_()
        torch.cuda.synchronize()
        err = lib.word2vecEvalNegNoAlloc(d, G, nwa, nwb, ptr(WAd), ptr(WBd), ptr(Ad), ptr(Bd),
                                         ptr(ret[0:1]))
        assert err == 0
        assert torch.cuda.mem_get_info()[0] == before      # no device memory was taken
        assert lib.word2vecEvalNeg(d, G, nwa, nwb, ptr(WAd), ptr(WBd), ptr(Ad), ptr(Bd),
                                   ptr(ret[1:2])) == 0
        got = ret.cpu().numpy()
        want = oracle.word2vecEvalNeg(d, G, nwa, nwb, WA, WB, A, B, 4)
        assert got[0] == got[1], (call, got)               # same kernels, same fold order
        assert got[0] == pytest.approx(want, rel=1e-5)
        assert want < -100.0
    assert torch.cuda.mem_get_info()[0] >= free0 - (4 << 20)


def test_no_alloc_entry_point_adds_into_retval_and_rejects_what_it_cannot_take():
    import torch
    from bidmach_amd.cumach import load_library
    lib = load_library()
    d, V, G = 64, 100, 50
    t = torch.randn(V, d, device="cuda") * 0.1
    ids = torch.randint(0, V, (G * 5,), dtype=torch.int32, device="cuda")
    ret = torch.full((2,), 10.0, dtype=torch.float32, device="cuda")

    def ptr(x):
        return ctypes.c_void_p(x.data_ptr())

    assert lib.word2vecEvalNegNoAlloc(d, G, 5, 5, ptr(ids), ptr(ids), ptr(t), ptr(t), ptr(ret[0:1])) == 0
    ref = torch.zeros(1, dtype=torch.float32, device="cuda")
    assert lib.word2vecEvalNeg(d, G, 5, 5, ptr(ids), ptr(ids), ptr(t), ptr(t), ptr(ref)) == 0
    assert float(ret[0].item()) == pytest.approx(10.0 + float(ref.item()), rel=1e-6)
    assert float(ret[1].item()) == 10.0
    limit = lib.w2v_no_alloc_max_groups()
    assert limit == 1 << 24
    # beyond the stated maximum: rejected before anything is launched (the id arrays are never read)
    assert lib.word2vecEvalNegNoAlloc(d, limit + 1, 5, 5, ptr(ids), ptr(ids), ptr(t), ptr(t),
                                      ptr(ret[0:1])) == 1
    assert lib.word2vecEvalNegNoAlloc(d, G, 5, 5, ptr(ids), ptr(ids), ptr(t), ptr(t), None) == 1
    assert lib.word2vecEvalNegNoAlloc(d, 0, 5, 5, ptr(ids), ptr(ids), ptr(t), ptr(t), ptr(ret[0:1])) == 0
    assert float(ret[1].item()) == 10.0
