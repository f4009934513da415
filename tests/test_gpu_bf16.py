"""The bfloat16-storage operators against their CPU oracle, through the C ABI (needs an MI355X).

Bars.  Forward sums: 1e-5 relative.  Updates on collision-free minibatches: the library and the
oracle round every element with the same random bits, so the stored bit patterns agree except
where the two fp32 values (which differ in their last bits because the dot is summed in another
order) fall on different sides of a rounding threshold: such elements must be rare and one
bfloat16 step apart (plus a few fp32 ulps of the column's scale where terms cancel).  With
tables at the reference's initial scale one bfloat16 step is below 1e-4, and the result is also
held to 1e-4 absolute against the fp32 oracle.
"""
import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import cpumach

pytestmark = pytest.mark.gpu

EVAL_RTOL = 1e-5
UPDATE_ATOL = 1e-4
MAX_FLIPPED = 0.005   # share of elements allowed to sit one bf16 step from the oracle's


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    from bidmach_amd.cumach import CUMACH, load_library
    load_library()
    return torch, CUMACH


@pytest.fixture(params=[0, 1024, 4096])
def hot(request):
    """Number of frequent words the library routes through fp32 side buffers; the oracle is told
    the same number."""
    from bidmach_amd.cumach import load_library
    lib = load_library()
    old = lib.w2v_get_bf16_hot_words()
    assert lib.w2v_set_bf16_hot_words(request.param) == 0
    yield request.param
    lib.w2v_set_bf16_hot_words(old)


def dev16(torch, h):
    """uint16 bit patterns -> device tensor of the same bits."""
    return torch.from_numpy(np.ascontiguousarray(h).view(np.int16)).cuda()


def host16(t):
    return t.cpu().numpy().view(np.uint16)


def dev(torch, x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def tables16(rng, vocab, d, scale):
    A = cpumach.bf16_truncate((rng.standard_normal((vocab, d)) * scale).astype(np.float32))
    B = cpumach.bf16_truncate((rng.standard_normal((vocab, d)) * scale).astype(np.float32))
    return A, B


def assert_same_roundings(got, want, old, what):
    """Bit patterns agree except on rare elements, and those are one bfloat16 step apart.  Where
    the terms of an update cancel (against the old value or against each other) the two fp32
    results differ by rounding errors of the size of the terms, so a few fp32 ulps of the
    column's largest value are allowed on top of the step."""
    assert (got != want).mean() <= MAX_FLIPPED, "%s: %.4f of the elements differ" % (
        what, (got != want).mean())
    g, w, o = cpumach.bf16_widen(got), cpumach.bf16_widen(want), cpumach.bf16_widen(old)
    allowed = np.abs(w) * 2.0 ** -7 + (np.abs(o) + np.abs(w)).max(axis=1, keepdims=True) * 2.0 ** -18
    assert (np.abs(g - w) <= allowed).all(), "%s: more than one bf16 step from the oracle" % what


@pytest.mark.parametrize("d,V,N,skip", [
    (100, 1000, 20000, 5), (300, 5000, 30000, 5), (512, 2000, 8000, 10), (1, 10, 100, 2),
    (64, 300, 3000, 3), (65, 300, 3000, 3), (1280, 200, 500, 5), (37, 100, 2000, 40),
    (130, 300, 3000, 4),
])
def test_eval_pos_bf16(gpu, oracle, d, V, N, skip):
    torch, CUMACH = gpu
    rng = np.random.default_rng(d + N)
    A, B = tables16(rng, V, d, 0.6 / d ** 0.25)
    W = corpus.zipf_stream(N, V, 1.0, seed=d)
    W[rng.random(N) < 0.07] = -1
    sent = np.cumsum(rng.random(N) < 0.03)
    LB, UB = corpus.window_bounds(N, skip, rng, sentence=sent)
    want = oracle.word2vecEvalPosBf16(d, N, skip, W, LB, UB, A, B)
    ret = torch.full((1,), 10.0, dtype=torch.float64, device="cuda")
    err = CUMACH.word2vecEvalPosBf16(d, N, skip, dev(torch, W), dev(torch, LB), dev(torch, UB),
                                     dev16(torch, A), dev16(torch, B), ret)
    assert err == 0
    assert want < -1.0
    assert float(ret.item()) - 10.0 == pytest.approx(want, rel=EVAL_RTOL)   # added into Retval


@pytest.mark.parametrize("d,V,G,nwa,nwb", [
    (100, 1000, 5000, 5, 5), (300, 5000, 6000, 5, 5), (512, 2000, 2000, 15, 5), (1, 10, 50, 1, 1),
    (64, 300, 500, 3, 2), (65, 300, 500, 7, 8), (1280, 200, 100, 5, 5), (50, 400, 300, 70, 4),
    (300, 500, 1000, 9, 1),
    # more B words than a wave holds at once
    (300, 500, 300, 5, 10), (100, 500, 200, 4, 21), (64, 300, 100, 3, 64),
])
def test_eval_neg_bf16(gpu, oracle, d, V, G, nwa, nwb):
    torch, CUMACH = gpu
    rng = np.random.default_rng(d + G)
    A, B = tables16(rng, V, d, 0.6 / d ** 0.25)
    WA = rng.integers(0, V, G * nwa).astype(np.int32)
    WB = corpus.zipf_stream(G * nwb, V, 1.0, seed=G)
    want = oracle.word2vecEvalNegBf16(d, G, nwa, nwb, WA, WB, A, B)
    ret = torch.zeros(1, dtype=torch.float64, device="cuda")
    err = CUMACH.word2vecEvalNegBf16(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB),
                                     dev16(torch, A), dev16(torch, B), ret)
    assert err == 0
    assert float(ret.item()) == pytest.approx(want, rel=EVAL_RTOL)


@pytest.mark.parametrize("vexp", [0.0, 0.5, 0.75])
@pytest.mark.parametrize("d,skip,ncentres", [(100, 5, 300), (300, 5, 300), (512, 10, 100),
                                             (1, 2, 50), (65, 3, 100), (1280, 5, 40),
                                             (24, 40, 30), (130, 4, 100)])
def test_pos_update_bf16(gpu, oracle, hot, vexp, d, skip, ncentres):
    torch, CUMACH = gpu
    rng = np.random.default_rng(d * 7 + skip)
    V = 20000
    A, B = tables16(rng, V, d, 0.5 / d ** 0.25)
    W, LB, UB = corpus.collision_free_pos(ncentres, skip, V, rng)
    W[rng.random(W.shape[0]) < 0.05] = -1
    seed = 0x1234567 + d
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecPosBf16(d, W.shape[0], skip, W, LB, UB, Ao, Bo, 0.025, vexp, seed, hot)
    Ad, Bd = dev16(torch, A), dev16(torch, B)
    err = CUMACH.word2vecPosBf16(d, W.shape[0], skip, dev(torch, W), dev(torch, LB),
                                 dev(torch, UB), Ad, Bd, 0.025, vexp, seed)
    assert err == 0
    assert_same_roundings(host16(Ad), Ao, A, "A")
    assert_same_roundings(host16(Bd), Bo, B, "B")
    assert (Ao != A).any() and (Bo != B).any()


@pytest.mark.parametrize("vexp", [0.0, 0.5, 0.75])
@pytest.mark.parametrize("d,nwa,nwb,G", [(100, 5, 5, 400), (300, 5, 5, 400), (512, 15, 5, 100),
                                         (1, 1, 1, 50), (65, 7, 8, 100), (1280, 5, 5, 30),
                                         (40, 70, 3, 40), (300, 6, 2, 100), (130, 4, 6, 100),
                                         # more than 8 B words: the row-by-row kernel
                                         (300, 5, 10, 100), (100, 4, 21, 50), (512, 16, 9, 30)])
def test_neg_update_bf16(gpu, oracle, hot, vexp, d, nwa, nwb, G):
    torch, CUMACH = gpu
    rng = np.random.default_rng(d * 5 + nwa)
    V = 20000
    A, B = tables16(rng, V, d, 0.5 / d ** 0.25)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    seed = 0x7654321 + d
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.025, vexp, seed, hot)
    Ad, Bd = dev16(torch, A), dev16(torch, B)
    err = CUMACH.word2vecNegBf16(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB), Ad, Bd, 0.025,
                                 vexp, seed)
    assert err == 0
    assert_same_roundings(host16(Ad), Ao, A, "A")
    assert_same_roundings(host16(Bd), Bo, B, "B")
    assert (Ao != A).any() and (Bo != B).any()


def test_neg_bf16_skips_pairs_with_a_dropped_word(gpu, oracle, hot):
    """Ids below zero in WA / WB skip their pairs (update and forward sum): the touched columns
    equal the oracle's, every other column keeps its bits."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(77)
    d, V, G, nwa, nwb = 300, 20000, 300, 6, 5
    A, B = tables16(rng, V, d, 0.5 / d ** 0.25)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    WA[rng.random(WA.shape[0]) < 0.2] = -1
    WB[rng.random(WB.shape[0]) < 0.2] = -1
    WA[:nwa] = -1
    WB[nwb:2 * nwb] = -1
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.025, 0.5, 21, hot)
    Ad, Bd = dev16(torch, A), dev16(torch, B)
    assert CUMACH.word2vecNegBf16(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB), Ad, Bd, 0.025,
                                  0.5, 21) == 0
    assert_same_roundings(host16(Ad), Ao, A, "A")
    assert_same_roundings(host16(Bd), Bo, B, "B")
    keep_a = (Ao == A).all(axis=1)
    keep_b = (Bo == B).all(axis=1)
    assert keep_a.sum() > V - G * nwa and keep_b.sum() > V - G * nwb
    assert (host16(Ad)[keep_a] == A[keep_a]).all() and (host16(Bd)[keep_b] == B[keep_b]).all()
    want = oracle.word2vecEvalNegBf16(d, G, nwa, nwb, WA, WB, A, B)
    ret = torch.zeros(1, dtype=torch.float64, device="cuda")
    assert CUMACH.word2vecEvalNegBf16(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB),
                                      dev16(torch, A), dev16(torch, B), ret) == 0
    assert float(ret.item()) == pytest.approx(want, rel=EVAL_RTOL)


def test_updates_within_1e_4_of_the_fp32_oracle_at_initial_scale(gpu, oracle):
    # tables as the reference starts them (Word2Vec.scala:112-117) plus a first update's worth
    # in the zero table; below 2**-6 one bfloat16 step is at most 6.1e-5, i.e. under 1e-4
    torch, CUMACH = gpu
    d, V, skip, lr = 300, 5000, 5, 0.015
    rng = np.random.default_rng(5)
    B32, _ = corpus.init_tables(V, d, 42)
    A32 = (rng.standard_normal((V, d)) * 0.002).astype(np.float32)
    A, B = cpumach.bf16_truncate(A32), cpumach.bf16_truncate(B32)
    Aw, Bw = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    W, LB, UB = corpus.collision_free_pos(400, skip, V, rng)
    oracle.word2vecPos(d, W.shape[0], skip, W, LB, UB, Aw, Bw, lr, 0.5, 1)
    assert max(np.abs(Aw).max(), np.abs(Bw).max()) < 2.0 ** -6
    Ad, Bd = dev16(torch, A), dev16(torch, B)
    assert CUMACH.word2vecPosBf16(d, W.shape[0], skip, dev(torch, W), dev(torch, LB),
                                  dev(torch, UB), Ad, Bd, lr, 0.5, 77) == 0
    assert np.abs(cpumach.bf16_widen(host16(Ad)) - Aw).max() <= UPDATE_ATOL
    assert np.abs(cpumach.bf16_widen(host16(Bd)) - Bw).max() <= UPDATE_ATOL
    assert np.abs(Aw - cpumach.bf16_widen(A)).max() > 10 * UPDATE_ATOL

    WA, WB = corpus.collision_free_neg(400, 5, 5, V, rng)
    Aw, Bw = cpumach.bf16_widen(A).copy(), cpumach.bf16_widen(B).copy()
    oracle.word2vecNeg(d, 400, 5, 5, WA, WB, Aw, Bw, lr, 0.5, 1)
    assert max(np.abs(Aw).max(), np.abs(Bw).max()) < 2.0 ** -6
    Ad, Bd = dev16(torch, A), dev16(torch, B)
    assert CUMACH.word2vecNegBf16(d, 400, 5, 5, dev(torch, WA), dev(torch, WB), Ad, Bd, lr, 0.5,
                                  78) == 0
    assert np.abs(cpumach.bf16_widen(host16(Ad)) - Aw).max() <= UPDATE_ATOL
    assert np.abs(cpumach.bf16_widen(host16(Bd)) - Bw).max() <= UPDATE_ATOL
    assert np.abs(Aw - cpumach.bf16_widen(A)).max() > 10 * UPDATE_ATOL


def test_unaligned_tables_take_the_halfword_path(gpu, oracle, hot):
    # an even d with a table that starts on an odd halfword: columns are 2-byte aligned only
    torch, CUMACH = gpu
    d, V, G, nwa, nwb = 64, 3000, 100, 5, 5
    rng = np.random.default_rng(9)
    A, B = tables16(rng, V, d, 0.2)
    WA, WB = corpus.collision_free_neg(G, nwa, nwb, V, rng)
    Ao, Bo = A.copy(), B.copy()
    oracle.word2vecNegBf16(d, G, nwa, nwb, WA, WB, Ao, Bo, 0.025, 0.0, 3, hot)
    buf_a = torch.zeros(V * d + 1, dtype=torch.int16, device="cuda")
    buf_b = torch.zeros(V * d + 1, dtype=torch.int16, device="cuda")
    Ad, Bd = buf_a[1:], buf_b[1:]
    Ad.copy_(dev16(torch, A).reshape(-1))
    Bd.copy_(dev16(torch, B).reshape(-1))
    assert Ad.data_ptr() % 4 == 2
    assert CUMACH.word2vecNegBf16(d, G, nwa, nwb, dev(torch, WA), dev(torch, WB), Ad, Bd, 0.025,
                                  0.0, 3) == 0
    assert_same_roundings(host16(Ad).reshape(V, d), Ao, A, "A")
    assert_same_roundings(host16(Bd).reshape(V, d), Bo, B, "B")
    assert int(buf_a[0].item()) == 0 and int(buf_b[0].item()) == 0


def test_column_offsets_beyond_2_to_31_elements_bf16(gpu, oracle):
    """Tables of 7.3 M x 300 bfloat16: every column used starts beyond element 2^31 (byte 2^32).
    With vexp = 0 neither the arithmetic nor the rounding keys depend on the id values, so the
    oracle runs on a compact copy of the touched columns with the ids renumbered (and told that
    none of them is a frequent word, as none of the large ids is)."""
    torch, CUMACH = gpu
    rng = np.random.default_rng(92)
    d, V, skip, nwa, nwb = 300, 7_300_000, 5, 5, 5
    first = (1 << 31) // d + 1
    n_ids = 4000
    big = (first + rng.permutation(V - first)[:n_ids]).astype(np.int64)
    assert (big * d > (1 << 31)).all()
    Ac, Bc = tables16(rng, n_ids, d, 0.1)
    A = torch.zeros((V, d), dtype=torch.int16, device="cuda")
    B = torch.zeros((V, d), dtype=torch.int16, device="cuda")
    idx = torch.from_numpy(big).cuda()
    A[idx] = dev16(torch, Ac)
    B[idx] = dev16(torch, Bc)
    Wc, LB, UB = corpus.collision_free_pos(100, skip, 1100, np.random.default_rng(1))
    WAc, WBc = corpus.collision_free_neg(200, nwa, nwb, 2000, np.random.default_rng(2))
    WAc, WBc = WAc + 1100, WBc + 1100
    Ao, Bo = Ac.copy(), Bc.copy()
    oracle.word2vecPosBf16(d, Wc.shape[0], skip, Wc, LB, UB, Ao, Bo, 0.025, 0.0, 41, 0)
    oracle.word2vecNegBf16(d, 200, nwa, nwb, WAc, WBc, Ao, Bo, 0.005, 0.0, 42, 0)
    tobig = big.astype(np.int32)
    assert CUMACH.word2vecPosBf16(d, Wc.shape[0], skip, dev(torch, tobig[Wc]), dev(torch, LB),
                                  dev(torch, UB), A, B, 0.025, 0.0, 41) == 0
    assert CUMACH.word2vecNegBf16(d, 200, nwa, nwb, dev(torch, tobig[WAc]),
                                  dev(torch, tobig[WBc]), A, B, 0.005, 0.0, 42) == 0
    assert_same_roundings(host16(A[idx]), Ao, Ac, "A")
    assert_same_roundings(host16(B[idx]), Bo, Bc, "B")
    assert (Ao != Ac).any() and (Bo != Bc).any()
    ret = torch.zeros(1, dtype=torch.float64, device="cuda")
    assert CUMACH.word2vecEvalPosBf16(d, Wc.shape[0], skip, dev(torch, tobig[Wc]),
                                      dev(torch, LB), dev(torch, UB), A, B, ret) == 0
    Ag, Bg = host16(A[idx]), host16(B[idx])
    want = oracle.word2vecEvalPosBf16(d, Wc.shape[0], skip, Wc, LB, UB,
                                      np.ascontiguousarray(Ag), np.ascontiguousarray(Bg))
    assert float(ret.item()) == pytest.approx(want, rel=EVAL_RTOL)
    # nothing else was touched
    A[idx] = 0
    B[idx] = 0
    assert int(A.abs().max().item()) == 0 and int(B.abs().max().item()) == 0


def test_table_conversions_match_torch(gpu):
    torch, _ = gpu
    from bidmach_amd.cumach import bf16_to_f32, f32_to_bf16
    g = torch.Generator(device="cpu").manual_seed(1)
    x = torch.randn(100003, generator=g) * 3.0
    x[:4] = torch.tensor([0.0, -0.0, float("inf"), 1.0])
    xd = x.cuda()
    h = torch.zeros(x.numel(), dtype=torch.int16, device="cuda")
    f32_to_bf16(x.numel(), xd, h)
    want = x.to(torch.bfloat16)                      # round to nearest, ties to even
    assert torch.equal(h.cpu(), want.view(torch.int16))
    back = torch.zeros(x.numel(), dtype=torch.float32, device="cuda")
    bf16_to_f32(x.numel(), h, back)
    assert torch.equal(back.cpu(), want.to(torch.float32))


def test_empty_and_rejected_arguments_bf16(gpu):
    torch, CUMACH = gpu
    t = torch.zeros(64, dtype=torch.int16, device="cuda")
    i = torch.zeros(8, dtype=torch.int32, device="cuda")
    r = torch.zeros(1, dtype=torch.float64, device="cuda")
    assert CUMACH.word2vecPosBf16(8, 0, 5, i, i, i, t, t, 0.1, 0.0, 1) == 0
    assert CUMACH.word2vecNegBf16(8, 0, 2, 2, i, i, t, t, 0.1, 0.0, 1) == 0
    assert CUMACH.word2vecNegBf16(8, 1, 0, 2, i, i, t, t, 0.1, 0.0, 1) == 0
    assert CUMACH.word2vecPosBf16(0, 1, 5, i, i, i, t, t, 0.1, 0.0, 1) == 1
    assert CUMACH.word2vecPosBf16(1281, 1, 5, i, i, i, t, t, 0.1, 0.0, 1) == 1
    assert CUMACH.word2vecPosBf16(8, 1, 5, None, i, i, t, t, 0.1, 0.0, 1) == 1
    assert CUMACH.word2vecNegBf16(8, 1, 2, 65, i, i, t, t, 0.1, 0.0, 1) == 1
    assert CUMACH.word2vecNegBf16(8, 1, 17, 9, i, i, t, t, 0.1, 0.0, 1) == 1   # no wide instance
    from bidmach_amd.cumach import load_library
    assert load_library().w2v_set_bf16_hot_words(-1) == 1
    assert load_library().w2v_set_bf16_hot_words(4097) == 1
    assert load_library().w2v_get_bf16_hot_words() == 1024
    assert CUMACH.word2vecEvalPosBf16(8, 1, 5, i, i, i, t, t, None) == 1
    assert CUMACH.word2vecEvalNegBf16(8, 1, 2, 2, i, i, t, None, r) == 1
    assert (t == 0).all()


# ---------------------------------------------------------------------------------------------
# Training on colliding minibatches: the order in which concurrent updates land is not fixed, so
# the check is the held-out loss next to the fp32 operators' (the sequential bf16 oracle reaches
# 1.35746 on this stream, the sequential fp32 oracle 1.35746 as well).
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("hot_words,zipf", [(1024, 1.0), (0, 1.0), (1024, 1.1)])
def test_heldout_loss_next_to_the_fp32_operators(hot_words, zipf):
    """Zipf(1.0) is the stream of the plumbing configuration, Zipf(1.1) that of the
    reduced-precision configuration; both behind the reference caller's default subsampling
    (the raw stream, which the ordered kernels take, is in tests/test_gpu_training.py)."""
    import torch
    from bidmach_amd.cumach import CUMACH, check, f32_to_bf16
    V, D, N, SKIP, NNEG, NREUSE, NMB, LR0 = 10000, 100, 100000, 5, 5, 5, 30, 0.025
    zc = corpus.zipf_cdf(V, zipf)
    nc = corpus.unigram_pow_cdf(V, zipf, 0.75)

    def minibatch(i):
        W = corpus.zipf_stream(N, V, zipf, seed=1234 + i, cdf=zc)
        rng = np.random.Generator(np.random.PCG64(99 + i))
        W = corpus.subsample(W, V, 1.0e-4, rng)
        LB, UB = corpus.window_bounds(N, SKIP, rng)
        WA, WB, G = corpus.negative_groups(W, LB, UB, NNEG, NREUSE, rng, neg_cdf=nc)
        return [torch.from_numpy(x).cuda() for x in (W, LB, UB, WA, WB)] + [G]

    stream = [minibatch(i) for i in range(NMB + 1)]
    from bidmach_amd.cumach import load_library
    assert load_library().w2v_set_bf16_hot_words(hot_words) == 0
    Bh, Ah = corpus.init_tables(V, D, 42)
    A32, B32 = torch.from_numpy(Ah).cuda(), torch.from_numpy(Bh).cuda()
    A16 = torch.zeros(V * D, dtype=torch.int16, device="cuda")
    B16 = torch.zeros(V * D, dtype=torch.int16, device="cuda")
    f32_to_bf16(V * D, A32, A16)
    f32_to_bf16(V * D, B32, B16)
    for i in range(NMB):
        W, LB, UB, WA, WB, G = stream[i]
        lr = max(LR0 * (1.0 - i / NMB), LR0 * 1e-4)
        check(CUMACH.word2vecPos(D, N, SKIP, W, LB, UB, A32, B32, lr, 0.0), "pos")
        check(CUMACH.word2vecNeg(D, G, NNEG, NREUSE, WA, WB, A32, B32, lr / NNEG, 0.0), "neg")
        check(CUMACH.word2vecPosBf16(D, N, SKIP, W, LB, UB, A16, B16, lr, 0.0, 2 * i), "pos16")
        check(CUMACH.word2vecNegBf16(D, G, NNEG, NREUSE, WA, WB, A16, B16, lr / NNEG, 0.0,
                                     2 * i + 1), "neg16")
    W, LB, UB, WA, WB, G = stream[NMB]
    r = torch.zeros(4, dtype=torch.float64, device="cuda")
    check(CUMACH.word2vecEvalPosF64(D, N, SKIP, W, LB, UB, A32, B32, r[0:1]), "epos")
    check(CUMACH.word2vecEvalNegF64(D, G, NNEG, NREUSE, WA, WB, A32, B32, r[1:2]), "eneg")
    check(CUMACH.word2vecEvalPosBf16(D, N, SKIP, W, LB, UB, A16, B16, r[2:3]), "epos16")
    check(CUMACH.word2vecEvalNegBf16(D, G, NNEG, NREUSE, WA, WB, A16, B16, r[3:4]), "eneg16")
    r = r.cpu().numpy()
    load_library().w2v_set_bf16_hot_words(1024)
    loss32 = -(r[0] + r[1] / NNEG) / (G * NREUSE)
    loss16 = -(r[2] + r[3] / NNEG) / (G * NREUSE)
    print("\nZipf(%.1f): held-out loss after %d minibatches: fp32 tables %.5f, bf16 tables (%d "
          "frequent words through side buffers) %.5f (%+.2f%%)"
          % (zipf, NMB, loss32, hot_words, loss16, 100.0 * (loss16 / loss32 - 1.0)))
    assert np.isfinite(loss16)
    assert loss16 < 1.386                        # better than the untrained model
    assert abs(loss16 - loss32) <= 0.005 * loss32
