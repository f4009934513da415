"""The two configurations whose full shapes the small parity cases do not reach, each under an
oracle check at its own size (needs an MI355X; about two minutes of host time).

  dim 512, window 10, 15 negatives, 500k-token minibatches, vocab 1M, Zipf(1.0) stream:
      four minibatches on the device (default settings) and on the oracle, (a) behind the
      reference caller's subsampling, where training works: held-out loss within 0.5 %, and the
      forward operators on the oracle-trained tables within 1e-5; (b) on the raw stream, where
      the ordered kernels run (with their 16-A-column instance) and where at lr 0.025 the oracle
      itself ends at seven times the untrained loss: the device must fail the same way, within
      the band the oracle's own runs span (two 16-thread runs against its 8-thread run) + 0.5 %.
  bfloat16 tables, vocab 3M, dim 300, 1M-token minibatch of a Zipf(1.1) stream:
      the forward operators against the bfloat16 oracle (1e-5) on tables that one full-size
      update call has gone over.  (That update call itself is checked against first-order sums,
      and the raw Zipf(1.1) loss against the bfloat16 oracle, in tests/test_gpu_bf16_full_size.py.)
"""
import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import cpumach

pytestmark = pytest.mark.gpu


def test_dim512_window10_neg15_full_shape(oracle):
    import torch
    from bidmach_amd.cumach import CUMACH, check
    V, D, N, SKIP, NNEG, NREUSE, K, LR0 = 1_000_000, 512, 500_000, 10, 15, 5, 4, 0.025
    zc = corpus.zipf_cdf(V, 1.0)
    nc = corpus.unigram_pow_cdf(V, 1.0, 0.75)

    def mb(i, wsample):
        W = corpus.zipf_stream(N, V, 1.0, seed=1234 + i, cdf=zc)
        rng = np.random.Generator(np.random.PCG64(99 + i))
        if wsample > 0:
            W = corpus.subsample(W, V, wsample, rng)
        LB, UB = corpus.window_bounds(N, SKIP, rng)
        WA, WB, G = corpus.negative_groups(W, LB, UB, NNEG, NREUSE, rng, neg_cdf=nc)
        return W, LB, UB, WA, WB, G

    def lr(i):
        return max(LR0 * (1.0 - i / K), LR0 * 1e-4)

    def dev(x):
        return torch.from_numpy(x).cuda()

    for wsample in (1.0e-4, 0.0):
        mbs = [mb(i, wsample) for i in range(K + 1)]

        def heldout(A, B):
            W, LB, UB, WA, WB, G = mbs[K]
            epos = oracle.word2vecEvalPos(D, N, SKIP, W, LB, UB, A, B, 16)
            eneg = oracle.word2vecEvalNeg(D, G, NNEG, NREUSE, WA, WB, A, B, 16)
            return -(epos + eneg / NNEG) / (G * NREUSE), epos, eneg

        def cpu_train(nthreads):
            B, A = corpus.init_tables(V, D, 42)
            for i in range(K):
                W, LB, UB, WA, WB, G = mbs[i]
                oracle.word2vecPos(D, N, SKIP, W, LB, UB, A, B, lr(i), 0.0, nthreads)
                oracle.word2vecNeg(D, G, NNEG, NREUSE, WA, WB, A, B, lr(i) / NNEG, 0.0, nthreads)
            return A, B

        A, B = cpu_train(16)
        ref, epos, eneg = heldout(A, B)
        # forward operators at the full shape on the oracle-trained tables
        W, LB, UB, WA, WB, G = mbs[K]
        Ad, Bd = dev(A), dev(B)
        ret = torch.zeros(2, dtype=torch.float64, device="cuda")
        check(CUMACH.word2vecEvalPosF64(D, N, SKIP, dev(W), dev(LB), dev(UB), Ad, Bd, ret[0:1]),
              "epos")
        check(CUMACH.word2vecEvalNegF64(D, G, NNEG, NREUSE, dev(WA), dev(WB), Ad, Bd, ret[1:2]),
              "eneg")
        r = ret.cpu().numpy()
        assert r[0] == pytest.approx(epos, rel=1e-5)
        assert r[1] == pytest.approx(eneg, rel=1e-5)
        del Ad, Bd, A, B
        # training on the device, default settings
        Bh, Ah = corpus.init_tables(V, D, 42)
        Ad, Bd = dev(Ah), dev(Bh)
        for i in range(K):
            W, LB, UB, WA, WB, G = mbs[i]
            check(CUMACH.word2vecPos(D, N, SKIP, dev(W), dev(LB), dev(UB), Ad, Bd, lr(i), 0.0),
                  "pos")
            check(CUMACH.word2vecNeg(D, G, NNEG, NREUSE, dev(WA), dev(WB), Ad, Bd, lr(i) / NNEG,
                                     0.0), "neg")
        got = heldout(Ad.cpu().numpy(), Bd.cpu().numpy())[0]
        del Ad, Bd
        print("\ndim 512, window 10, 15 negatives, %s: held-out loss cpu(16 threads) %.5f, gpu, "
              "default settings %.5f (%+.2f%%)"
              % ("subsampled 1e-4" if wsample > 0 else "raw stream", ref, got,
                 100.0 * (got / ref - 1.0)))
        assert np.isfinite(got)
        if wsample > 0:
            assert ref < 1.5                       # four minibatches in: still near the start
            assert abs(got / ref - 1.0) <= 0.005, (got, ref)
        else:
            # This one does not train, on the CPU either (the loss ends far above the untrained
            # 1.386), and where it ends moves by several percent from one multi-threaded run of
            # the oracle to the next (16 threads: 9.98 to 10.41 seen).  The run with fewer threads
            # is the one nearer to the sequential order: the device is compared with an 8-thread
            # run, within what two 16-thread runs of the oracle itself use up, plus 0.5 %.
            assert ref > 5.0
            ref8 = heldout(*cpu_train(8))[0]
            ref16b = heldout(*cpu_train(16))[0]
            # (two runs can happen to agree: the spread is taken to be 1.5 % at least, the smallest
            # seen between an 8- and a 16-thread run here)
            band = max(abs(ref / ref8 - 1.0), abs(ref16b / ref8 - 1.0), 0.015) + 0.005
            print("raw stream: the oracle on 8 threads %.5f (16 threads %+.2f%% and %+.2f%%, gpu "
                  "%+.2f%%); band %.1f%%"
                  % (ref8, 100.0 * (ref / ref8 - 1.0), 100.0 * (ref16b / ref8 - 1.0),
                     100.0 * (got / ref8 - 1.0), 100.0 * band))
            assert band <= 0.10, band
            assert abs(got / ref8 - 1.0) <= band, (got, ref8, band)


def test_bf16_vocab3m_zipf11_full_shape(oracle):
    import torch
    from bidmach_amd.cumach import CUMACH, check, f32_to_bf16
    V, D, N, SKIP, NNEG, NREUSE = 3_000_000, 300, 1_000_000, 5, 5, 5
    zc = corpus.zipf_cdf(V, 1.1)
    nc = corpus.unigram_pow_cdf(V, 1.1, 0.75)
    W = corpus.zipf_stream(N, V, 1.1, seed=1234, cdf=zc)
    rng = np.random.Generator(np.random.PCG64(99))
    LB, UB = corpus.window_bounds(N, SKIP, rng)
    WA, WB, G = corpus.negative_groups(W, LB, UB, NNEG, NREUSE, rng, neg_cdf=nc)

    def dev(x):
        return torch.from_numpy(x).cuda()

    # tables: B random (the reference's start), A small random instead of zero, so that the
    # forward sums are not just log(1/2) per pair
    Bh, _ = corpus.init_tables(V, D, 42)
    A32 = dev(Bh.copy())
    A32 *= 40.0                                   # N(0, ~0.04) columns: |a.b| up to a few tenths
    B32 = dev(Bh)
    B32 *= 40.0
    A16 = torch.empty(V * D, dtype=torch.int16, device="cuda")
    B16 = torch.empty(V * D, dtype=torch.int16, device="cuda")
    f32_to_bf16(V * D, A32, A16)
    f32_to_bf16(V * D, B32, B16)
    del A32, B32
    dW, dLB, dUB, dWA, dWB = dev(W), dev(LB), dev(UB), dev(WA), dev(WB)
    # one full-size update call (raw stream: what bench.py times), tiny step: the tables stay
    # finite and every table column moves by at most a few bf16 steps
    before = A16.clone()
    check(CUMACH.word2vecPosBf16(D, N, SKIP, dW, dLB, dUB, A16, B16, 1e-4, 0.0, 5), "pos16")
    check(CUMACH.word2vecNegBf16(D, G, NNEG, NREUSE, dWA, dWB, A16, B16, 2e-5, 0.0, 6), "neg16")
    assert bool(torch.isfinite(A16.view(torch.bfloat16)).all())
    assert bool(torch.isfinite(B16.view(torch.bfloat16)).all())
    assert bool((A16 != before).any())
    del before
    # forward operators at the full shape against the bfloat16 oracle on the same (updated) tables
    ret = torch.zeros(2, dtype=torch.float64, device="cuda")
    check(CUMACH.word2vecEvalPosBf16(D, N, SKIP, dW, dLB, dUB, A16, B16, ret[0:1]), "epos16")
    check(CUMACH.word2vecEvalNegBf16(D, G, NNEG, NREUSE, dWA, dWB, A16, B16, ret[1:2]), "eneg16")
    r = ret.cpu().numpy()
    Ah = A16.cpu().numpy().view(np.uint16).reshape(V, D)
    Bh16 = B16.cpu().numpy().view(np.uint16).reshape(V, D)
    # the oracle's forward sums equal the fp32 oracle's on the widened tables bit for bit
    # (tests/test_oracle_bf16.py), which has threads
    Aw, Bw = cpumach.bf16_widen(Ah), cpumach.bf16_widen(Bh16)
    epos = oracle.word2vecEvalPos(D, N, SKIP, W, LB, UB, Aw, Bw, 16)
    eneg = oracle.word2vecEvalNeg(D, G, NNEG, NREUSE, WA, WB, Aw, Bw, 16)
    print("\nbf16, vocab 3M, Zipf(1.1), 1M tokens: forward sums gpu %.3f / %.3f, oracle %.3f / %.3f"
          % (r[0], r[1], epos, eneg))
    assert r[0] == pytest.approx(epos, rel=1e-5)
    assert r[1] == pytest.approx(eneg, rel=1e-5)
