"""The Word2Vec mirror's dobatch / evalbatch / train on the GPU against the same minibatch step
done with the CPU oracle on identical index arrays (needs an MI355X)."""
import math

import numpy as np
import pytest

from bidmach_amd import corpus
from bidmach_amd.word2vec import Options, Word2Vec

pytestmark = pytest.mark.gpu


def make_stream(n, vocab, seed=3):
    rng = np.random.default_rng(seed)
    w = corpus.zipf_stream(n, vocab, 1.0, seed=seed)
    w[rng.random(n) < 0.01] = vocab + 1
    sent = np.cumsum(rng.random(n) < 0.04).astype(np.int32)
    return np.stack([w, sent]).astype(np.int32)


def test_dobatch_and_evalbatch_match_cpu_twin(oracle):
    import torch
    assert torch.cuda.is_available()
    o = dict(vocabSize=4000, dim=64, batchSize=8000, lrate=0.005, vexp=0.5, texp=0.5, seed=11,
             deviceWordMats=False)     # host-built index arrays, so the CPU twin sees the same ones
    gpu = Word2Vec(Options(**o), device="cuda:0")
    twin = Word2Vec(Options(**o), device="cpu")     # same seed: same init, same wordMats draws
    gpu.init()
    twin.init()
    m0 = twin.modelmats[0].numpy()
    m1 = twin.modelmats[1].numpy()
    stream = make_stream(8000 * 4, 4000)
    bs, nneg, nreuse, nskip = 8000, 5, 5, 5
    first = None
    for k in range(3):
        mats = stream[:, k * bs:(k + 1) * bs]
        pos = (k + 1) * bs
        gpu.dobatch(mats, 0, pos)
        first = first or pos
        lr = 0.005 * math.pow(pos / first, -0.5)
        words, lb, ub, negs, ctx = twin.wordMats(mats)
        oracle.word2vecPos(64, bs, nskip, words, lb, ub, m1, m0, lr, 0.5, 1)
        oracle.word2vecNeg(64, ctx.shape[0] // nreuse, nneg, nreuse, negs, ctx, m1, m0,
                           lr / nneg, 0.5, 1)
    mats = stream[:, 3 * bs:4 * bs]
    got = gpu.evalbatch(mats, 0, 4 * bs)
    words, lb, ub, negs, ctx = twin.wordMats(mats)
    epos = oracle.word2vecEvalPos(64, bs, nskip, words, lb, ub, m1, m0, 4)
    eneg = oracle.word2vecEvalNeg(64, ctx.shape[0] // nreuse, nneg, nreuse, negs, ctx, m1, m0, 4)
    want = (epos + eneg / nneg) / ctx.shape[0]
    print("\nevalbatch: gpu %.6f cpu twin %.6f" % (got, want))
    assert want < -0.1
    assert got == pytest.approx(want, rel=2e-3)
    # the tables themselves: Hogwild order differs, so compare loosely but element-wise
    g0 = gpu.modelmats[0].cpu().numpy()
    g1 = gpu.modelmats[1].cpu().numpy()
    assert np.abs(g0 - m0).max() < 0.05 * max(1.0, np.abs(m0).max())
    assert np.abs(g1 - m1).max() < 0.05 * max(1.0, np.abs(m1).max())


def test_train_loop_scores_held_out_minibatches():
    o = Options(vocabSize=3000, dim=32, batchSize=4000, lrate=0.05, evalStep=3, seed=5)
    m = Word2Vec(o)
    stream = make_stream(4000 * 9, 3000, seed=8)
    res = m.train(stream, npasses=2)
    # minibatches 1, 4, 7 and the last (8) of each pass are scored, not trained on
    assert len(res) == 8
    assert [r[0] for r in res[:4]] == [2 * 4000, 5 * 4000, 8 * 4000, 9 * 4000]
    scores = [r[1] for r in res]
    assert all(np.isfinite(s) and s < 0 for s in scores)
    assert scores[-1] > scores[0]            # the log-likelihood per context word went up


def test_device_wordmats_path_matches_oracle_step(oracle):
    """dobatch with index arrays built on the device: the arrays are read back and the same step
    is replayed with the CPU oracle."""
    o = Options(vocabSize=4000, dim=64, batchSize=6000, lrate=0.005, vexp=0.5, seed=3)
    m = Word2Vec(o)
    m.init()
    m0 = m.modelmats[0].cpu().numpy().copy()
    m1 = m.modelmats[1].cpu().numpy().copy()
    mats = make_stream(6000, 4000, seed=21)
    m.dobatch(mats, 0, 6000)
    b = m._wm
    npairs, G = b["counts"].cpu().tolist()
    words, lb, ub = (b[k].cpu().numpy() for k in ("words", "lb", "ub"))
    negs = b["negs"].cpu().numpy()[:G * o.nneg].copy()
    ctx = b["ctx"].cpu().numpy()[:G * o.nreuse].copy()
    assert G > 100 and npairs // o.nreuse == G
    oracle.word2vecPos(64, 6000, o.nskip, words, lb, ub, m1, m0, 0.005, 0.5, 1)
    oracle.word2vecNeg(64, G, o.nneg, o.nreuse, negs, ctx, m1, m0, 0.005 / o.nneg, 0.5, 1)
    assert np.abs(m.modelmats[0].cpu().numpy() - m0).max() < 2e-3
    assert np.abs(m.modelmats[1].cpu().numpy() - m1).max() < 2e-3


def test_odd_sized_minibatch_is_skipped():
    import torch
    o = Options(vocabSize=500, dim=16, batchSize=1000, seed=1)
    m = Word2Vec(o)
    m.init()
    before = [x.clone() for x in m.modelmats]
    mats = make_stream(777, 500)
    m.dobatch(mats, 0, 1000)
    assert torch.equal(before[0], m.modelmats[0]) and torch.equal(before[1], m.modelmats[1])
    assert m.evalbatch(mats, 0, 1000) == 0.0
