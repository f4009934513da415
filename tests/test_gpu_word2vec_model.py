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
    b = m._wm_last
    npairs, G = b["counts"].cpu().tolist()
    words, lb, ub = (b[k].cpu().numpy() for k in ("words", "lb", "ub"))
    negs = b["negs"].cpu().numpy()[:G * o.nneg].copy()
    ctx = b["ctx"].cpu().numpy()[:G * o.nreuse].copy()
    assert G > 100 and npairs // o.nreuse == G
    oracle.word2vecPos(64, 6000, o.nskip, words, lb, ub, m1, m0, 0.005, 0.5, 1)
    oracle.word2vecNeg(64, G, o.nneg, o.nreuse, negs, ctx, m1, m0, 0.005 / o.nneg, 0.5, 1)
    assert np.abs(m.modelmats[0].cpu().numpy() - m0).max() < 2e-3
    assert np.abs(m.modelmats[1].cpu().numpy() - m1).max() < 2e-3


def test_back_to_back_minibatches_do_not_overwrite_index_arrays_in_use():
    """dobatch only enqueues the update kernels, and the next call builds its index arrays on
    another stream into the other buffer set: six different minibatches in a row, without waiting,
    must train the same model as six calls that wait for the device after each one.  The second
    table starts at zero and the step is tiny, so every update is, to first order, a sum that does
    not depend on the order of the updates; index arrays overwritten while a kernel still reads them
    would move whole contributions to other words."""
    import torch

    def run(wait):
        o = Options(vocabSize=50000, dim=64, batchSize=200000, lrate=1e-5, vexp=0.0, texp=0.0,
                    seed=9)
        m = Word2Vec(o)
        m.init()
        stream = make_stream(200000 * 6, 50000, seed=31)
        for k in range(6):
            m.dobatch(stream[:, k * 200000:(k + 1) * 200000], 0, (k + 1) * 200000)
            if wait:
                m.synchronize()
                torch.cuda.synchronize()
        m.synchronize()
        torch.cuda.synchronize()
        return [x.cpu().numpy().astype(np.float64) for x in m.modelmats]

    a0, a1 = run(False)
    b0, b1 = run(True)
    moved = np.abs(b1).max()                    # modelmats(1) starts at zero
    assert moved > 1e-6
    assert np.abs(a1 - b1).max() < 2e-2 * moved
    assert np.abs(a0 - b0).max() < 2e-2 * moved


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


@pytest.mark.parametrize("dual", [False, True])
def test_sliced_multipart_model_matches_oracle_step(oracle, dual):
    """A two-worker, several-part model (every part its own device allocation): dobatch and
    evalbatch go through the device Slice operators; the same step is replayed with the oracle's
    Slice functions on the index arrays read back from the device."""
    o = Options(vocabSize=4000, dim=64, batchSize=6000, lrate=0.005, vexp=0.5, seed=4,
                nSlices=2, iSlice=1, nHeadTerms=300, maxArraySize=64 * 700, doHead=1,
                dualMode=dual)
    m = Word2Vec(o)
    m.init()
    assert m.maxCols == 700 and m.nmmats == 4        # 300 + 1 + 3699 // 2 = 2150 columns
    assert len(m.modelmats) == 2 * (4 + (1 if dual else 0))
    assert [x.shape[0] for x in m.modelmats[-8::2]] == [700, 700, 700, 50]
    host = [x.cpu().numpy().copy() for x in m.modelmats]
    mats = make_stream(6000, 4000, seed=22)
    m.dobatch(mats, 0, 6000)
    b = m._wm_last
    npairs, G = b["counts"].cpu().tolist()
    words, lb, ub = (b[k].cpu().numpy() for k in ("words", "lb", "ub"))
    negs = b["negs"].cpu().numpy()[:G * o.nneg].copy()
    ctx = b["ctx"].cpu().numpy()[:G * o.nreuse].copy()
    sl = (1, 1, 2, 700, 300, dual)
    oracle.word2vecPosSlice(64, 6000, o.nskip, words, lb, ub, host, 0.005, 0.5, *sl, 1)
    oracle.word2vecNegSlice(64, G, o.nneg, o.nreuse, negs, ctx, host, 0.005 / o.nneg, 0.5, *sl, 1)
    moved = 0.0
    for g, h in zip(m.modelmats, host):
        assert np.abs(g.cpu().numpy() - h).max() < 2e-3
        moved = max(moved, float(np.abs(h).max()))
    if dual:      # the leading pair is not part of the sliced model
        assert np.array_equal(m.modelmats[1].cpu().numpy(), np.zeros_like(host[1]))
    held = make_stream(6000, 4000, seed=23)
    got = m.evalbatch(held, 0, 12000)
    b = m._wm_last
    npairs, G = b["counts"].cpu().tolist()
    words, lb, ub = (b[k].cpu().numpy() for k in ("words", "lb", "ub"))
    negs = b["negs"].cpu().numpy()[:G * o.nneg].copy()
    ctx = b["ctx"].cpu().numpy()[:G * o.nreuse].copy()
    host = [x.cpu().numpy().copy() for x in m.modelmats]
    epos = oracle.word2vecEvalPosSlice(64, 6000, o.nskip, words, lb, ub, host, 4, 1, 2, 700, 300,
                                       dual, floor=1e-40)
    eneg = oracle.word2vecEvalNegSlice(64, G, o.nneg, o.nreuse, negs, ctx, host, 4, 1, 2, 700, 300,
                                       dual, floor=1e-40)
    want = (epos + eneg / o.nneg) / ctx.shape[0]
    assert want < -0.05
    assert got == pytest.approx(want, rel=1e-5)


def test_train_from_word_file_then_checkpoint_round_trip(tmp_path):
    """The files either side of the path: a (word id, sentence id) .imat.lz4 input file feeds the
    training loop, the model is written in the checkpoint layout, and a fresh model loaded from it
    scores a held-out minibatch identically."""
    import os
    from bidmach_amd import matio
    words = str(tmp_path / "words.imat.lz4")
    matio.saveIMat(words, make_stream(4000 * 6, 3000, seed=31))
    o = Options(vocabSize=3000, dim=32, batchSize=4000, lrate=0.05, evalStep=100, seed=6)
    m = Word2Vec(o)
    res = m.train(matio.loadIMat(words), npasses=1)
    assert len(res) == 2 and all(np.isfinite(r[1]) for r in res)    # minibatch 1 and the last one
    prefix = str(tmp_path / "model") + os.sep
    m.save(prefix)
    m2 = Word2Vec(Options(dim=32, batchSize=4000))
    m2.load(prefix)
    m2.ncols = 4000
    for a, b in zip(m.modelmats, m2.modelmats):
        assert a.is_cuda and b.is_cuda and bool((a == b).all())
    held = make_stream(4000, 3000, seed=32)
    m.rng = np.random.Generator(np.random.PCG64(1))
    m2.rng = np.random.Generator(np.random.PCG64(1))
    m._call = m2._call = 1000
    s1 = m.evalbatch(held, 0, 4000)
    s2 = m2.evalbatch(held, 0, 4000)
    assert s1 < -0.1 and s1 == s2


def test_bf16_storage_trains_like_fp32_and_round_trips_through_a_checkpoint(tmp_path):
    """The same training loop on a bfloat16 model (no counterpart in the reference): scores
    follow the fp32 model's, and a checkpoint written from it (widened to fp32 files) loads back
    into an identical bf16 model."""
    import os
    import torch
    stream = make_stream(4000 * 9, 3000, seed=8)
    scores = {}
    models = {}
    for storage in ("fp32", "bf16"):
        o = Options(vocabSize=3000, dim=32, batchSize=4000, lrate=0.05, evalStep=3, seed=5,
                    storage=storage)
        m = Word2Vec(o)
        res = m.train(stream, npasses=2)
        assert len(res) == 8
        scores[storage] = [r[1] for r in res]
        models[storage] = m
    assert models["bf16"].modelmats[0].dtype == torch.bfloat16
    assert all(np.isfinite(s) and s < 0 for s in scores["bf16"])
    assert scores["bf16"][-1] > scores["bf16"][0]
    # both runs see the same minibatches; the scores differ by rounding noise only
    for a, b in zip(scores["fp32"], scores["bf16"]):
        assert b == pytest.approx(a, rel=0.01)
    m = models["bf16"]
    prefix = str(tmp_path / "model16") + os.sep
    m.save(prefix)
    m2 = Word2Vec(Options(dim=32, batchSize=4000))
    m2.load(prefix)
    assert m2.opts.storage == "bf16"
    for a, b in zip(m.modelmats, m2.modelmats):
        assert b.dtype == torch.bfloat16 and bool((a.view(torch.int16) == b.view(torch.int16)).all())
    with pytest.raises(ValueError):
        Word2Vec(Options(vocabSize=3000, dim=32, nSlices=2, storage="bf16")).init(4000)
