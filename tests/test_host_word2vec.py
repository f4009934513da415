"""Host logic of the Word2Vec mirror: the arrays wordMats hands to the operators keep the
reference's contract (Word2Vec.scala:214-364).  The reference has no test or fixture for this
preprocessing and its random stream comes from BIDMat, which is not in its tree, so the draws
themselves are parity-unpinned; what is pinned here is the output contract and the distributions.
"""
import math

import numpy as np
import pytest

from bidmach_amd import corpus
from bidmach_amd.word2vec import Options, Word2Vec


def model(**kw):
    m = Word2Vec(Options(**kw), device="cpu")
    m.expt = 1.0 / (1.0 - m.opts.wexpt)
    m.salpha = m.opts.wsample * math.log(m.opts.vocabSize)
    return m


def stream(n, vocab, seed=3, sentence_p=0.05, oov_p=0.02):
    rng = np.random.default_rng(seed)
    w = corpus.zipf_stream(n, vocab, 1.0, seed=seed)
    w[rng.random(n) < oov_p] = vocab + 5          # out-of-vocabulary ids
    sent = np.cumsum(rng.random(n) < sentence_p).astype(np.int32)
    return np.stack([w, sent]).astype(np.int32)


def test_defaults_are_the_reference_defaults():
    o = Options()
    assert (o.nskip, o.nneg, o.nreuse, o.vocabSize) == (5, 5, 5, 100000)
    assert (o.wexpt, o.wsample, o.headlen) == (0.75, 1e-4, 10000)
    assert (o.dim, o.lrate, o.texp, o.vexp, o.evalStep) == (256, 1.0, 0.5, 0.5, 11)
    with pytest.raises(AttributeError):
        Options(nosuchoption=1)


@pytest.mark.parametrize("nskip,nneg,nreuse", [(5, 5, 5), (10, 15, 5), (2, 3, 4)])
def test_wordmats_contract(nskip, nneg, nreuse):
    V, n = 5000, 20000
    m = model(vocabSize=V, nskip=nskip, nneg=nneg, nreuse=nreuse, wsample=1e-3)
    mats = stream(n, V)
    words, lb, ub, negs, ctx = m.wordMats(mats)
    assert words.dtype == lb.dtype == ub.dtype == negs.dtype == ctx.dtype == np.int32
    assert words.shape == lb.shape == ub.shape == (n,)
    # -1 marks dropped / OOV words; kept words are unchanged
    kept = words >= 0
    assert np.all(words[~kept] == -1)
    assert np.array_equal(words[kept], mats[0][kept])
    assert not np.any(kept & (mats[0] >= V))
    # window bounds: lb <= 0 <= ub, |.| <= nskip, never across a sentence boundary or the edges
    assert np.all(lb <= 0) and np.all(ub >= 0)
    assert np.all(-lb <= nskip) and np.all(ub <= nskip)
    idx = np.arange(n)
    assert np.all(idx + lb >= 0) and np.all(idx + ub < n)
    assert np.all(mats[1][idx + lb] == mats[1]) and np.all(mats[1][idx + ub] == mats[1])
    # groups: G = floor(#valid pairs / nreuse); contexts are the valid pairs' context words
    npairs, _ = corpus.count_pairs(words, lb, ub)
    G = npairs // nreuse
    assert ctx.shape == (G * nreuse,) and negs.shape == (G * nneg,)
    allctx = corpus.valid_context_words(words, lb, ub)
    assert np.all(ctx >= 0)
    have = np.bincount(ctx, minlength=V)
    avail = np.bincount(allctx, minlength=V)
    assert np.all(have <= avail)                       # a sub-multiset (the remainder is dropped)
    assert avail.sum() - have.sum() == npairs - G * nreuse
    assert np.all(negs >= 0) and np.all(negs < V)


def test_subsampling_keep_probability():
    """keep probability min(1, sqrt(x) + x), x = (id+1) * wsample * ln V (Word2Vec.scala:150,221-225)."""
    V, n = 1000, 400000
    m = model(vocabSize=V, wsample=1e-3)
    ids = np.zeros(n, np.int32)
    ids[n // 2:] = 200
    mats = np.stack([ids, np.zeros(n, np.int32)])
    words, *_ = m.wordMats(mats)
    for wid, sl in ((0, slice(0, n // 2)), (200, slice(n // 2, n))):
        x = (wid + 1) * 1e-3 * math.log(V)
        want = min(1.0, math.sqrt(x) + x)
        got = float((words[sl] >= 0).mean())
        assert got == pytest.approx(want, abs=4e-3)


def test_window_width_distribution():
    """ub = min(nskip, floor(u*nskip) + 1): uniform on 1..nskip away from boundaries."""
    V, n, nskip = 100, 200000, 5
    m = model(vocabSize=V, nskip=nskip, wsample=1.0)
    mats = np.stack([np.zeros(n, np.int32), np.zeros(n, np.int32)])
    _, lb, ub, *_ = m.wordMats(mats)
    inner = slice(nskip, n - nskip)
    assert np.array_equal(lb[inner], -ub[inner])
    freq = np.bincount(ub[inner], minlength=nskip + 1)[1:] / (n - 2 * nskip)
    assert np.allclose(freq, 1.0 / nskip, atol=5e-3)


def test_negative_sampler_is_the_closed_form_power_law():
    """min(V-1, floor(V * u**4)) for wexpt = 0.75: P(id < k) = (k/V)**0.25."""
    V, n = 10000, 300000
    m = model(vocabSize=V, wsample=1.0, nneg=5, nreuse=5)
    mats = np.stack([corpus.zipf_stream(n, V, 1.0, seed=1), np.zeros(n, np.int32)]).astype(np.int32)
    *_, negs, _ = m.wordMats(mats)
    for k in (10, 100, 1000, 5000):
        assert float((negs < k).mean()) == pytest.approx((k / V) ** 0.25, abs=5e-3)


def test_iflip_swaps_rows():
    V, n = 500, 2000
    mats = stream(n, V)
    a = model(vocabSize=V, wsample=1.0, seed=4).wordMats(mats)
    b = model(vocabSize=V, wsample=1.0, seed=4, iflip=True).wordMats(mats[::-1])
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


def test_sliced_model_list_has_the_reference_shape():
    """Word2Vec.scala:100-131: columns on this worker, number of parts, dual-mode list."""
    from bidmach_amd.word2vec import Options, Word2Vec
    o = Options(vocabSize=1000, dim=8, nSlices=3, iSlice=2, nHeadTerms=100, maxArraySize=8 * 150)
    m = Word2Vec(o, device="cpu")
    m.init()
    actual = 100 + 1 + (1000 - 100 - 1) // 3
    assert actual == 400 and m.maxCols == 150 and m.nmmats == 3 and m._sliced()
    assert [tuple(x.shape) for x in m.modelmats] == [(150, 8)] * 4 + [(100, 8)] * 2
    assert all(float(x.abs().max()) == 0.0 for x in m.modelmats[1::2])       # A tables start at 0
    assert all(0 < float(x.abs().max()) <= 0.5 / 8 for x in m.modelmats[0::2])
    o.dualMode = True
    m = Word2Vec(o, device="cpu")
    m.init()
    assert len(m.modelmats) == 8 and m._dual
    assert (m.modelmats[0] == m.modelmats[2]).all() and (m.modelmats[1] == m.modelmats[3]).all()
    plain = Word2Vec(Options(vocabSize=1000, dim=8), device="cpu")
    plain.init()
    assert not plain._sliced() and [tuple(x.shape) for x in plain.modelmats] == [(1000, 8)] * 2
