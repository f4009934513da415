"""Synthetic corpora and minibatch index arrays for the SGNS operators (host side, numpy).

Produces exactly the arrays the reference's Word2Vec.wordMats hands to the native calls
(src/main/scala/BIDMach/networks/Word2Vec.scala:214-364): W, LB, UB (int32[N]) for the positive
pass and WA (nneg x G), WB (nreuse x G), both group-contiguous int32, for the negative pass.
Word ids are frequency ranks (0 = most frequent); -1 marks a dropped or out-of-vocabulary token.

The random streams are numpy's (PCG64), not BIDMat's, so only the output contract and the
distributions match the reference, not its draws.
"""
import numpy as np


def zipf_cdf(vocab, s=1.0):
    """Cumulative distribution of p(rank r) ~ 1 / r**s over ranks 1..vocab (float64)."""
    p = 1.0 / np.arange(1, vocab + 1, dtype=np.float64) ** s
    c = np.cumsum(p)
    c /= c[-1]
    return c


def zipf_stream(n, vocab, s=1.0, seed=1234, cdf=None):
    """n word ids drawn i.i.d. from Zipf(s) by inverse CDF; id = rank - 1."""
    if cdf is None:
        cdf = zipf_cdf(vocab, s)
    rng = np.random.Generator(np.random.PCG64(seed))
    u = rng.random(n)
    ids = np.searchsorted(cdf, u, side="left")
    return np.minimum(ids, vocab - 1).astype(np.int32)


def unigram_pow_cdf(vocab, s=1.0, power=0.75):
    """CDF of the negative-sampling distribution unigram**power for a Zipf(s) vocabulary."""
    p = (1.0 / np.arange(1, vocab + 1, dtype=np.float64) ** s) ** power
    c = np.cumsum(p)
    c /= c[-1]
    return c


def sample_from_cdf(n, cdf, rng):
    ids = np.searchsorted(cdf, rng.random(n), side="left")
    return np.minimum(ids, cdf.shape[0] - 1).astype(np.int32)


def closed_form_negatives(n, vocab, wexpt, rng):
    """The reference's own sampler: min(V-1, floor(V * u**(1/(1-wexpt)))) (Word2Vec.scala:139,353)."""
    expt = 1.0 / (1.0 - wexpt)
    ids = np.floor(vocab * rng.random(n) ** expt).astype(np.int64)
    return np.minimum(ids, vocab - 1).astype(np.int32)


def window_bounds(n, nskip, rng, sentence=None):
    """ub = min(nskip, floor(u*nskip)+1), lb = -ub (Word2Vec.scala:228-230), then clipped so a
    window never crosses a sentence boundary (:233-237).  With sentence=None the whole minibatch
    is one sentence, i.e. windows are clipped at the minibatch edges."""
    ub = np.minimum(nskip, np.floor(rng.random(n) * nskip).astype(np.int32) + 1).astype(np.int32)
    lb = -ub
    idx = np.arange(n, dtype=np.int64)
    if sentence is None:
        first = np.zeros(n, dtype=np.int64)
        last = np.full(n, n - 1, dtype=np.int64)
    else:
        sentence = np.asarray(sentence)
        change = np.flatnonzero(sentence[1:] != sentence[:-1]) + 1
        starts = np.concatenate(([0], change))
        ends = np.concatenate((change, [n])) - 1
        seg = np.searchsorted(starts, idx, side="right") - 1
        first = starts[seg]
        last = ends[seg]
    lb = np.maximum(lb, (first - idx)).astype(np.int32)
    ub = np.minimum(ub, (last - idx)).astype(np.int32)
    return lb, ub


def subsample(words, vocab, wsample, rng):
    """Frequent-word subsampling: keep with probability min(1, sqrt(x) + x),
    x = (id+1) * wsample * ln(vocab); dropped and out-of-vocabulary words become -1
    (Word2Vec.scala:150,218-225)."""
    words = np.asarray(words, dtype=np.int32)
    good = words < vocab
    x = (words.astype(np.float32) + 1.0) * np.float32(wsample * np.log(vocab))
    keep = rng.random(words.shape[0]).astype(np.float32) < (np.sqrt(x) + x)
    good &= keep
    return np.where(good, words, -1).astype(np.int32)


def valid_context_words(W, LB, UB):
    """Context word of every valid (centre, context) pair, in centre-major order
    (the compaction of Word2Vec.scala:283-330)."""
    W = np.asarray(W)
    n = W.shape[0]
    if n == 0:
        return np.zeros(0, np.int32)
    lo = int(min(LB.min(), 0))
    hi = int(max(UB.max(), 0))
    offs = np.array([j for j in range(lo, hi + 1) if j != 0], dtype=np.int64)
    if offs.size == 0:
        return np.zeros(0, np.int32)
    idx = np.arange(n, dtype=np.int64)[:, None]
    p = idx + offs[None, :]
    ok = (W[:, None] >= 0) & (LB[:, None] <= offs[None, :]) & (offs[None, :] <= UB[:, None])
    ok &= (p >= 0) & (p < n)
    pc = np.clip(p, 0, n - 1)
    ok &= W[pc] >= 0
    return W[pc][ok].astype(np.int32)


def count_pairs(W, LB, UB):
    """(number of valid pairs, number of centres with at least one valid pair)."""
    W = np.asarray(W)
    n = W.shape[0]
    if n == 0:
        return 0, 0
    lo = int(min(LB.min(), 0))
    hi = int(max(UB.max(), 0))
    per = np.zeros(n, dtype=np.int64)
    idx = np.arange(n, dtype=np.int64)
    for j in range(lo, hi + 1):
        if j == 0:
            continue
        p = idx + j
        ok = (W >= 0) & (LB <= j) & (j <= UB) & (p >= 0) & (p < n)
        ok[ok] &= W[p[ok]] >= 0
        per += ok
    return int(per.sum()), int((per > 0).sum())


def negative_groups(W, LB, UB, nneg, nreuse, rng, neg_cdf=None, vocab=None, wexpt=0.75):
    """WA (negatives, nneg per group) and WB (permuted contexts, nreuse per group), both
    group-contiguous, G = floor(#pairs / nreuse) groups (Word2Vec.scala:305,334-358)."""
    ctx = valid_context_words(W, LB, UB)
    g = ctx.shape[0] // nreuse
    ctx = rng.permutation(ctx)[: g * nreuse]
    if neg_cdf is not None:
        negs = sample_from_cdf(g * nneg, neg_cdf, rng)
    else:
        negs = closed_form_negatives(g * nneg, vocab, wexpt, rng)
    return negs.astype(np.int32), ctx.astype(np.int32), g


def init_tables(vocab, dim, seed=42):
    """Model start of the reference (Word2Vec.scala:112-117): modelmats(0) ~ U(-0.5/d, 0.5/d),
    modelmats(1) = 0.  Returned as (vocab, dim) C-order arrays = dim x vocab column-major."""
    rng = np.random.Generator(np.random.PCG64(seed))
    m0 = ((rng.random((vocab, dim), dtype=np.float32) - np.float32(0.5)) / np.float32(dim))
    m1 = np.zeros((vocab, dim), dtype=np.float32)
    return m0.astype(np.float32), m1


def collision_free_pos(n_centres, skip, vocab, rng):
    """A positive-pass minibatch in which every column is touched by exactly one work unit:
    distinct word ids, centres every 2*skip+1 tokens with the full window, all other tokens with
    an empty window."""
    period = 2 * skip + 1
    n = n_centres * period
    assert n <= vocab
    W = rng.permutation(vocab)[:n].astype(np.int32)
    LB = np.zeros(n, np.int32)
    UB = np.zeros(n, np.int32)
    centres = np.arange(n_centres) * period + skip
    LB[centres] = -skip
    UB[centres] = skip
    return W, LB, UB


def collision_free_neg(ngroups, nwa, nwb, vocab, rng):
    """A negative-pass minibatch whose nwa+nwb ids per group are distinct across all groups."""
    need = ngroups * (nwa + nwb)
    assert need <= vocab
    ids = rng.permutation(vocab)[:need].astype(np.int32)
    WA = ids[: ngroups * nwa].copy()
    WB = ids[ngroups * nwa:].copy()
    return WA, WB
