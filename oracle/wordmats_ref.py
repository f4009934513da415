"""numpy twin of the device minibatch preprocessing (TEST INFRASTRUCTURE).

Regenerates, from the same counter-based random numbers (Philox4x32-10 keyed by seed, call, stream
and element index), exactly what w2v_wordmats must produce, following the reference's
Word2Vec.wordMats / getnegs (src/main/scala/BIDMach/networks/Word2Vec.scala:214-364) step by
step.  The reference's own draws come from BIDMat and cannot be reproduced, so this pins the
device code against the reference's *rules*, not its random stream.
"""
import numpy as np

M0, M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
W0, W1 = np.uint32(0x9E3779B9), np.uint32(0xBB67AE85)
SUBSAMPLE, WINDOW, PERMUTE, NEGATIVE = 0, 1, 2, 3


def philox_word0(index, stream, call, seed):
    index = np.asarray(index, dtype=np.uint64)
    c0 = (index & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    c1 = (index >> np.uint64(32)).astype(np.uint32)
    c2 = np.full_like(c0, stream)
    c3 = np.full_like(c0, call)
    k0 = np.uint32(seed & 0xFFFFFFFF)
    k1 = np.uint32((seed >> 32) & 0xFFFFFFFF)
    with np.errstate(over="ignore"):
        for _ in range(10):
            p0 = M0 * c0.astype(np.uint64)
            p1 = M1 * c2.astype(np.uint64)
            n0 = (p1 >> np.uint64(32)).astype(np.uint32) ^ c1 ^ k0
            n1 = (p1 & np.uint64(0xFFFFFFFF)).astype(np.uint32)
            n2 = (p0 >> np.uint64(32)).astype(np.uint32) ^ c3 ^ k1
            n3 = (p0 & np.uint64(0xFFFFFFFF)).astype(np.uint32)
            c0, c1, c2, c3 = n0, n1, n2, n3
            k0 = np.uint32(k0 + W0)
            k1 = np.uint32(k1 + W1)
    return c0


def uniform01(x):
    return (x >> np.uint32(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)


def wordmats(words_in, sentence, vocab, nskip, nneg, nreuse, wsample_lnv, wexpt, seed, call):
    """Returns (words, lb, ub, negs, ctx, npairs, ngroups) as the device code must."""
    words_in = np.asarray(words_in, dtype=np.int32)
    sentence = np.asarray(sentence)
    n = words_in.shape[0]
    idx = np.arange(n, dtype=np.uint64)
    # OOV and frequent-word subsampling (Word2Vec.scala:218-225)
    good = (words_in >= 0) & (words_in < vocab)
    wrat = (words_in.astype(np.float32) + np.float32(1.0)) * np.float32(wsample_lnv)
    with np.errstate(invalid="ignore"):
        wrat = np.sqrt(wrat) + wrat
    good &= uniform01(philox_word0(idx, SUBSAMPLE, call, seed)) < wrat
    words = np.where(good, words_in, -1).astype(np.int32)
    # window bounds (:228-230) clipped at sentence boundaries (:233-237)
    u = uniform01(philox_word0(idx, WINDOW, call, seed))
    ub = np.minimum(nskip, (u * np.float32(nskip)).astype(np.int32) + 1).astype(np.int32)
    lb = -ub
    i64 = np.arange(n, dtype=np.int64)
    change = np.flatnonzero(sentence[1:] != sentence[:-1]) + 1
    starts = np.concatenate(([0], change))
    ends = np.concatenate((change, [n])) - 1
    seg = np.searchsorted(starts, i64, side="right") - 1
    lb = np.maximum(lb, starts[seg] - i64).astype(np.int32)
    ub = np.minimum(ub, ends[seg] - i64).astype(np.int32)
    # contexts in centre-major order (:283-330)
    ctx = []
    for i in range(n):
        if words[i] >= 0:
            for j in range(lb[i], ub[i] + 1):
                if j != 0 and words[i + j] >= 0:
                    ctx.append(words[i + j])
    ctx = np.array(ctx, dtype=np.int32)
    npairs = ctx.shape[0]
    ngroups = npairs // nreuse
    # permutation by stable sort on random keys (the reference's GPU branch sorts random values)
    keys = philox_word0(np.arange(npairs, dtype=np.uint64), PERMUTE, call, seed)
    ctx = ctx[np.argsort(keys, kind="stable")]
    # negatives min(V-1, floor(V * u**expt)) (:349-358)
    un = uniform01(philox_word0(np.arange(ngroups * nneg, dtype=np.uint64), NEGATIVE, call, seed))
    expt = 1.0 / (1.0 - float(np.float32(wexpt)))
    un = un.astype(np.float64)
    if expt == np.floor(expt) and 1.0 <= expt <= 16.0:
        p = np.ones_like(un)
        for _ in range(int(expt)):
            p = p * un
    else:
        p = un ** expt
    negs = np.minimum((vocab * p).astype(np.int64), vocab - 1).astype(np.int32)
    return words, lb, ub, negs, ctx, npairs, ngroups
