"""Writes tests/golden/raw_stream_oracle_losses.json: held-out losses of the C oracle (the CPU
restatement of jni/src/BIDMach_CPUMACH.c of the reference) on raw Zipf streams, at sizes or in
numbers that the GPU tests cannot afford to recompute on every run.

    python tests/golden/make_raw_stream_golden.py [--headline]

"constant_lr": the 10k-vocabulary configuration of tests/test_gpu_training.py (50 minibatches of
100k tokens, raw stream) at a CONSTANT learning rate, one thread (deterministic: the sequential
order) and 4 and 8 threads (not deterministic: one observed run each, kept as the oracle's own
spread at that rate).  "headline": vocab 1M, dim 300, 8 raw minibatches of 1M tokens with the
linear-decay schedule of test_headline_shape_raw_stream..., one thread (minutes of CPU), and one
observed run at 2 and 4 threads.
"""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from bidmach_amd import corpus  # noqa: E402
from oracle.cpumach import CPUMACH  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "raw_stream_oracle_losses.json")


def constant_lr(rates, threads=(1, 4, 8)):
    import test_gpu_training as T
    stream = T.make_stream(0.0)
    out = {}
    for lr in rates:
        row = {}
        for nt in threads:
            B, A = corpus.init_tables(T.V, T.D, 42)
            for i in range(T.NMB):
                W, LB, UB, WA, WB, G = stream[i]
                CPUMACH.word2vecPos(T.D, T.N, T.SKIP, W, LB, UB, A, B, lr, 0.0, nt)
                CPUMACH.word2vecNeg(T.D, G, T.NNEG, T.NREUSE, WA, WB, A, B, lr / T.NNEG, 0.0, nt)
            W, LB, UB, WA, WB, G = stream[T.NMB]
            row[str(nt)] = T.score(CPUMACH.word2vecEvalPos(T.D, T.N, T.SKIP, W, LB, UB, A, B, 8),
                                   CPUMACH.word2vecEvalNeg(T.D, G, T.NNEG, T.NREUSE, WA, WB, A, B, 8), G)
            print("constant lr %g, %d thread(s): %.6f" % (lr, nt, row[str(nt)]), flush=True)
        out["%g" % lr] = row
    return out


def headline(threads=(1, 2, 4)):
    Vh, Dh, Nh, K = 1_000_000, 300, 1_000_000, 8
    SKIP, NNEG, NREUSE, LR0 = 5, 5, 5, 0.025
    zc = corpus.zipf_cdf(Vh, 1.0)
    nc = corpus.unigram_pow_cdf(Vh, 1.0, 0.75)

    def mb(i):
        W = corpus.zipf_stream(Nh, Vh, 1.0, seed=1234 + i, cdf=zc)
        rng = np.random.Generator(np.random.PCG64(99 + i))
        LB, UB = corpus.window_bounds(Nh, SKIP, rng)
        WA, WB, G = corpus.negative_groups(W, LB, UB, NNEG, NREUSE, rng, neg_cdf=nc)
        return W, LB, UB, WA, WB, G

    mbs = [mb(i) for i in range(K + 1)]
    out = {}
    for nt in threads:
        t = time.time()
        B, A = corpus.init_tables(Vh, Dh, 42)
        for i in range(K):
            W, LB, UB, WA, WB, G = mbs[i]
            lr = max(LR0 * (1.0 - i / K), LR0 * 1e-4)
            CPUMACH.word2vecPos(Dh, Nh, SKIP, W, LB, UB, A, B, lr, 0.0, nt)
            CPUMACH.word2vecNeg(Dh, G, NNEG, NREUSE, WA, WB, A, B, lr / NNEG, 0.0, nt)
        W, LB, UB, WA, WB, G = mbs[K]
        epos = CPUMACH.word2vecEvalPos(Dh, Nh, SKIP, W, LB, UB, A, B, 8)
        eneg = CPUMACH.word2vecEvalNeg(Dh, G, NNEG, NREUSE, WA, WB, A, B, 8)
        out[str(nt)] = -(epos + eneg / NNEG) / (G * NREUSE)
        print("headline shape, %d thread(s): %.6f (%.0f s)" % (nt, out[str(nt)], time.time() - t),
              flush=True)
    return out


if __name__ == "__main__":
    data = json.load(open(OUT)) if os.path.exists(OUT) else {}
    if "--headline" in sys.argv:
        data["headline"] = headline()
    else:
        data["constant_lr"] = constant_lr([0.025, 0.0125, 0.005, 0.0035, 0.001])
    json.dump(data, open(OUT, "w"), indent=1, sort_keys=True)
    print("wrote", OUT)
