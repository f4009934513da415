#!/usr/bin/env python3
"""Headline benchmark: SGNS training step (word2vecPos + word2vecNeg) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one minibatch of the headline configuration (vocab 1M, dim 300, fp32, 1M tokens from a
Zipf(1.0) stream, window half-width 5, 5 negatives per positive drawn from unigram^0.75, groups of
5 contexts) pushed through the two update operators.  Index arrays and tables are resident in HBM
before the timed region starts.  Prints ONE JSON line.

Other workloads (--workload) are the remaining configurations at their full shapes: dim 512 with
window 10 and 15 negatives, the small vocab-10k configuration, forward-only scoring (--mode eval),
and bfloat16 tables at vocab 3M (word2vecPosBf16 + word2vecNegBf16; its CPU baseline is the
fp32 oracle on all host threads on the widened tables, with the single-threaded bfloat16 oracle
on a 300k-token sample beside it).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# w2v_last_launch_form: what the device-side count of a call's word ids decided
FORM_NAMES = {1: "ordered", 0: "throughput"}

# HBM bytes per launch of the update kernels, measured offline with rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE on this same command (summaries under profiles/, named in `source`), scaled by
# what the same counters read for a plain copy of known size in the same run (FETCH x2.0, WRITE
# x1.0).
HEADLINE = "sgns_v1m_d300_w5_neg5_fp32"
MEASURED_TRAFFIC = {
    HEADLINE: {
        # the kernels the library takes for this raw stream by itself
        "ordered": {"neg_kernel": 32.81e9, "pos_kernel": 20.69e9,
                    "source": "profiles/sgns_v1m_d300_ordered_step_kernel_stats_and_hbm_traffic.md"},
        # --ordered-mode 0
        "throughput": {"neg_kernel": 29.35e9, "pos_kernel": 4.63e9,
                       "source": "profiles/sgns_v1m_d300_step_hbm_traffic.md"},
    },
}

WORKLOADS = {
    # name: vocab, dim, tokens per minibatch, window half-width, nneg, nreuse, zipf exponent
    "sgns_v1m_d300_w5_neg5_fp32": dict(vocab=1_000_000, dim=300, tokens=1_000_000, skip=5, nneg=5,
                                       nreuse=5, zipf=1.0),
    "sgns_v1m_d512_w10_neg15_fp32": dict(vocab=1_000_000, dim=512, tokens=500_000, skip=10,
                                         nneg=15, nreuse=5, zipf=1.0),
    "sgns_v10k_d100_w5_neg5_fp32": dict(vocab=10_000, dim=100, tokens=100_000, skip=5, nneg=5,
                                        nreuse=5, zipf=1.0),
    # reduced-precision storage: bfloat16 tables, fp32 arithmetic, stochastic-rounded write-back
    # (word2vecPosBf16 + word2vecNegBf16)
    "sgns_v3m_d300_w5_neg5_bf16": dict(vocab=3_000_000, dim=300, tokens=1_000_000, skip=5, nneg=5,
                                       nreuse=5, zipf=1.1, storage="bf16"),
    # forward-only scoring configuration (use with --mode eval)
    "sgns_v100k_d300_w5_neg5_fp32": dict(vocab=100_000, dim=300, tokens=1_000_000, skip=5, nneg=5,
                                         nreuse=5, zipf=1.0),
}


def make_minibatch(cfg, index, zcdf, ncdf, wsample=0.0):
    """Index arrays of minibatch `index` of the stream (seeded, reproducible)."""
    from bidmach_amd import corpus
    n = cfg["tokens"]
    W = corpus.zipf_stream(n, cfg["vocab"], cfg["zipf"], seed=1234 + index, cdf=zcdf)
    rng = np.random.Generator(np.random.PCG64(99 + index))
    if wsample > 0.0:       # the reference caller's frequent-word subsampling: dropped words are -1
        W = corpus.subsample(W, cfg["vocab"], wsample, rng)
    LB, UB = corpus.window_bounds(n, cfg["skip"], rng)
    WA, WB, G = corpus.negative_groups(W, LB, UB, cfg["nneg"], cfg["nreuse"], rng, neg_cdf=ncdf)
    pairs, centres = corpus.count_pairs(W, LB, UB)
    return dict(W=W, LB=LB, UB=UB, WA=WA, WB=WB, G=G, pairs=pairs, centres=centres)


def algorithmic_bytes(cfg, mb):
    """Gather-scatter model: one read and one write of every column a work unit touches, plus the
    index arrays.  Pos: 2*C*(centres + pairs) + 12*N.  Neg: 2*C*G*(nwa+nwb) + 4*G*(nwa+nwb)."""
    C = cfg["dim"] * (2 if cfg.get("storage") == "bf16" else 4)
    pos = 2 * C * (mb["centres"] + mb["pairs"]) + 12 * cfg["tokens"]
    k = cfg["nneg"] + cfg["nreuse"]
    neg = 2 * C * mb["G"] * k + 4 * mb["G"] * k
    return pos, neg


def cpu_baseline(cfg, mbs, lr_pos, lr_neg, vexp, threads):
    """Times the C oracle (a port of the reference CPU path, built with the reference's flags) on
    full minibatches of the same workload, on this machine's host cores."""
    from bidmach_amd import corpus
    from oracle.cpumach import CPUMACH
    d, n = cfg["dim"], cfg["tokens"]
    B, A = corpus.init_tables(cfg["vocab"], d, seed=42)
    # warm-up on a slice so page faults and thread start-up stay out of the timing
    mb = mbs[0]
    m = min(n, 20000)
    CPUMACH.word2vecPos(d, m, cfg["skip"], mb["W"][:m].copy(), mb["LB"][:m].copy(),
                        mb["UB"][:m].copy(), A, B, lr_pos, vexp, threads)
    t0 = time.perf_counter()
    for mb in mbs:
        CPUMACH.word2vecPos(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B, lr_pos, vexp,
                            threads)
        CPUMACH.word2vecNeg(d, mb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"], mb["WB"], A, B,
                            lr_neg, vexp, threads)
    dt = time.perf_counter() - t0
    return len(mbs) * n / dt, dt


def cpu_baseline_bf16(cfg, mb, lr_pos, lr_neg, vexp, tokens):
    """Times the single-threaded bfloat16-storage oracle on the first `tokens` tokens of one
    minibatch and the groups that go with them."""
    from bidmach_amd import corpus
    from oracle.cpumach import CPUMACH, bf16_truncate
    d, n = cfg["dim"], cfg["tokens"]
    B, A = corpus.init_tables(cfg["vocab"], d, seed=42)
    A16, B16 = bf16_truncate(A), bf16_truncate(B)
    del A, B
    m = min(n, tokens)
    g = int(mb["G"] * (m / float(n)))
    W, LB, UB = mb["W"][:m].copy(), mb["LB"][:m].copy(), mb["UB"][:m].copy()
    WA, WB = mb["WA"][:g * cfg["nneg"]].copy(), mb["WB"][:g * cfg["nreuse"]].copy()
    CPUMACH.word2vecPosBf16(d, 2000, cfg["skip"], W, LB, UB, A16, B16, lr_pos, vexp, 1)  # warm-up
    t0 = time.perf_counter()
    CPUMACH.word2vecPosBf16(d, m, cfg["skip"], W, LB, UB, A16, B16, lr_pos, vexp, 2)
    CPUMACH.word2vecNegBf16(d, g, cfg["nneg"], cfg["nreuse"], WA, WB, A16, B16, lr_neg, vexp, 3)
    dt = time.perf_counter() - t0
    return m / dt, dt, m


def host_threads():
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        n = min(n, int(env))
    return max(1, n)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--vexp", type=float, default=0.0)
    ap.add_argument("--lrate", type=float, default=0.025)
    ap.add_argument("--distinct", type=int, default=8,
                    help="number of distinct minibatches generated; steps cycle through them")
    ap.add_argument("--mode", default="train", choices=["train", "eval"],
                    help="train: word2vecPos + word2vecNeg (the headline); eval: forward-only "
                         "word2vecEvalPos + word2vecEvalNeg")
    ap.add_argument("--parts", type=int, default=0,
                    help="train mode only: cut each table into this many separate allocations and "
                         "run the step through word2vecPosSlice + word2vecNegSlice (one worker)")
    ap.add_argument("--slices", type=int, default=1,
                    help="with --parts: number of workers the tail of the vocabulary is dealt to; "
                         "this process is worker 0 and holds only its share of the model")
    ap.add_argument("--head", type=int, default=0,
                    help="with --parts: number of head words (resident on every worker)")
    ap.add_argument("--rare-mode", type=int, default=-1,
                    help="w2v_set_rare_update_mode: 0 = float atomics for every column, -1/1 = "
                         "plain read-modify-write for words that are rare within a call "
                         "(default), n >= 2 = for words with at most n occurrences in the call")
    ap.add_argument("--tokens", type=int, default=0,
                    help="tokens per minibatch, overriding the workload's (the reference's own "
                         "default minibatch is 100000 tokens)")
    ap.add_argument("--wsample", type=float, default=0.0,
                    help="frequent-word subsampling threshold of the reference caller (its default "
                         "is 1e-4); 0 = the raw stream the headline metric is defined on")
    ap.add_argument("--hot-mode", type=int, default=-1, choices=[-1, 0, 1, 2],
                    help="w2v_set_hot_update_mode: -1 the library's per-launch choice (default), "
                         "0 exact shadow copies, 1 combining shadow copies, 2 no shadow copies")
    ap.add_argument("--bf16-hot-words", type=int, default=-1,
                    help="bf16 workload: w2v_set_bf16_hot_words (frequent words updated through "
                         "fp32 side buffers); -1 = the library's default")
    ap.add_argument("--max-workgroups", type=int, default=0,
                    help="w2v_set_max_workgroups: bound on the workgroups of the update kernels "
                         "(0 = the whole device)")
    ap.add_argument("--ordered-mode", type=int, default=-1, choices=(-1, 0, 1),
                    help="w2v_set_ordered_mode: -1 the library's per-launch choice (default: "
                         "launches full of frequent words run in the reference's order on a few "
                         "hundred wavefronts), 0 never (throughput kernels whatever the stream), "
                         "1 always")
    ap.add_argument("--ordered-workers", default="",
                    help="w2v_set_ordered_workers as POS,NEG (wavefronts of the ordered kernels; "
                         "default: the library's own numbers)")
    ap.add_argument("--ordered-copies", default="",
                    help="w2v_set_ordered_copies as COPIES,TWINS (delta slots of the 16 most "
                         "frequent columns in the ordered kernels; default: the library's 2,2)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-pcie", action="store_true",
                    help="skip the extra leg that uploads the index arrays from the host each step")
    ap.add_argument("--no-extra", action="store_true",
                    help="headline run only: skip the extra legs (the same workload on the "
                         "throughput kernels, at vexp 0.5 and with subsampling, and the other "
                         "configurations)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run one plain 1 GiB device copy before the timed region (gives a "
                         "kernel of known traffic to scale rocprofv3 FETCH_SIZE/WRITE_SIZE by)")
    return ap.parse_args()


def saturated_pair_share(torch, cfg, mb, A, B, sample=200_000):
    """Share of a minibatch's pairs whose pre-activation lies beyond the sigmoid's clamps (|s| > 16,
    BIDMach_CPUMACH.c:48-55) on the side where the step is exactly zero: positive pairs with
    s > 16, negative pairs with s < -16.  Estimated on a sample of the pairs of minibatch `mb`
    against the tables as the timed run left them."""
    rng = np.random.default_rng(7)
    n = cfg["tokens"]
    W, LB, UB = mb["W"], mb["LB"], mb["UB"]
    centres = rng.integers(0, n, sample)
    offs = rng.integers(1, cfg["skip"] + 1, sample) * rng.choice((-1, 1), sample)
    ctx = centres + offs
    ok = (ctx >= 0) & (ctx < n) & (offs >= LB[centres]) & (offs <= UB[centres])
    ok &= W[centres] >= 0
    ok[ok] &= W[ctx[ok]] >= 0
    wa = torch.from_numpy(W[centres[ok]].astype(np.int64)).cuda()
    wb = torch.from_numpy(W[ctx[ok]].astype(np.int64)).cuda()
    pos = float(((A[wa] * B[wb]).sum(1) > 16.0).float().mean().item()) if wa.numel() else 0.0
    g = rng.integers(0, mb["G"], sample // 5)
    j = rng.integers(0, cfg["nneg"], g.shape[0])
    k = rng.integers(0, cfg["nreuse"], g.shape[0])
    wa = torch.from_numpy(mb["WA"][g * cfg["nneg"] + j].astype(np.int64)).cuda()
    wb = torch.from_numpy(mb["WB"][g * cfg["nreuse"] + k].astype(np.int64)).cuda()
    neg = float(((A[wa] * B[wb]).sum(1) < -16.0).float().mean().item())
    return {"positive_pairs": pos, "negative_pairs": neg, "sampled_pairs": int(ok.sum())}


class Leg:
    """One workload on the device: its minibatches, tables and the timed loop."""

    def __init__(self, torch, name, tokens=0, wsample=0.0, distinct=8, steps=20, warmup=3,
                 vexp=0.0, lrate=0.025, mode="train", parts=0, slices=1, head=0):
        from bidmach_amd import corpus
        self.torch, self.name = torch, name
        self.forms = {}   # which kernels the library took, filled in by run()
        self.cfg = cfg = dict(WORKLOADS[name])
        if tokens > 0:
            cfg["tokens"] = tokens
        self.steps, self.warmup, self.vexp, self.lrate0, self.mode = steps, warmup, vexp, lrate, mode
        self.wsample, self.parts, self.slices, self.head = wsample, parts, slices, head
        d, V = cfg["dim"], cfg["vocab"]
        t0 = time.perf_counter()
        zcdf = corpus.zipf_cdf(V, cfg["zipf"])
        ncdf = corpus.unigram_pow_cdf(V, cfg["zipf"], 0.75)
        self.ndistinct = max(1, min(distinct, steps + warmup))
        self.host_mbs = [make_minibatch(cfg, i, zcdf, ncdf, wsample) for i in range(self.ndistinct)]
        self.dev_mbs = [{k: torch.from_numpy(mb[k]).cuda() for k in ("W", "LB", "UB", "WA", "WB")}
                        for mb in self.host_mbs]
        Bh, Ah = corpus.init_tables(V, d, seed=42)
        self.A = torch.from_numpy(Ah).cuda()
        self.B = torch.from_numpy(Bh).cuda()
        del Ah, Bh
        self.bf16 = cfg.get("storage") == "bf16"
        self.evaluating = mode == "eval"
        if self.bf16:
            if self.evaluating or parts > 0:
                sys.exit("bench.py: the bf16 workload runs in train mode on one unsliced model")
            from bidmach_amd.cumach import f32_to_bf16
            A16 = torch.empty(V * d, dtype=torch.int16, device="cuda")
            B16 = torch.empty(V * d, dtype=torch.int16, device="cuda")
            f32_to_bf16(V * d, self.A, A16)
            f32_to_bf16(V * d, self.B, B16)
            self.A, self.B = A16, B16
        if self.evaluating:   # scoring needs non-trivial tables: N(0, 0.1) as the forward-only config says
            self.A.normal_(0.0, 0.1)
            self.B.normal_(0.0, 0.1)
        self.ret = torch.zeros(2, dtype=torch.float32, device="cuda")
        self.MM, self.maxcols = None, 0
        if parts > 0 and not self.evaluating:
            # worker 0 of `slices`: head words, then its tail words in id order, cut into parts
            ids = torch.arange(V, device="cuda")
            keep = (ids < head) | ((ids >= head) & (ids % slices == 0))
            packedB, packedA = self.B[keep], self.A[keep]
            resident = packedB.shape[0]
            self.maxcols = (resident + parts - 1) // parts
            self.MM = []
            for c0 in range(0, resident, self.maxcols):
                self.MM += [packedB[c0:c0 + self.maxcols].clone(),
                            packedA[c0:c0 + self.maxcols].clone()]
        torch.cuda.synchronize()
        self.prep_s = time.perf_counter() - t0

    def lrate(self, step):   # linear decay over the run, floor at 1e-4 of the start
        total = self.steps + self.warmup
        return max(self.lrate0 * (1.0 - step / float(max(total, 1))), self.lrate0 * 1e-4)

    def step(self, s, timers=None, forms=None):
        """One pass of both operators over minibatch s.  `forms` (a dict), if given, is told after
        each of the two calls which kernels the library took for it (w2v_last_launch_form: read
        back from the device, so it waits for the call)."""
        from bidmach_amd.cumach import CUMACH, check, load_library
        cfg, A, B, ret, MM = self.cfg, self.A, self.B, self.ret, self.MM
        d, n = cfg["dim"], cfg["tokens"]
        mb, hmb = self.dev_mbs[s % self.ndistinct], self.host_mbs[s % self.ndistinct]
        lr = self.lrate(s)
        if timers:
            timers[0].start()
        if self.evaluating:
            check(CUMACH.word2vecEvalPosAsync(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B,
                                              ret[0:1]), "word2vecEvalPos")
        elif self.bf16:
            check(CUMACH.word2vecPosBf16Async(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B,
                                              lr, self.vexp, 2 * s), "word2vecPosBf16")
        elif MM:
            check(CUMACH.word2vecPosSlice(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], MM, lr,
                                          self.vexp, 0, self.slices, self.maxcols, self.head, False,
                                          1), "word2vecPosSlice")
        else:
            check(CUMACH.word2vecPosAsync(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B, lr,
                                          self.vexp), "word2vecPos")
        if timers:
            timers[0].stop()
            timers[1].start()
        if forms is not None and not self.evaluating:
            forms["pos"] = FORM_NAMES.get(load_library().w2v_last_launch_form(), "unknown")
        if self.evaluating:
            check(CUMACH.word2vecEvalNegAsync(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                              mb["WB"], A, B, ret[1:2]), "word2vecEvalNeg")
        elif self.bf16:
            check(CUMACH.word2vecNegBf16Async(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                              mb["WB"], A, B, lr / cfg["nneg"], self.vexp,
                                              2 * s + 1), "word2vecNegBf16")
        elif MM:
            check(CUMACH.word2vecNegSlice(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                          mb["WB"], MM, lr / cfg["nneg"], self.vexp, 0, self.slices,
                                          self.maxcols, self.head, False, 1), "word2vecNegSlice")
        else:
            check(CUMACH.word2vecNegAsync(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                          mb["WB"], A, B, lr / cfg["nneg"], self.vexp),
                  "word2vecNeg")
        if timers:
            timers[1].stop()
        if forms is not None and not self.evaluating:
            forms["neg"] = FORM_NAMES.get(load_library().w2v_last_launch_form(), "unknown")

    def finite(self):
        torch = self.torch
        ts = self.MM if self.MM else [self.A, self.B]
        return all(bool(torch.isfinite(t.view(torch.bfloat16) if self.bf16 else t).all())
                   for t in ts)

    def run(self):
        """Warm-up, then exactly `steps` timed steps between two device synchronisations.  Each
        pass is bracketed by HIP events on the library's launch stream."""
        from bidmach_amd.cumach import Timer, synchronize
        torch, K, Wm, cfg = self.torch, self.steps, self.warmup, self.cfg
        for s in range(Wm):
            self.step(s)
        synchronize()
        torch.cuda.synchronize()
        timers = [(Timer(), Timer()) for _ in range(K)]
        t0 = time.perf_counter()
        for s in range(K):
            self.step(Wm + s, timers[s])
        synchronize()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        pos_ms = float(np.mean([t[0].elapsed_ms() for t in timers]))
        neg_ms = float(np.mean([t[1].elapsed_ms() for t in timers]))
        pos_b, neg_b = zip(*[algorithmic_bytes(cfg, self.host_mbs[(Wm + s) % self.ndistinct])
                             for s in range(K)])
        pos_b, neg_b = float(np.mean(pos_b)), float(np.mean(neg_b))
        if self.evaluating:   # reads only: half of the read-and-write model
            pos_b, neg_b = pos_b / 2, neg_b / 2
        assert self.finite(), "tables diverged"
        # one more, untimed step that asks the library which kernels it takes for this stream
        self.forms = {}
        if not self.evaluating:
            self.step(Wm + K, forms=self.forms)
            synchronize()
        gbps = lambda b, ms: b / (ms * 1e-3) / 1e9
        return {
            "elapsed": elapsed, "words_per_s": K * cfg["tokens"] / elapsed,
            "ms_per_step": elapsed / K * 1e3,
            "pos_ms": pos_ms, "neg_ms": neg_ms, "pos_bytes": pos_b, "neg_bytes": neg_b,
            "pos_gbps": gbps(pos_b, pos_ms), "neg_gbps": gbps(neg_b, neg_ms),
            "step_gbps": gbps(pos_b + neg_b, pos_ms + neg_ms),
        }

    def roofline(self, r, traffic=None, traffic_source=None):
        """The dominant kernel: whichever pass takes longer (the negative pass, 63 % of the step's
        algorithmic bytes, on the throughput kernels; the positive pass on the ordered ones).
        `traffic` maps "neg_kernel" / "pos_kernel" to measured HBM bytes per launch, or is None."""
        k = "neg" if r["neg_ms"] >= r["pos_ms"] else "pos"
        out = {"bound": "hbm", "kernel": k + "_kernel", "achieved": r[k + "_gbps"],
               "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": r[k + "_gbps"] / HBM_PEAK_GBPS,
               "traffic": traffic.get(k + "_kernel") if traffic else None,
               "algorithmic_bytes_per_launch": r[k + "_bytes"], "avg_launch_ms": r[k + "_ms"]}
        if traffic and traffic_source:
            out["traffic_source"] = traffic_source
        return out

    def kernels(self, r):
        return {
            "pos_kernel": {"avg_launch_ms": r["pos_ms"],
                           "algorithmic_bytes_per_launch": r["pos_bytes"],
                           "achieved_GBps": r["pos_gbps"], "frac": r["pos_gbps"] / HBM_PEAK_GBPS},
            "neg_kernel": {"avg_launch_ms": r["neg_ms"],
                           "algorithmic_bytes_per_launch": r["neg_bytes"],
                           "achieved_GBps": r["neg_gbps"], "frac": r["neg_gbps"] / HBM_PEAK_GBPS},
            "step": {"achieved_GBps": r["step_gbps"], "frac": r["step_gbps"] / HBM_PEAK_GBPS,
                     "kernel_ms": r["pos_ms"] + r["neg_ms"]},
        }

    def cpu(self, nmb):
        """The CPU baseline of this leg on `nmb` of its minibatches (bf16: a 300k-token sample on
        the single-threaded bf16 oracle)."""
        cfg = self.cfg
        threads = host_threads()
        if self.bf16:
            # the same arithmetic on fp32 tables (the bfloat16 tables widened), all host threads,
            # is what a CPU would run; the bfloat16 oracle itself has one thread
            wps32, dt32 = cpu_baseline(cfg, self.host_mbs[:1], self.lrate0,
                                       self.lrate0 / cfg["nneg"], self.vexp, threads)
            wps, dt, m = cpu_baseline_bf16(cfg, self.host_mbs[0], self.lrate0,
                                           self.lrate0 / cfg["nneg"], self.vexp, 300_000)
            return {"value": wps32, "unit": "words/s", "cores": threads, "kind": "port",
                    "sample": "one full minibatch (%d tokens) of the same workload on fp32 tables "
                              "(the fp32 oracle: same arithmetic, no rounding of the write-back), "
                              "pos+neg, %.1f s wall" % (cfg["tokens"], dt32),
                    "bf16_oracle_one_thread": {
                        "value": wps, "unit": "words/s", "cores": 1,
                        "sample": "the first %d tokens of one minibatch and their groups, "
                                  "pos+neg, %.1f s wall" % (m, dt)}}
        sample = self.host_mbs[:nmb]
        wps, dt = cpu_baseline(cfg, sample, self.lrate0, self.lrate0 / cfg["nneg"], self.vexp,
                               threads)
        return {"value": wps, "unit": "words/s", "cores": threads, "kind": "port",
                "sample": "%d full minibatches (%d tokens each) of the same workload, pos+neg, "
                          "%.1f s wall" % (len(sample), cfg["tokens"], dt)}

    def config(self):
        cfg = self.cfg
        return {"workload": self.name, "vocab": cfg["vocab"], "dim": cfg["dim"],
                "tokens_per_minibatch": cfg["tokens"], "window": cfg["skip"], "nneg": cfg["nneg"],
                "nreuse": cfg["nreuse"], "zipf_s": cfg["zipf"], "vexp": self.vexp,
                "lrate": self.lrate0, "distinct_minibatches": self.ndistinct,
                "pairs_per_minibatch": int(np.mean([m["pairs"] for m in self.host_mbs])),
                "groups_per_minibatch": int(np.mean([m["G"] for m in self.host_mbs]))}

    def free(self):
        self.A = self.B = self.MM = self.dev_mbs = None
        self.torch.cuda.empty_cache()


def brief(leg, r, with_cpu_mbs=0):
    """The short record of an extra leg."""
    out = {"workload": leg.name, "words_per_s": r["words_per_s"], "ms_per_step": r["ms_per_step"],
           "pos_ms": r["pos_ms"], "neg_ms": r["neg_ms"], "steps": leg.steps,
           "roofline": leg.roofline(r),
           "step_frac_of_hbm_peak": r["step_gbps"] / HBM_PEAK_GBPS}
    if leg.forms:
        out["update_kernels_ran"] = dict(leg.forms)
    if with_cpu_mbs:
        out["cpu_baseline"] = leg.cpu(with_cpu_mbs)
        out["cpu_baseline"]["gpu_over_cpu"] = r["words_per_s"] / out["cpu_baseline"]["value"]
    return out


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); "
                 "run it with --gpus 1")

    import torch
    from bidmach_amd.cumach import check, load_library, synchronize

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    lib = load_library()
    lib.w2v_set_hot_update_mode(args.hot_mode)
    lib.w2v_set_rare_update_mode(args.rare_mode)
    lib.w2v_set_ordered_mode(args.ordered_mode)
    if args.ordered_workers:
        pw, nw = (int(x) for x in args.ordered_workers.split(","))
        check(lib.w2v_set_ordered_workers(pw, nw), "w2v_set_ordered_workers")
    if args.ordered_copies:
        cc, tt = (int(x) for x in args.ordered_copies.split(","))
        check(lib.w2v_set_ordered_copies(cc, tt), "w2v_set_ordered_copies")
    if args.bf16_hot_words >= 0:
        check(lib.w2v_set_bf16_hot_words(args.bf16_hot_words), "w2v_set_bf16_hot_words")
    if args.max_workgroups > 0:
        lib.w2v_set_max_workgroups(args.max_workgroups)

    leg = Leg(torch, args.workload, tokens=args.tokens, wsample=args.wsample,
              distinct=args.distinct, steps=args.steps, warmup=args.warmup, vexp=args.vexp,
              lrate=args.lrate, mode=args.mode, parts=args.parts, slices=args.slices,
              head=args.head)
    cfg, n, K, Wm = leg.cfg, leg.cfg["tokens"], args.steps, args.warmup
    evaluating, bf16, MM = leg.evaluating, leg.bf16, leg.MM

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    r = leg.run()
    words_per_s = r["words_per_s"]
    plain = (not evaluating and not MM and not bf16 and args.tokens == 0 and args.wsample == 0.0
             and args.hot_mode == -1 and args.rare_mode == -1 and args.max_workgroups == 0
             and args.ordered_mode == -1 and not args.ordered_workers)
    # HBM bytes per launch measured with rocprofv3 counters apply to the kernels they were taken on
    traffic = traffic_source = None
    if args.workload in MEASURED_TRAFFIC and not evaluating and not MM and args.tokens == 0 \
            and args.wsample == 0.0 and not args.ordered_workers and args.rare_mode == -1 \
            and args.max_workgroups == 0 and args.hot_mode == -1:
        key = "ordered" if args.ordered_mode != 0 else "throughput"
        m = MEASURED_TRAFFIC[args.workload].get(key)
        if m:
            traffic, traffic_source = m, m["source"]
    out = {
        "metric": ("scored words/sec (forward only), " + args.workload) if evaluating
                  else "updated words/sec, SGNS V=1M d=300 w=5 neg=5 fp32"
                  if args.workload == HEADLINE else "updated words/sec, " + args.workload,
        "value": words_per_s,
        "unit": "words/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": Wm,
        "ms_per_step": r["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",   # arithmetic type; the bf16 workload stores bf16 and computes in fp32
        "data": "synthetic",
        "config": leg.config(),
        "roofline": leg.roofline(r, traffic, traffic_source),
        "kernels": leg.kernels(r),
        "host_prep_s": leg.prep_s,
    }
    if leg.forms:
        # as the library reports it for the step after the timed ones (w2v_last_launch_form)
        out["config"]["update_kernels_ran"] = dict(leg.forms)
    if not evaluating and not MM and not bf16:
        # which form of the update operators the library took for this stream (its own choice
        # unless --ordered-mode says otherwise): launches full of frequent words run in the
        # reference's order on a bounded number of wavefronts
        out["config"]["update_kernels"] = (
            "ordered (pos_chain_kernel + neg_rows_kernel)"
            if (args.ordered_mode == 1 or (args.ordered_mode == -1 and args.wsample == 0.0
                                           and args.hot_mode == -1))
            else "throughput (pos_tile_kernel + neg_train_kernel)")
    if evaluating:
        out["config"]["mode"] = "eval"
    if args.max_workgroups > 0:
        out["config"]["max_workgroups"] = args.max_workgroups
    if bf16:
        out["config"]["storage"] = "bf16"
        out["config"]["hot_words"] = lib.w2v_get_bf16_hot_words()
        out["config"]["operators"] = "word2vecPosBf16+word2vecNegBf16"
    if args.hot_mode != -1:
        out["config"]["hot_update_mode"] = args.hot_mode
    if args.rare_mode != -1:
        out["config"]["rare_update_mode"] = args.rare_mode
    if args.ordered_mode != -1:
        out["config"]["ordered_mode"] = args.ordered_mode
    if args.ordered_workers:
        out["config"]["ordered_workers"] = args.ordered_workers
    if args.wsample > 0.0:
        out["config"]["wsample"] = args.wsample
    if MM:
        out["config"]["parts"] = len(MM) // 2
        out["config"]["slices"] = args.slices
        out["config"]["head_words"] = args.head
        out["config"]["operators"] = "word2vecPosSlice+word2vecNegSlice"
    if not evaluating and not MM and not bf16:
        out["saturated_pair_share"] = saturated_pair_share(torch, cfg, leg.host_mbs[0], leg.A,
                                                           leg.B)
    if not evaluating and not MM and not bf16 and not args.no_pcie:
        # The same step with the five index arrays uploaded from pinned host memory first (what a
        # caller that builds them on the host pays); serialised with the kernels, not overlapped.
        # Reported beside the headline value, never as it.
        pinned = [{k: torch.from_numpy(mb[k]).pin_memory() for k in ("W", "LB", "UB", "WA", "WB")}
                  for mb in leg.host_mbs]
        k2 = min(K, 10)
        for rep in range(2):                       # first repetition warms the copies up
            synchronize()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for s_ in range(k2):
                src, dst = pinned[s_ % leg.ndistinct], leg.dev_mbs[s_ % leg.ndistinct]
                for key in dst:
                    dst[key].copy_(src[key], non_blocking=True)
                leg.step(Wm + K + s_)
            synchronize()
            torch.cuda.synchronize()
            t_h2d = time.perf_counter() - t1
        upload = sum(v.numel() * 4 for v in pinned[0].values())
        out["pcie_inclusive"] = {"value": k2 * n / t_h2d, "unit": "words/s",
                                 "ms_per_step": 1e3 * t_h2d / k2, "steps": k2,
                                 "uploaded_bytes_per_step": upload}
        del pinned
        assert leg.finite(), "tables diverged"

    # The streaming ceiling of this box, for scale: a plain 1 GiB device-to-device copy.
    src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    copy_gbps = 5 * 2 * src.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst
    out["hbm_copy"] = {"achieved": copy_gbps, "unit": "GB/s read+write",
                       "step_algorithmic_over_copy": r["step_gbps"] / copy_gbps}

    if not args.no_cpu_baseline and not evaluating:
        out["cpu_baseline"] = leg.cpu(3)
        out["cpu_baseline"]["gpu_over_cpu"] = words_per_s / out["cpu_baseline"]["value"]

    if plain and args.workload == HEADLINE and not args.no_extra:
        leg.free()
        out.update(extra_legs(torch, lib, args, out))

    print(json.dumps(out))


def extra_legs(torch, lib, args, headline):
    """The figures that belong next to the headline: the same workload on the throughput kernels
    and in the other regimes, and the other configurations, each a short run of its own."""
    extra = {}
    few = dict(steps=6, warmup=2, distinct=4, lrate=args.lrate)

    # (a) the headline stream on the throughput kernels, which the library does not take for it
    # by itself: what the ordered form costs.  On this stream these kernels are fast and wrong:
    # the held-out loss ends many times the reference's (tests/test_gpu_training.py).
    lib.w2v_set_ordered_mode(0)
    leg = Leg(torch, HEADLINE, vexp=args.vexp, **few)
    r = leg.run()
    m = MEASURED_TRAFFIC[HEADLINE]["throughput"]
    extra["throughput_kernels_on_the_raw_stream"] = {
        "note": "w2v_set_ordered_mode(0): thousands of work units in flight; does not hold the "
                "held-out-loss tolerance on a raw (not subsampled) stream, shown for the cost of "
                "the ordered form only",
        "words_per_s": r["words_per_s"], "ms_per_step": r["ms_per_step"], "pos_ms": r["pos_ms"],
        "neg_ms": r["neg_ms"],
        "roofline": leg.roofline(r, m, m["source"]),
        "step_frac_of_hbm_peak": r["step_gbps"] / HBM_PEAK_GBPS,
        "saturated_pair_share": saturated_pair_share(torch, leg.cfg, leg.host_mbs[0], leg.A, leg.B),
        "ordered_over_throughput_time": headline["ms_per_step"] / r["ms_per_step"],
        "update_kernels_ran": dict(leg.forms)}
    leg.free()
    lib.w2v_set_ordered_mode(-1)

    # (b) the step sizes of the reference's own recipe: vexp = 0.5 with lrate = 1e-3
    # (scripts/testword2vec.ssc:11-12); at lrate 0.025 a vexp of 0.5 multiplies the step of a
    # word of rank 1M by 1000 and the tables overflow
    leg = Leg(torch, HEADLINE, vexp=0.5, steps=6, warmup=2, distinct=4, lrate=1.0e-3)
    r = leg.run()
    extra["headline_at_vexp_0.5_lrate_1e-3"] = brief(leg, r)
    extra["headline_at_vexp_0.5_lrate_1e-3"]["saturated_pair_share"] = saturated_pair_share(
        torch, leg.cfg, leg.host_mbs[0], leg.A, leg.B)
    leg.free()

    # (c) the headline shape behind the reference caller's default frequent-word subsampling
    # (wsample = 1e-4, Word2Vec.scala:150,221-225): no frequent words left, throughput kernels
    leg = Leg(torch, HEADLINE, wsample=1.0e-4, vexp=args.vexp, **few)
    r = leg.run()
    extra["headline_shape_subsampled_1e-4"] = brief(leg, r, with_cpu_mbs=0 if args.no_cpu_baseline else 2)
    extra["headline_shape_subsampled_1e-4"]["note"] = (
        "words/s counts raw tokens (dropped ones included), as the caller feeds them")
    leg.free()

    configs = {}
    # configuration 2: forward only, vocab 100k
    leg = Leg(torch, "sgns_v100k_d300_w5_neg5_fp32", mode="eval", **few)
    r = leg.run()
    configs["cfg2_forward_only_v100k_d300"] = brief(leg, r)
    configs["cfg2_forward_only_v100k_d300"]["unit"] = "scored words/s"
    if not args.no_cpu_baseline:
        configs["cfg2_forward_only_v100k_d300"]["cpu_baseline"] = cpu_eval_baseline(leg)
    leg.free()
    # configuration 4: bfloat16 tables, vocab 3M, raw Zipf(1.1) stream (ordered kernels by the
    # device-side count, like the fp32 operators on the headline stream)
    leg = Leg(torch, "sgns_v3m_d300_w5_neg5_bf16", steps=4, warmup=1, distinct=2, lrate=args.lrate)
    r = leg.run()
    configs["cfg4_bf16_v3m_d300_zipf1.1"] = brief(leg, r, with_cpu_mbs=0 if args.no_cpu_baseline else 1)
    leg.free()
    # configuration 5: dim 512, window 10, 15 negatives, 500k tokens
    leg = Leg(torch, "sgns_v1m_d512_w10_neg15_fp32", steps=4, warmup=1, distinct=2,
              lrate=args.lrate)
    r = leg.run()
    configs["cfg5_v1m_d512_w10_neg15"] = brief(leg, r, with_cpu_mbs=0 if args.no_cpu_baseline else 1)
    leg.free()
    extra["configs"] = configs
    return extra


def cpu_eval_baseline(leg):
    """Forward-only CPU baseline: the oracle's two scoring functions on one minibatch."""
    from oracle.cpumach import CPUMACH
    cfg, mb = leg.cfg, leg.host_mbs[0]
    d, n = cfg["dim"], cfg["tokens"]
    A, B = leg.A.cpu().numpy(), leg.B.cpu().numpy()
    threads = host_threads()
    t0 = time.perf_counter()
    CPUMACH.word2vecEvalPos(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B, threads)
    CPUMACH.word2vecEvalNeg(d, mb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"], mb["WB"], A, B,
                            threads)
    dt = time.perf_counter() - t0
    return {"value": n / dt, "unit": "scored words/s", "cores": threads, "kind": "port",
            "sample": "one full minibatch (%d tokens), EvalPos+EvalNeg, %.1f s wall" % (n, dt)}


if __name__ == "__main__":
    main()
