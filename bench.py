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
single-threaded bf16 oracle on a 300k-token sample).
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

# HBM bytes per launch of the dominant kernel, measured offline with rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE on this same command (summaries under profiles/), scaled by what the same
# counters read for a plain copy of known size in the same run (FETCH x2.0, WRITE x1.0).
MEASURED_TRAFFIC_BYTES = {
    "sgns_v1m_d300_w5_neg5_fp32": {"neg_kernel": 29.35e9, "pos_kernel": 4.63e9},
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="sgns_v1m_d300_w5_neg5_fp32", choices=sorted(WORKLOADS))
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
    ap.add_argument("--rare-mode", type=int, default=-1, choices=(-1, 0, 1),
                    help="w2v_set_rare_update_mode: 0 = float atomics for every column, -1/1 = "
                         "plain read-modify-write for words that are rare within a call (default)")
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
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-pcie", action="store_true",
                    help="skip the extra leg that uploads the index arrays from the host each step")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run one plain 1 GiB device copy before the timed region (gives a "
                         "kernel of known traffic to scale rocprofv3 FETCH_SIZE/WRITE_SIZE by)")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); "
                 "run it with --gpus 1")

    import torch
    from bidmach_amd import corpus
    from bidmach_amd.cumach import CUMACH, Timer, check, synchronize

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    from bidmach_amd.cumach import load_library
    load_library().w2v_set_hot_update_mode(args.hot_mode)
    load_library().w2v_set_rare_update_mode(args.rare_mode)
    load_library().w2v_set_ordered_mode(args.ordered_mode)
    if args.bf16_hot_words >= 0:
        check(load_library().w2v_set_bf16_hot_words(args.bf16_hot_words), "w2v_set_bf16_hot_words")
    if args.max_workgroups > 0:
        load_library().w2v_set_max_workgroups(args.max_workgroups)
    cfg = dict(WORKLOADS[args.workload])
    if args.tokens > 0:
        cfg["tokens"] = args.tokens
    d, V, n = cfg["dim"], cfg["vocab"], cfg["tokens"]
    K, Wm = args.steps, args.warmup

    t_prep = time.perf_counter()
    zcdf = corpus.zipf_cdf(V, cfg["zipf"])
    ncdf = corpus.unigram_pow_cdf(V, cfg["zipf"], 0.75)
    ndistinct = max(1, min(args.distinct, K + Wm))
    host_mbs = [make_minibatch(cfg, i, zcdf, ncdf, args.wsample) for i in range(ndistinct)]
    dev_mbs = []
    for mb in host_mbs:
        dev_mbs.append({k: torch.from_numpy(mb[k]).cuda() for k in ("W", "LB", "UB", "WA", "WB")})
    Bh, Ah = corpus.init_tables(V, d, seed=42)
    A = torch.from_numpy(Ah).cuda()
    B = torch.from_numpy(Bh).cuda()
    del Ah, Bh
    torch.cuda.synchronize()
    t_prep = time.perf_counter() - t_prep

    total = K + Wm

    def lrate(step):   # linear decay over the run, floor at 1e-4 of the start
        return max(args.lrate * (1.0 - step / float(max(total, 1))), args.lrate * 1e-4)

    evaluating = args.mode == "eval"
    bf16 = cfg.get("storage") == "bf16"
    if bf16:
        if evaluating or args.parts > 0:
            sys.exit("bench.py: the bf16 workload runs in train mode on one unsliced model")
        from bidmach_amd.cumach import f32_to_bf16
        A16 = torch.empty(V * d, dtype=torch.int16, device="cuda")
        B16 = torch.empty(V * d, dtype=torch.int16, device="cuda")
        f32_to_bf16(V * d, A, A16)
        f32_to_bf16(V * d, B, B16)
        del A, B
        A, B = A16, B16
    if evaluating:   # scoring needs non-trivial tables: N(0, 0.1) as the forward-only config says
        A.normal_(0.0, 0.1)
        B.normal_(0.0, 0.1)
    ret = torch.zeros(2, dtype=torch.float32, device="cuda")
    MM, maxcols = None, 0
    if args.parts > 0 and not evaluating:
        # worker 0 of --slices: head words, then its tail words in id order, cut into --parts parts
        ids = torch.arange(V, device="cuda")
        keep = (ids < args.head) | ((ids >= args.head) & (ids % args.slices == 0))
        packedB, packedA = B[keep], A[keep]
        resident = packedB.shape[0]
        maxcols = (resident + args.parts - 1) // args.parts
        MM = []
        for c0 in range(0, resident, maxcols):
            MM += [packedB[c0:c0 + maxcols].clone(), packedA[c0:c0 + maxcols].clone()]
        del ids, keep, packedA, packedB

    def step(s, timers=None):
        mb, hmb = dev_mbs[s % ndistinct], host_mbs[s % ndistinct]
        lr = lrate(s)
        if timers:
            timers[0].start()
        if evaluating:
            check(CUMACH.word2vecEvalPosAsync(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B,
                                              ret[0:1]), "word2vecEvalPos")
        elif bf16:
            check(CUMACH.word2vecPosBf16Async(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B,
                                              lr, args.vexp, 2 * s), "word2vecPosBf16")
        elif MM:
            check(CUMACH.word2vecPosSlice(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], MM, lr,
                                          args.vexp, 0, args.slices, maxcols, args.head, False, 1),
                  "word2vecPosSlice")
        else:
            check(CUMACH.word2vecPosAsync(d, n, cfg["skip"], mb["W"], mb["LB"], mb["UB"], A, B, lr,
                                          args.vexp), "word2vecPos")
        if timers:
            timers[0].stop()
            timers[1].start()
        if evaluating:
            check(CUMACH.word2vecEvalNegAsync(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                              mb["WB"], A, B, ret[1:2]), "word2vecEvalNeg")
        elif bf16:
            check(CUMACH.word2vecNegBf16Async(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                              mb["WB"], A, B, lr / cfg["nneg"], args.vexp,
                                              2 * s + 1), "word2vecNegBf16")
        elif MM:
            check(CUMACH.word2vecNegSlice(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                          mb["WB"], MM, lr / cfg["nneg"], args.vexp, 0, args.slices,
                                          maxcols, args.head, False, 1), "word2vecNegSlice")
        else:
            check(CUMACH.word2vecNegAsync(d, hmb["G"], cfg["nneg"], cfg["nreuse"], mb["WA"],
                                          mb["WB"], A, B, lr / cfg["nneg"], args.vexp),
                  "word2vecNeg")
        if timers:
            timers[1].stop()

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for s in range(Wm):
        step(s)
    synchronize()
    torch.cuda.synchronize()

    timers = [(Timer(), Timer()) for _ in range(K)]
    t0 = time.perf_counter()
    for s in range(K):
        step(Wm + s, timers[s])
    synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    pos_ms = [t[0].elapsed_ms() for t in timers]
    neg_ms = [t[1].elapsed_ms() for t in timers]
    pos_b, neg_b = zip(*[algorithmic_bytes(cfg, host_mbs[(Wm + s) % ndistinct]) for s in range(K)])
    avg_pos_ms, avg_neg_ms = float(np.mean(pos_ms)), float(np.mean(neg_ms))
    avg_pos_b, avg_neg_b = float(np.mean(pos_b)), float(np.mean(neg_b))
    if evaluating:   # reads only: half of the read-and-write model
        avg_pos_b, avg_neg_b = avg_pos_b / 2, avg_neg_b / 2
    pos_gbps = avg_pos_b / (avg_pos_ms * 1e-3) / 1e9
    neg_gbps = avg_neg_b / (avg_neg_ms * 1e-3) / 1e9
    step_gbps = (avg_pos_b + avg_neg_b) / ((avg_pos_ms + avg_neg_ms) * 1e-3) / 1e9

    def finite(t):
        return bool(torch.isfinite(t.view(torch.bfloat16) if bf16 else t).all())

    assert finite(A) and finite(B), "tables diverged"
    if MM:
        assert all(bool(torch.isfinite(m).all()) for m in MM), "tables diverged"

    words_per_s = K * n / elapsed
    out = {
        "metric": ("scored words/sec (forward only), " + args.workload) if evaluating
                  else "updated words/sec, SGNS V=1M d=300 w=5 neg=5 fp32"
                  if args.workload == "sgns_v1m_d300_w5_neg5_fp32"
                  else "updated words/sec, " + args.workload,
        "value": words_per_s,
        "unit": "words/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": Wm,
        "ms_per_step": elapsed / K * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",   # arithmetic type; the bf16 workload stores bf16 and computes in fp32
        "data": "synthetic",
        "config": {"workload": args.workload, "vocab": V, "dim": d, "tokens_per_minibatch": n,
                   "window": cfg["skip"], "nneg": cfg["nneg"], "nreuse": cfg["nreuse"],
                   "zipf_s": cfg["zipf"], "vexp": args.vexp, "lrate": args.lrate,
                   "distinct_minibatches": ndistinct,
                   "pairs_per_minibatch": int(np.mean([m["pairs"] for m in host_mbs])),
                   "groups_per_minibatch": int(np.mean([m["G"] for m in host_mbs]))},
        # the negative pass moves ~63% of the step's algorithmic bytes: it is the dominant kernel
        "roofline": {"bound": "hbm", "kernel": "neg_kernel", "achieved": neg_gbps,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": neg_gbps / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload, {}).get("neg_kernel"),
                     "algorithmic_bytes_per_launch": avg_neg_b,
                     "avg_launch_ms": avg_neg_ms},
        "kernels": {
            "pos_kernel": {"avg_launch_ms": avg_pos_ms, "algorithmic_bytes_per_launch": avg_pos_b,
                           "achieved_GBps": pos_gbps, "frac": pos_gbps / HBM_PEAK_GBPS},
            "neg_kernel": {"avg_launch_ms": avg_neg_ms, "algorithmic_bytes_per_launch": avg_neg_b,
                           "achieved_GBps": neg_gbps, "frac": neg_gbps / HBM_PEAK_GBPS},
            "step": {"achieved_GBps": step_gbps, "frac": step_gbps / HBM_PEAK_GBPS,
                     "kernel_ms": avg_pos_ms + avg_neg_ms},
        },
        "host_prep_s": t_prep,
    }

    if evaluating:
        out["config"]["mode"] = "eval"
        out["roofline"]["traffic"] = None
    if args.max_workgroups > 0:
        out["config"]["max_workgroups"] = args.max_workgroups
    if bf16:
        out["config"]["storage"] = "bf16"
        out["config"]["hot_words"] = load_library().w2v_get_bf16_hot_words()
        out["config"]["operators"] = "word2vecPosBf16+word2vecNegBf16"
    if args.hot_mode != -1:
        out["config"]["hot_update_mode"] = args.hot_mode
    if args.rare_mode != -1:
        out["config"]["rare_update_mode"] = args.rare_mode
    if args.ordered_mode != -1:
        out["config"]["ordered_mode"] = args.ordered_mode
    if args.tokens > 0:
        out["roofline"]["traffic"] = None       # measured at the workload's own size only
    if args.wsample > 0.0:
        out["config"]["wsample"] = args.wsample
        out["roofline"]["traffic"] = None
    if MM:
        out["config"]["parts"] = len(MM) // 2
        out["config"]["slices"] = args.slices
        out["config"]["head_words"] = args.head
        out["config"]["operators"] = "word2vecPosSlice+word2vecNegSlice"
        out["roofline"]["traffic"] = None
    if not evaluating and not MM and not bf16 and not args.no_pcie:
        # The same step with the five index arrays uploaded from pinned host memory first (what a
        # caller that builds them on the host pays); serialised with the kernels, not overlapped.
        # Reported beside the headline value, never as it.
        pinned = [{k: torch.from_numpy(mb[k]).pin_memory() for k in ("W", "LB", "UB", "WA", "WB")}
                  for mb in host_mbs]
        k2 = min(K, 10)
        for rep in range(2):                       # first repetition warms the copies up
            synchronize()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for s_ in range(k2):
                src, dst = pinned[s_ % ndistinct], dev_mbs[s_ % ndistinct]
                for key in dst:
                    dst[key].copy_(src[key], non_blocking=True)
                step(Wm + K + s_)
            synchronize()
            torch.cuda.synchronize()
            t_h2d = time.perf_counter() - t1
        upload = sum(v.numel() * 4 for v in pinned[0].values())
        out["pcie_inclusive"] = {"value": k2 * n / t_h2d, "unit": "words/s",
                                 "ms_per_step": 1e3 * t_h2d / k2, "steps": k2,
                                 "uploaded_bytes_per_step": upload}
        assert bool(torch.isfinite(A).all()) and bool(torch.isfinite(B).all()), "tables diverged"

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
                       "step_algorithmic_over_copy": step_gbps / copy_gbps}

    if not args.no_cpu_baseline and bf16:
        cpu_wps, cpu_dt, m = cpu_baseline_bf16(cfg, host_mbs[0], args.lrate,
                                               args.lrate / cfg["nneg"], args.vexp, 300_000)
        out["cpu_baseline"] = {"value": cpu_wps, "unit": "words/s", "cores": 1, "kind": "port",
                               "sample": "the first %d tokens of one minibatch and their groups, "
                                         "pos+neg, single-threaded bf16 oracle, %.1f s wall"
                                         % (m, cpu_dt),
                               "gpu_over_cpu": words_per_s / cpu_wps}
    elif not args.no_cpu_baseline and not evaluating:
        threads = host_threads()
        sample = host_mbs[:3]
        cpu_wps, cpu_dt = cpu_baseline(cfg, sample, args.lrate, args.lrate / cfg["nneg"],
                                       args.vexp, threads)
        out["cpu_baseline"] = {"value": cpu_wps, "unit": "words/s", "cores": threads,
                               "kind": "port",
                               "sample": "%d full minibatches (%d tokens each) of the same "
                                         "workload, pos+neg, %.1f s wall" % (len(sample), n, cpu_dt),
                               "gpu_over_cpu": words_per_s / cpu_wps}

    print(json.dumps(out))


if __name__ == "__main__":
    main()
