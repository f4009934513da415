"""Host-side mirror of the minibatch step of BIDMach.networks.Word2Vec around the HIP operators.

What is mirrored (src/main/scala/BIDMach/networks/Word2Vec.scala of the reference):
  Options         the option names and defaults of Word2Vec.Opts (:574-591) plus the borrowed
                  dim (models/Model.scala:537), lrate/texp (updaters/Grad.scala:242-243) and
                  vexp (updaters/ADAGrad.scala:158)
  init            model matrices: modelmats(0) ~ (U[0,1) - 0.5)/dim, modelmats(1) = 0 (:112-117)
  wordMats        OOV and subsampling to -1, random window bounds clipped at sentence
                  boundaries, compaction and permutation of the context words, negatives by the
                  closed form min(V-1, floor(V * u**(1/(1-wexpt)))) (:214-364)
  dobatch         learning-rate decay lrate * (pos/firstPos)**(-texp), then procPositives and
                  procNegatives with A = modelmats(1), B = modelmats(0) (:167-190, :366-402)
  evalbatch       (epos + eneg/nneg) / #context words (:192-212, :469-523)
  sliced models   nSlices / iSlice / nHeadTerms / maxArraySize / dualMode / doHead: the packed,
                  multi-part list of model matrices of :100-131 and the dispatch to the Slice
                  operators when nSlices != 1 or the model needs more than one part (:178-187,
                  :196-207).  The reference runs those on the CPU only; here every part is a
                  device allocation and the library's device Slice operators are used.
  save / load     the checkpoint layout of Model.save / Model.load (models/Model.scala:245-315):
                  `options.json` and one `modelmat%02d.lz4` per model matrix under a path prefix
                  (the Java-serialised `options.ser` is not written)
  train           Learner.nextPass' loop: minibatch istep is scored instead of trained on when
                  (istep - 1) % evalStep == 0, and so is the last one of a pass
                  (Learner.scala:187-222, evalStep default 11 at :1064)

The arithmetic runs in the HIP library through bidmach_amd.cumach.CUMACH.  The index arrays are
prepared either on the device (w2v_wordmats, the counterpart of the reference's GPU branch of
wordMats, :241-270; the default on a GPU) or with numpy on the host (like the reference's CPU
branch `getnegs`, :280-364); this module owns the device buffers (torch tensors: plumbing).
Random draws come from numpy or from the library's counter-based generator, not from BIDMat, so
a run reproduces the reference's distributions and array contracts, not its random stream.
"""
import math

import numpy as np

from . import corpus
from .cumach import CUMACH, check, wordmats as _device_wordmats


class Options:
    """Word2Vec.Opts with the reference's defaults."""

    def __init__(self, **kw):
        self.nskip = 5
        self.nneg = 5
        self.nreuse = 5
        self.vocabSize = 100000
        self.wexpt = 0.75
        self.wsample = 1e-4
        self.headlen = 10000
        self.iflip = False
        self.eqPosNeg = False
        self.dim = 256
        self.lrate = 1.0
        self.texp = 0.5
        self.vexp = 0.5
        self.batchSize = 100000
        self.evalStep = 11
        self.seed = 0
        self.maxArraySize = 2047 * 1024 * 1024
        self.nHeadTerms = 0
        self.nSlices = 1
        self.iSlice = 0
        self.dualMode = False
        self.doHead = 1
        self.deviceWordMats = True   # build the index arrays on the GPU when the model is on one
        # element type of the model on the device: "fp32" (the reference's), or "bf16" (no
        # counterpart in the reference: fp32 arithmetic, stochastic-rounded write-back, half the
        # memory; single-table models only)
        self.storage = "fp32"
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("unknown Word2Vec option %r" % k)
            setattr(self, k, v)


class Word2Vec:
    def __init__(self, opts=None, device="cuda:0"):
        self.opts = opts or Options()
        self.device = device
        self.modelmats = None
        self.firstPos = -1
        self.ncols = None
        self.rng = np.random.Generator(np.random.PCG64(self.opts.seed))
        self._ret = None
        self._call = 0
        self._wm = None
        self._wm_last = None
        self._prep = None

    # ---- Word2Vec.init ------------------------------------------------------------------
    def init(self, ncols=None, modelmats=None):
        """modelmats: optional host arrays in the layout of the reference's list, B table of part
        m at 2m (+2 with a dual-mode list), A table at 2m+1; each (columns, dim) in C order."""
        import torch
        o = self.opts
        self.ncols = ncols if ncols is not None else o.batchSize
        self.maxCols = o.maxArraySize // o.dim
        # columns this worker holds: the head and its share of the tail (:106)
        actual = o.nHeadTerms + 1 + (o.vocabSize - o.nHeadTerms - 1) // o.nSlices
        self.nmmats = 1 + (actual - 1) // self.maxCols
        self._dual = bool(o.dualMode) and self.nmmats > 1
        if modelmats is None:
            def fresh(cols):
                m0 = (self.rng.random((cols, o.dim), dtype=np.float32) - np.float32(0.5)) \
                    / np.float32(o.dim)
                return m0, np.zeros((cols, o.dim), dtype=np.float32)
            if self.nmmats == 1:
                modelmats = list(fresh(actual))
            else:
                modelmats = []
                for i in range(self.nmmats):
                    last = i == self.nmmats - 1
                    modelmats += list(fresh(actual - i * self.maxCols if last else self.maxCols))
                if self._dual:                         # the device copy of the first part (:128-131)
                    modelmats = [modelmats[0].copy(), modelmats[1].copy()] + modelmats
        # (columns, dim) C-order == dim x columns column-major, the layout the operators take
        self.modelmats = [torch.from_numpy(np.ascontiguousarray(m)).to(self.device)
                          for m in modelmats]
        if o.storage == "bf16":
            if self._sliced():
                raise ValueError("bf16 storage takes a single-table model (nSlices = 1, one part)")
            from .cumach import f32_to_bf16
            narrow = []
            for m in self.modelmats:
                h = torch.empty(m.shape, dtype=torch.bfloat16, device=self.device)
                f32_to_bf16(m.numel(), m, h)
                narrow.append(h)
            self.modelmats = narrow
        elif o.storage != "fp32":
            raise ValueError("unknown storage %r" % (o.storage,))
        self._seed16 = 0
        self.expt = 1.0 / (1.0 - o.wexpt)
        self.salpha = o.wsample * math.log(o.vocabSize)
        self._ret = torch.zeros(2, dtype=torch.float32, device=self.device)
        self._ret64 = torch.zeros(2, dtype=torch.float64, device=self.device)
        self.firstPos = -1

    def _sliced(self):
        return self.opts.nSlices != 1 or self.nmmats != 1

    # ---- Word2Vec.wordMats (host branch) ------------------------------------------------
    def wordMats(self, mats):
        """mats: int32 array 2 x N (row 0 word ids, row 1 sentence ids; swapped if iflip).
        Returns host arrays (words, lb, ub, trandwords, contextwords)."""
        o = self.opts
        wordsens = np.asarray(mats)
        words = (wordsens[1] if o.iflip else wordsens[0]).astype(np.int32)
        sentence = wordsens[0] if o.iflip else wordsens[1]
        n = words.shape[0]
        wgood = words < o.vocabSize
        wrat = (words.astype(np.float32) + np.float32(1.0)) * np.float32(self.salpha)
        wrat = np.sqrt(wrat) + wrat
        wgood &= self.rng.random(n, dtype=np.float32) < wrat
        words = np.where(wgood, words, -1).astype(np.int32)

        ubrand = np.minimum(o.nskip, (self.rng.random(n, dtype=np.float32) * o.nskip)
                            .astype(np.int32) + 1).astype(np.int32)
        lbrand = -ubrand
        # nearest sentence boundaries: position inside the run of equal sentence ids
        idx = np.arange(n, dtype=np.int64)
        change = np.flatnonzero(sentence[1:] != sentence[:-1]) + 1
        starts = np.concatenate(([0], change))
        ends = np.concatenate((change, [n])) - 1
        seg = np.searchsorted(starts, idx, side="right") - 1
        lb = np.maximum(lbrand, (starts[seg] - idx)).astype(np.int32)
        ub = np.minimum(ubrand, (ends[seg] - idx)).astype(np.int32)

        ctx = corpus.valid_context_words(words, lb, ub)
        ngroups = ctx.shape[0] // o.nreuse
        ctx = self.rng.permutation(ctx)[: ngroups * o.nreuse].astype(np.int32)
        u = self.rng.random(ngroups * o.nneg, dtype=np.float32)
        negs = np.minimum(o.vocabSize - 1,
                          (o.vocabSize * np.power(u, np.float32(self.expt))).astype(np.int64))
        return words, lb, ub, negs.astype(np.int32), ctx

    def _dev(self, x):
        import torch
        return torch.from_numpy(np.ascontiguousarray(x)).to(self.device)

    # ---- Word2Vec.wordMats (device branch) ----------------------------------------------
    def wordMatsDevice(self, mats):
        """Same outputs as wordMats, as device tensors, built by the library on the GPU.

        The upload and the preprocessing kernels run on a stream of their own, so that they are
        not queued behind the update kernels of the previous minibatch, which the host has only
        enqueued: the host prepares minibatch i+1 while the device still trains on minibatch i.
        The outputs alternate between two sets of buffers; a set is written again only after the
        update kernels that read it have finished (_release_index_arrays records that point), so
        the tensors returned here stay valid until the call after next."""
        import torch
        from .cumach import load_library
        o = self.opts
        wordsens = np.asarray(mats)
        n = wordsens.shape[1]
        cap = 2 * o.nskip * n
        if self._wm is None or self._wm[0]["n"] != n:
            def ibuf(k):
                return torch.empty(max(k, 1), dtype=torch.int32, device=self.device)
            self._wm = [dict(n=n, words=ibuf(n), lb=ibuf(n), ub=ibuf(n), ctx=ibuf(cap),
                             negs=ibuf(o.nneg * (cap // o.nreuse + 1)), counts=ibuf(2),
                             free=None) for _ in range(2)]
            self._prep = torch.cuda.Stream(device=self.device)
        self._call += 1
        b = self._wm[self._call % 2]
        self._wm_last = b
        lib = load_library()
        launch_stream = lib.w2v_get_stream()
        with torch.cuda.stream(self._prep):
            if b["free"] is not None:
                self._prep.wait_event(b["free"])
            # the data source's 2 x n matrix, column-major: (word, sentence) pairs interleaved (no
            # copy on the host if it already is, as matio.loadIMat returns it)
            dmats = torch.from_numpy(np.ascontiguousarray(wordsens.T, dtype=np.int32)).to(
                self.device)
            lib.w2v_set_stream(self._prep.cuda_stream)
            try:
                npairs, ngroups = _device_wordmats(n, dmats, o.iflip, o.vocabSize, o.nskip, o.nneg,
                                                   o.nreuse, float(np.float32(self.salpha)),
                                                   o.wexpt, o.seed, self._call, b["words"],
                                                   b["lb"], b["ub"], b["negs"], b["ctx"],
                                                   b["counts"])
            finally:
                lib.w2v_set_stream(launch_stream)
        # w2v_wordmats has waited for its stream: the outputs are complete, whichever stream reads
        # them next
        return (b["words"], b["lb"], b["ub"], b["negs"][:ngroups * o.nneg],
                b["ctx"][:ngroups * o.nreuse])

    def _release_index_arrays(self):
        """Marks the point on the launch stream after which the buffers of the last
        wordMatsDevice call may be overwritten (everything enqueued so far has read them)."""
        import torch
        b = getattr(self, "_wm_last", None)
        if b is None:
            return
        if b["free"] is None:
            b["free"] = torch.cuda.Event()
        from .cumach import load_library
        stream = load_library().w2v_get_stream()
        b["free"].record(torch.cuda.ExternalStream(stream, device=self.device) if stream
                         else torch.cuda.default_stream(self.device))

    def _index_arrays(self, mats):
        """(words, lb, ub, trandwords, contextwords) on the model's device."""
        if self.opts.deviceWordMats and str(self.device).startswith("cuda"):
            return self.wordMatsDevice(mats)
        return tuple(self._dev(x) for x in self.wordMats(mats))

    # ---- the four dispatchers (Word2Vec.scala:366-402, 469-523) --------------------------
    # The update calls are enqueued without waiting (the Async entry points): the host then
    # prepares the next minibatch while the device works.  Everything that reads the model
    # afterwards (the scoring calls, torch on the same stream, synchronize()) is ordered behind
    # them.
    def procPositives(self, nskip, words, lb, ub, model1, model2, lrate, vexp):
        nrows = model1.shape[1]
        if self.opts.storage == "bf16":
            check(CUMACH.word2vecPosBf16Async(nrows, words.shape[0], nskip, words, lb, ub, model1,
                                              model2, lrate, vexp, self._next_seed16()),
                  "word2vecPosBf16")
            return
        check(CUMACH.word2vecPosAsync(nrows, words.shape[0], nskip, words, lb, ub, model1, model2,
                                      lrate, vexp), "word2vecPos")

    def procNegatives(self, nwa, nwb, wordsa, wordsb, modela, modelb, lrate, vexp):
        nrows = modela.shape[1]
        if self.opts.storage == "bf16":
            check(CUMACH.word2vecNegBf16Async(nrows, wordsa.shape[0] // nwa, nwa, nwb, wordsa,
                                              wordsb, modela, modelb, lrate, vexp,
                                              self._next_seed16()),
                  "word2vecNegBf16")
            return
        check(CUMACH.word2vecNegAsync(nrows, wordsa.shape[0] // nwa, nwa, nwb, wordsa, wordsb,
                                      modela, modelb, lrate, vexp), "word2vecNeg")

    def _next_seed16(self):
        """A new key for the stochastic rounding of every bf16 update call."""
        self._seed16 += 1
        return ((int(self.opts.seed) & 0xFFFFFFFF) << 32) | (self._seed16 & 0xFFFFFFFF)

    def synchronize(self):
        """Waits for the enqueued updates and raises if any of them failed."""
        from .cumach import synchronize
        synchronize()

    def evalPositives(self, nskip, words, lb, ub, model1, model2):
        nrows = model1.shape[1]
        if self.opts.storage == "bf16":
            self._ret64[0:1].zero_()
            check(CUMACH.word2vecEvalPosBf16(nrows, words.shape[0], nskip, words, lb, ub, model1,
                                             model2, self._ret64[0:1]), "word2vecEvalPosBf16")
            return float(self._ret64[0].item())
        self._ret[0:1].zero_()                                  # retEvalPos.clear (:476)
        check(CUMACH.word2vecEvalPos(nrows, words.shape[0], nskip, words, lb, ub, model1, model2,
                                     self._ret[0:1]), "word2vecEvalPos")
        return float(self._ret[0].item())

    def evalNegatives(self, nwa, nwb, wordsa, wordsb, modela, modelb):
        nrows = modela.shape[1]
        if self.opts.storage == "bf16":
            self._ret64[1:2].zero_()
            check(CUMACH.word2vecEvalNegBf16(nrows, wordsa.shape[0] // nwa, nwa, nwb, wordsa,
                                             wordsb, modela, modelb, self._ret64[1:2]),
                  "word2vecEvalNegBf16")
            return float(self._ret64[1].item())
        self._ret[1:2].zero_()
        check(CUMACH.word2vecEvalNeg(nrows, wordsa.shape[0] // nwa, nwa, nwb, wordsa, wordsb,
                                     modela, modelb, self._ret[1:2]), "word2vecEvalNeg")
        return float(self._ret[1].item())

    # ---- the Slice dispatchers (Word2Vec.scala:404-467, 491-534) ------------------------
    def _slice_args(self):
        o = self.opts
        return (o.iSlice, o.nSlices, self.maxCols, o.nHeadTerms, self._dual)

    def procPositivesSlice(self, nskip, words, lb, ub, modelmats, lrate, vexp):
        check(CUMACH.word2vecPosSlice(self.opts.dim, words.shape[0], nskip, words, lb, ub,
                                      modelmats, lrate, vexp, *self._slice_args(),
                                      self.opts.doHead), "word2vecPosSlice")

    def procNegativesSlice(self, nwa, nwb, wordsa, wordsb, modelmats, lrate, vexp):
        check(CUMACH.word2vecNegSlice(self.opts.dim, wordsa.shape[0] // nwa, nwa, nwb, wordsa,
                                      wordsb, modelmats, lrate, vexp, *self._slice_args(),
                                      self.opts.doHead), "word2vecNegSlice")

    def evalPositivesSlice(self, nskip, words, lb, ub, modelmats):
        self._ret64[0:1].zero_()
        check(CUMACH.word2vecEvalPosSlice(self.opts.dim, words.shape[0], nskip, words, lb, ub,
                                          modelmats, *self._slice_args(), self._ret64[0:1]),
              "word2vecEvalPosSlice")
        return float(self._ret64[0].item())

    def evalNegativesSlice(self, nwa, nwb, wordsa, wordsb, modelmats):
        self._ret64[1:2].zero_()
        check(CUMACH.word2vecEvalNegSlice(self.opts.dim, wordsa.shape[0] // nwa, nwa, nwb, wordsa,
                                          wordsb, modelmats, *self._slice_args(),
                                          self._ret64[1:2]), "word2vecEvalNegSlice")
        return float(self._ret64[1].item())

    # ---- Word2Vec.dobatch / evalbatch ---------------------------------------------------
    def dobatch(self, mats, ipass, pos):
        o = self.opts
        if np.asarray(mats).shape[1] != self.ncols:
            return                                              # odd-sized minibatch: skipped (:169)
        if self.firstPos < 0:
            self.firstPos = pos
        nsteps = float(pos) / float(self.firstPos)
        lrate = float(o.lrate) * math.pow(nsteps, -o.texp)
        words, lb, ub, trandwords, goodwords = self._index_arrays(mats)
        lrpos = lrate
        lrneg = lrpos if o.eqPosNeg else lrpos / o.nneg
        if self._sliced():
            self.procPositivesSlice(o.nskip, words, lb, ub, self.modelmats, lrpos, o.vexp)
            if goodwords.shape[0] > 0:
                self.procNegativesSlice(o.nneg, o.nreuse, trandwords, goodwords, self.modelmats,
                                        lrneg, o.vexp)
        else:
            self.procPositives(o.nskip, words, lb, ub, self.modelmats[1], self.modelmats[0], lrpos,
                               o.vexp)
            if goodwords.shape[0] > 0:
                self.procNegatives(o.nneg, o.nreuse, trandwords, goodwords, self.modelmats[1],
                                   self.modelmats[0], lrneg, o.vexp)
        self._release_index_arrays()

    def evalbatch(self, mats, ipass, pos):
        o = self.opts
        if np.asarray(mats).shape[1] != self.ncols:
            return 0.0                                          # row(0) (:211)
        words, lb, ub, trandwords, goodwords = self._index_arrays(mats)
        if goodwords.shape[0] == 0:
            return 0.0
        if self._sliced():
            epos = self.evalPositivesSlice(o.nskip, words, lb, ub, self.modelmats)
            eneg = self.evalNegativesSlice(o.nneg, o.nreuse, trandwords, goodwords, self.modelmats)
        else:
            epos = self.evalPositives(o.nskip, words, lb, ub, self.modelmats[1], self.modelmats[0])
            eneg = self.evalNegatives(o.nneg, o.nreuse, trandwords, goodwords, self.modelmats[1],
                                      self.modelmats[0])
        return (epos + eneg / (1 if o.eqPosNeg else o.nneg)) / goodwords.shape[0]

    # ---- Model.save / Model.load (models/Model.scala:245-315) ---------------------------
    def save(self, fname):
        """Writes `fname + "options.json"` and `fname + "modelmat%02d.lz4"` for every model matrix
        (BIDMat dense-matrix files, dim x columns, LZ4 block stream).  `fname` is a path prefix,
        normally a directory name ending in a separator, created if needed."""
        import json
        import os
        from . import matio
        parent = os.path.dirname(fname + "options.json")
        if parent:
            os.makedirs(parent, exist_ok=True)
        with open(fname + "options.json", "w") as f:
            json.dump({k: v for k, v in vars(self.opts).items()}, f, indent=1, sort_keys=True)
        for i, m in enumerate(self.modelmats):
            # a bf16 model is written widened: the files hold fp32, as the reference's do
            matio.saveMat(fname + "modelmat%02d.lz4" % i, m.float().cpu().numpy().T)

    def load(self, fname, useJson=True):
        """Reads the model matrices `fname + "modelmat%02d.lz4"` (as many as exist) and, with
        useJson, the options; a model loaded this way is not re-initialised (`refresh = false`,
        Model.scala:314)."""
        import json
        import os
        from . import matio
        if useJson and os.path.exists(fname + "options.json"):
            with open(fname + "options.json") as f:
                for k, v in json.load(f).items():
                    if hasattr(self.opts, k):
                        setattr(self.opts, k, v)
        mats = []
        while os.path.exists(fname + "modelmat%02d.lz4" % len(mats)):
            m = matio.loadFMat(fname + "modelmat%02d.lz4" % len(mats))
            if m.shape[0] != self.opts.dim:
                raise ValueError("modelmat%02d has %d rows, the model's dim is %d"
                                 % (len(mats), m.shape[0], self.opts.dim))
            mats.append(np.ascontiguousarray(m.T))
        if len(mats) < 2 or len(mats) % 2:
            raise ValueError("no model matrices under %r" % fname)
        self.init(self.ncols, modelmats=mats)

    # ---- Learner.nextPass, reduced to what Word2Vec uses (no updater, no mixins) ---------
    def train(self, stream, npasses=1):
        """stream: int32 array 2 x total.  Returns [(position, held-out score)], one entry per
        evalStep-th minibatch, as Learner collects in `results` (Learner.scala:276)."""
        o = self.opts
        stream = np.asarray(stream)
        if self.modelmats is None:
            self.init(o.batchSize)
        results = []
        here = 0
        for ipass in range(npasses):
            istep = 0
            starts = list(range(0, stream.shape[1] - o.batchSize + 1, o.batchSize))
            for s in starts:
                mats = stream[:, s:s + o.batchSize]
                here += o.batchSize
                last = s == starts[-1]
                if (istep >= 1 and (istep - 1) % o.evalStep == 0) or (istep > 0 and last):
                    results.append((here, self.evalbatch(mats, ipass, here)))
                else:
                    self.dobatch(mats, ipass, here)
                istep += 1
        self.synchronize()
        return results
