"""Minibatch preprocessing: the numpy twin's generator against the published Philox4x32-10
known answers and the reference's rules (CPU), and the device code against the twin, bit for bit
(GPU).  The reference's own random stream (BIDMat) cannot be reproduced: parity of the draws is
unpinned, parity of the rules is what these tests hold."""
import math

import numpy as np
import pytest

from bidmach_amd import corpus
from oracle import wordmats_ref as ref


def test_philox_known_answers():
    # Random123 kat_vectors for philox4x32-10, first output word
    assert int(ref.philox_word0(np.array([0], np.uint64), 0, 0, 0)[0]) == 0x6627E8D5
    assert int(ref.philox_word0(np.array([0xFFFFFFFFFFFFFFFF], np.uint64), 0xFFFFFFFF, 0xFFFFFFFF,
                                0xFFFFFFFFFFFFFFFF)[0]) == 0x408F276D
    # counter {243f6a88, 85a308d3, 13198a2e, 03707344}, key {a4093822, 299f31d0}
    idx = np.array([(0x85A308D3 << 32) | 0x243F6A88], np.uint64)
    assert int(ref.philox_word0(idx, 0x13198A2E, 0x03707344, (0x299F31D0 << 32) | 0xA4093822)[0]) \
        == 0xD16CFE09


def make_mats(n, vocab, seed):
    rng = np.random.default_rng(seed)
    w = corpus.zipf_stream(n, vocab, 1.0, seed=seed)
    w[rng.random(n) < 0.02] = vocab + 3
    sent = np.cumsum(rng.random(n) < 0.06).astype(np.int32)
    return w.astype(np.int32), sent


def test_twin_follows_the_reference_rules():
    V, n, nskip, nneg, nreuse = 3000, 6000, 5, 5, 5
    w, sent = make_mats(n, V, 1)
    words, lb, ub, negs, ctx, npairs, G = ref.wordmats(w, sent, V, nskip, nneg, nreuse,
                                                       1e-3 * math.log(V), 0.75, 7, 0)
    kept = words >= 0
    assert np.array_equal(words[kept], w[kept]) and not np.any(kept & (w >= V))
    idx = np.arange(n)
    assert np.all(lb <= 0) and np.all(ub >= 0) and np.all(-lb <= nskip) and np.all(ub <= nskip)
    assert np.all(sent[idx + lb] == sent) and np.all(sent[idx + ub] == sent)
    # away from sentence boundaries the window is symmetric and uniform on 1..nskip
    inner = (sent[np.clip(idx - nskip, 0, n - 1)] == sent) & (sent[np.clip(idx + nskip, 0, n - 1)] == sent) \
        & (idx >= nskip) & (idx < n - nskip)
    assert np.array_equal(lb[inner], -ub[inner])
    assert set(np.unique(ub[inner])) == set(range(1, nskip + 1))
    want_pairs, _ = corpus.count_pairs(words, lb, ub)
    assert npairs == want_pairs and G == npairs // nreuse
    assert np.array_equal(np.sort(ctx), np.sort(corpus.valid_context_words(words, lb, ub)))
    assert negs.shape == (G * nneg,) and negs.min() >= 0 and negs.max() < V
    for k in (30, 300):
        assert float((negs < k).mean()) == pytest.approx((k / V) ** 0.25, abs=0.02)


@pytest.mark.gpu
@pytest.mark.parametrize("n,V,nskip,nneg,nreuse,wsample,wexpt,iflip", [
    (20000, 5000, 5, 5, 5, 1e-3, 0.75, False),
    (7001, 800, 10, 15, 5, 1e-2, 0.75, True),
    (3000, 100, 2, 3, 4, 1.0, 0.5, False),
    (64, 10, 5, 5, 5, 1.0, 0.75, False),
])
def test_device_wordmats_equals_twin(n, V, nskip, nneg, nreuse, wsample, wexpt, iflip):
    import torch
    from bidmach_amd.cumach import wordmats
    w, sent = make_mats(n, V, n)
    rows = (sent, w) if iflip else (w, sent)
    mats = np.stack(rows, axis=1).astype(np.int32)          # 2 x n column-major = n x 2 C-order
    salpha = np.float32(wsample * math.log(V))
    seed, call = 0x1234567890ABCDEF, 17
    want = ref.wordmats(w, sent, V, nskip, nneg, nreuse, salpha, wexpt, seed, call)

    def ibuf(k):
        return torch.full((max(k, 1),), -7, dtype=torch.int32, device="cuda")

    cap = 2 * nskip * n
    d_words, d_lb, d_ub = ibuf(n), ibuf(n), ibuf(n)
    d_negs, d_ctx, d_counts = ibuf(nneg * (cap // nreuse + 1)), ibuf(cap), ibuf(2)
    npairs, G = wordmats(n, torch.from_numpy(mats).cuda(), iflip, V, nskip, nneg, nreuse,
                         float(salpha), wexpt, seed, call, d_words, d_lb, d_ub, d_negs, d_ctx,
                         d_counts)
    assert (npairs, G) == (want[5], want[6])
    assert d_counts.cpu().tolist() == [npairs, G]
    assert np.array_equal(d_words.cpu().numpy(), want[0])
    assert np.array_equal(d_lb.cpu().numpy(), want[1])
    assert np.array_equal(d_ub.cpu().numpy(), want[2])
    assert np.array_equal(d_ctx.cpu().numpy()[:npairs], want[4])
    assert np.array_equal(d_negs.cpu().numpy()[:G * nneg], want[3])


@pytest.mark.gpu
def test_device_wordmats_empty_and_all_dropped():
    import torch
    from bidmach_amd.cumach import wordmats
    z = torch.zeros(16, dtype=torch.int32, device="cuda")
    counts = torch.full((2,), 5, dtype=torch.int32, device="cuda")
    assert wordmats(0, z, False, 10, 5, 5, 5, 1.0, 0.75, 1, 0, z, z, z, z, z, counts) == (0, 0)
    assert counts.cpu().tolist() == [0, 0]
    n = 8
    mats = torch.full((n, 2), 99, dtype=torch.int32, device="cuda")    # every word out of vocabulary
    words = torch.zeros(n, dtype=torch.int32, device="cuda")
    lb, ub = torch.zeros_like(words), torch.zeros_like(words)
    ctx = torch.zeros(2 * 5 * n, dtype=torch.int32, device="cuda")
    assert wordmats(n, mats, False, 10, 5, 5, 5, 1.0, 0.75, 1, 0, words, lb, ub, z, ctx,
                    counts) == (0, 0)
    assert words.cpu().tolist() == [-1] * n
