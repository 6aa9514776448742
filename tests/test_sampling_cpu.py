"""The CPU oracle's sampler against the compiled reference's sample_token (golden tokens) and against what the
mathematics fixes (reference: GGUFModel::sample_token, torch/io/gguf_model.h:7658-7751; repetition penalty
:4926-4938; generator: function-local static std::mt19937(42), :7740)."""
import os

import numpy as np
import pytest

from prometorch_amd.testing import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_sampling.npz")


def numpy_distribution(x, temperature, top_k, top_p):
    """float64 restatement: the distribution sample_token draws from."""
    z = x.astype(np.float32) / np.float32(temperature)
    V = z.size
    if 0 < top_k < V:
        thr = np.partition(z, V - top_k)[V - top_k]           # k-th largest, duplicates counted
        z = np.where(z < thr, np.float32(-1e9), z)
    p = np.exp(z.astype(np.float64) - z.max())
    p /= p.sum()
    if top_p < 1.0:
        order = np.lexsort((np.arange(V), -p))                # descending, index breaks ties
        order = order[p[order] > 1e-10]
        csum = np.cumsum(p[order])
        n_keep = int(np.searchsorted(csum, top_p, side="left")) + 1   # first position with csum >= top_p, inclusive
        keep = np.zeros(V, bool)
        keep[order[:n_keep]] = True
        p = np.where(keep, p, 0.0)
        p /= p.sum()
    return p


def test_mt19937_known_answer_and_uniform(po):
    g = po.MT19937(5489)
    for _ in range(9999):
        g.next_u32()
    assert g.next_u32() == 4123659995           # ISO C++ [rand.predef]: 10000th value of a default mt19937
    a, b = po.MT19937(42), po.MT19937(42)
    for _ in range(1000):
        u = a.next_u32()
        r = np.float32(u) / np.float32(4294967296.0)
        r = np.nextafter(np.float32(1), np.float32(0)) if r >= 1 else r
        assert b.uniform01() == float(r)
    assert abs(po.MT19937(42).uniform01() - 0.3745401) < 1e-7


def test_sampler_matches_the_compiled_reference(po):
    want = np.load(GOLDEN)["tokens"]
    assert len(want) == len(synth.SAMPLING_CASES)
    rng = po.MT19937(42)
    for i, (vocab, kind, temperature, top_k, top_p) in enumerate(synth.SAMPLING_CASES):
        r = rng.uniform01() if temperature >= 1e-6 else 0.0     # the greedy branch returns before drawing
        tok, gap = po.sample_token(synth.sampling_logits(i), temperature, top_k, top_p, r)
        assert tok == int(want[i]), (i, kind, temperature, top_k, top_p, r, gap)


@pytest.mark.parametrize("case", range(0, 22))
def test_sampler_distribution_vs_numpy(po, case):
    vocab, kind, temperature, top_k, top_p = synth.SAMPLING_CASES[case]
    if temperature < 1e-6:
        pytest.skip("greedy")
    x = synth.sampling_logits(case)
    want = numpy_distribution(x, temperature, top_k, top_p)
    rs = np.random.default_rng(case).random(8).astype(np.float32)
    cdf = np.cumsum(want)
    for r in rs:
        tok, gap, probs = po.sample_token(x, temperature, top_k, top_p, float(r), want_probs=True)
        assert np.abs(probs - want).max() <= 2e-6
        assert abs(float(probs.astype(np.float64).sum()) - 1.0) <= 1e-4
        if 0 < top_k < vocab:
            assert int((probs > 0).sum()) <= max(top_k, int((x >= np.sort(x)[-top_k]).sum()))
        if gap > 1e-4:
            assert tok == int(np.searchsorted(cdf, r, side="left"))


def test_sampler_edges(po):
    x = synth.sampling_logits(0)
    assert po.sample_token(x, 0.8, 40, 0.9, 0.0)[0] == 0                       # cumsum >= 0 holds at index 0
    assert po.sample_token(x, 0.0, 40, 0.9, 0.5)[0] == int(np.argmax(x))        # greedy
    assert po.sample_token(x, 1e-7, 0, 1.0, 0.9)[0] == int(np.argmax(x))
    assert po.sample_token(x, 0.8, 1, 1.0, 0.99)[0] == int(np.argmax(x))        # top-1
    flat = np.zeros(16, np.float32)                                             # all tied: top-k keeps everything
    tok, gap, probs = po.sample_token(flat, 1.0, 4, 1.0, 0.51, want_probs=True)
    assert np.allclose(probs, 1 / 16) and tok == 8
    tok, gap = po.sample_token(x, 0.8, 40, 0.9, float(np.nextafter(np.float32(1), np.float32(0))))
    p = numpy_distribution(x, 0.8, 40, 0.9)
    assert tok >= int(np.nonzero(p)[0][-1])                                     # last kept token, or vocab - 1 on round-off


def test_repetition_penalty_once_per_occurrence(po):
    x = np.array([2.0, -1.0, 0.0, 3.0, -4.0, 5.0], np.float32)
    gen = [0, 1, 0, 3, 4, 4, 4, 7, -1, 2]
    got = po.repetition_penalty(x, gen, 1.1)
    want = x.copy()
    for t in gen:
        if 0 <= t < x.size:
            want[t] = want[t] / np.float32(1.1) if want[t] > 0 else want[t] * np.float32(1.1)
    assert np.array_equal(got, want)
    assert np.array_equal(po.repetition_penalty(x, gen, 1.0), x)                # penalty <= 1: untouched
    assert np.array_equal(po.repetition_penalty(x, [], 1.3), x)
