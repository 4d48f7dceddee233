"""Pins the oracle's restatement of the distribution pipeline ahead of the samplers (neural/neuralchatengine.pas:
1374-1396, 1495-1501; neural/neuraldecode.pas:4710-4754; neural/neuralvolume.pas:5335-5376) with what the mathematics
fixes: probability-domain temperature equals softmax(logits / T); the penalty cases have closed forms; the candidate
prefix is the head of the fully sorted row."""
import numpy as np

from helpers import oracle_lib as O


def softmax64(x):
    x = np.asarray(x, np.float64); e = np.exp(x - x.max()); return e / e.sum()


def test_plain_candidates_are_the_sorted_softmax_head():
    rng = np.random.default_rng(1)
    logits = (rng.standard_normal(5000) * 3).astype(np.float32)
    tok, p = O.sample_candidates(logits, 64)
    ref = softmax64(logits); order = np.argsort(-ref, kind="stable")[:64]
    np.testing.assert_array_equal(tok, order)
    np.testing.assert_allclose(p, ref[order], rtol=2e-5)
    assert np.all(np.diff(p) <= 0)
    tok_all, p_all = O.sample_candidates(logits[:50], 64)          # m larger than the vocabulary
    assert tok_all.size == 50 and abs(float(p_all.sum()) - 1) < 1e-5


def test_ties_take_the_lower_token_first():
    logits = np.zeros(40, np.float32); logits[[7, 3, 30]] = 2.0
    tok, p = O.sample_candidates(logits, 6)
    np.testing.assert_array_equal(tok, [3, 7, 30, 0, 1, 2])
    assert p[0] == p[1] == p[2] and p[3] == p[4]


def test_temperature_is_softmax_of_scaled_logits():
    rng = np.random.default_rng(2)
    logits = (rng.standard_normal(3000) * 2).astype(np.float32)
    for T in (0.5, 0.8, 1.7):
        tok, p = O.sample_candidates(logits, 32, temperature=T)
        ref = softmax64(logits.astype(np.float64) / T); order = np.argsort(-ref, kind="stable")[:32]
        np.testing.assert_array_equal(tok, order)
        np.testing.assert_allclose(p, ref[order], rtol=3e-4)
    tok, p = O.sample_candidates(logits, 4, temperature=0.0)         # clamped to 1e-6: one-hot on the arg-max
    assert tok[0] == int(np.argmax(logits)) and abs(p[0] - 1) < 1e-6 and p[1] == 0
    a = O.sample_candidates(logits, 16, temperature=1.0); b = O.sample_candidates(logits, 16)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])   # T = 1 changes nothing


def test_history_penalties_closed_forms():
    rng = np.random.default_rng(3)
    n = 400
    logits = rng.standard_normal(n).astype(np.float32)
    hist = [5, 9, 9, 9, 200, n + 10, -1]                             # ids outside the row are ignored
    base = softmax64(logits)
    for rep, freq, pres in ((1.3, 0.0, 0.0), (1.0, 0.4, 0.0), (1.0, 0.0, 0.7), (1.2, 0.1, 0.3)):
        want = base.copy()
        for t, c in ((5, 1), (9, 3), (200, 1)):
            want[t] = want[t] ** rep * np.exp(-(freq * c + pres))
        want /= want.sum()
        tok, p = O.sample_candidates(logits, n, history=hist, repetition=rep, frequency=freq, presence=pres)
        got = np.zeros(n); got[tok] = p
        np.testing.assert_allclose(got, want, rtol=3e-5, atol=1e-9)
        assert want[9] < base[9]                                     # a repeated token loses mass
    # all knobs at their defaults: bit-for-bit the plain row even with a history
    a = O.sample_candidates(logits, 50, history=hist); b = O.sample_candidates(logits, 50)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
