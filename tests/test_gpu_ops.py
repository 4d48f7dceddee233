"""Elementwise layer ops on the device against the oracle restatements of the reference kernels."""
import ctypes as C

import numpy as np
import pytest

from helpers import oracle_lib as O

pytestmark = pytest.mark.gpu


def test_rmsnorm():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(0)
    for n, t in ((8, 1), (576, 3), (3584, 2), (5120, 1)):
        x = rng.standard_normal((t, n)).astype(np.float32); g = rng.standard_normal(n).astype(np.float32)
        y = np.empty_like(x)
        cai.check(cai.load().cai_rmsnorm(x.ctypes.data, g.ctypes.data, n, t, 1e-6, y.ctypes.data, 0))
        want = np.empty_like(x)
        for i in range(t):
            O.lib().orc_rmsnorm(x[i].ctypes.data, g.ctypes.data, n, 1e-6, want[i].ctypes.data)
        assert np.max(np.abs(y - want)) < 2e-6 * np.max(np.abs(want))


@pytest.mark.parametrize("pos", [0, 1, 17, 511, 8319, 32767, 65535, 131071])   # (angles up to 131071 rad: the fp32 product of the reference, accurate sine / cosine)
@pytest.mark.parametrize("base,hd", [(10000.0, 64), (1e6, 128), (10000.0, 4)])
def test_rope_interleaved(pos, base, hd):
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(pos)
    heads = 5
    x = rng.standard_normal(heads * hd).astype(np.float32)
    want = x.copy(); th = np.empty(hd // 2, np.float32)
    O.lib().orc_rope_thetas(base, hd, th.ctypes.data)
    O.lib().orc_rope_interleaved(want.ctypes.data, heads, hd, pos, th.ctypes.data)
    got = x.copy()
    cai.check(cai.load().cai_rope(got.ctypes.data, heads, hd, pos, base, 0))
    assert np.max(np.abs(got - want)) < 2e-6
    # rotation preserves pair norms
    assert np.allclose((got.reshape(-1, 2) ** 2).sum(1), (x.reshape(-1, 2) ** 2).sum(1), rtol=1e-5)


def test_swiglu():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((2, 2 * 1000)) * 4).astype(np.float32)
    x[0, 1000] = -90.0; x[0, 1001] = 90.0   # both sigmoid branches at the extremes
    y = np.empty((2, 1000), np.float32); want = np.empty_like(y)
    cai.check(cai.load().cai_swiglu(x.ctypes.data, 1000, 2, y.ctypes.data, 0))
    for i in range(2):
        O.lib().orc_swiglu(x[i].ctypes.data, 1000, want[i].ctypes.data)
    assert np.max(np.abs(y - want)) < 1e-5 * max(1, np.max(np.abs(want)))


def test_argmax_lowest_index_on_ties():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(4)
    for n in (1, 11, 1024, 152064):
        x = rng.standard_normal(n).astype(np.float32)
        if n > 10:
            x[[7, n - 1, n // 2]] = 99.0
        idx = C.c_int32()
        cai.check(cai.load().cai_argmax(x.ctypes.data, n, C.byref(idx), 0))
        assert idx.value == O.lib().orc_argmax(x.ctypes.data, n)


def test_router_softmax_topk():
    from helpers.device import dev
    cai = dev()
    # reference known answer (tests/TestNeuralNumerical.pas:74997-75042) through softmax-free probabilities
    rng = np.random.default_rng(5)
    for n, k, renorm in ((4, 2, 1), (64, 8, 0), (64, 8, 1), (7, 7, 1)):
        logits = rng.standard_normal(n).astype(np.float32) * 2
        e = np.empty(k, np.int32); g = np.empty(k, np.float32)
        cai.check(cai.load().cai_router_topk(logits.ctypes.data, n, k, renorm, e.ctypes.data, g.ctypes.data, 0))
        p = np.empty(n, np.float32); O.lib().orc_softmax(logits.ctypes.data, n, p.ctypes.data)
        gw = np.zeros(n, np.float32); iw = np.zeros(k, np.int32)
        O.lib().orc_topk_gate(p.ctypes.data, n, k, renorm, gw.ctypes.data, iw.ctypes.data)
        assert list(e) == list(iw)
        assert np.allclose(g, gw[iw], rtol=1e-5, atol=1e-7)
    # the known answer itself: probabilities (0.5,0.1,0.3,0.1) <-> logits log(p)
    logits = np.log(np.array([0.5, 0.1, 0.3, 0.1], np.float32))
    e = np.empty(2, np.int32); g = np.empty(2, np.float32)
    cai.check(cai.load().cai_router_topk(logits.ctypes.data, 4, 2, 1, e.ctypes.data, g.ctypes.data, 0))
    assert list(e) == [0, 2] and np.allclose(g, [0.625, 0.375], atol=1e-5)


@pytest.mark.parametrize("n,k", [(64, 8), (16, 4), (200, 8), (512, 64)])
def test_router_selection_stays_inside_the_bank_on_non_finite_logits(n, k):
    """A poisoned activation row reaches the router as NaN logits.  The selection must still be k DISTINCT experts inside
    [0, n) (the ids address rows of the expert bank); the NaN travels on in the gates.  Also checked: the large-expert path
    (more than 64) against the oracle on ordinary logits, and the refusal of more experts than the kernel ranks."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(n + k)
    e = np.empty(k, np.int32); g = np.empty(k, np.float32)
    rows = [np.full(n, np.nan, np.float32), np.full(n, np.inf, np.float32), rng.standard_normal(n).astype(np.float32)]
    rows[2][::3] = np.nan
    for logits in rows:
        e[:] = -7
        cai.check(cai.load().cai_router_topk(logits.ctypes.data, n, k, 0, e.ctypes.data, g.ctypes.data, 0))
        assert e.min() >= 0 and e.max() < n and len(set(e.tolist())) == k, e
    logits = rng.standard_normal(n).astype(np.float32) * 2
    cai.check(cai.load().cai_router_topk(logits.ctypes.data, n, k, 1, e.ctypes.data, g.ctypes.data, 0))
    p = np.empty(n, np.float32); O.lib().orc_softmax(logits.ctypes.data, n, p.ctypes.data)
    gw = np.zeros(n, np.float32); iw = np.zeros(k, np.int32)
    O.lib().orc_topk_gate(p.ctypes.data, n, k, 1, gw.ctypes.data, iw.ctypes.data)
    assert list(e) == list(iw) and np.allclose(g, gw[iw], rtol=1e-5, atol=1e-7)
    big = np.zeros(1024, np.float32)
    assert cai.load().cai_router_topk(big.ctypes.data, 1024, 8, 0, e.ctypes.data, g.ctypes.data, 0) == -4   # CAI_ERR_UNSUPPORTED
