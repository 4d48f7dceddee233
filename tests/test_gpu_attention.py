"""Cached GQA decode attention (append + split-K online softmax) against the oracle's three-phase restatement
of the reference kernel (neural.cl:2354-2499).  Tolerance 1e-5 like the reference's tiled-softmax test
(tests/TestNeuralDecode.pas:1642-1706)."""
import numpy as np
import pytest

from helpers import oracle_lib as O

pytestmark = pytest.mark.gpu


def oracle_run(rows, hq, hkv, dk, ctx, window=0, kv_f16=0, softcap=0.0):
    kc = np.zeros((hkv, ctx, dk), np.float32); vc = np.zeros_like(kc)
    outs = []
    for pos in range(rows.shape[0]):
        out = np.zeros(hq * dk, np.float32)
        O.lib().orc_attn_decode(rows[pos].ctypes.data, hq, hkv, dk, kc.ctypes.data, vc.ctypes.data, ctx, pos, window, softcap, kv_f16, out.ctypes.data)
        outs.append(out)
    return np.array(outs)


@pytest.mark.parametrize("hq,hkv,dk", [(2, 1, 4), (9, 3, 64), (28, 4, 128), (16, 16, 128), (40, 8, 128), (8, 1, 32)])
@pytest.mark.parametrize("window", [0, 5])
def test_decode_matches_oracle(hq, hkv, dk, window):
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(hq * 100 + dk)
    n, ctx = 45, 80           # crosses split boundaries (split length 32)
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    want = oracle_run(rows, hq, hkv, dk, ctx, window)
    kv = cai.KVCache(2, hkv, dk, ctx)
    for pos in range(n):
        got = kv.attn_decode(1, rows[pos], hq, window)
        assert np.max(np.abs(got - want[pos])) < 1e-5, pos
    assert kv.len(1) == n and kv.len(0) == 0


def test_long_context_many_splits_and_f16_cache():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(1)
    hq, hkv, dk, n, ctx = 10, 2, 128, 700, 4096
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    for dtype, f16, tol in ((cai.KV_F32, 0, 1e-5), (cai.KV_F16, 1, 1e-5)):
        want = oracle_run(rows, hq, hkv, dk, ctx, 0, f16)
        kv = cai.KVCache(1, hkv, dk, ctx, dtype)
        for pos in range(n):
            got = kv.attn_decode(0, rows[pos], hq)
            if pos % 97 == 0 or pos == n - 1:
                assert np.max(np.abs(got - want[pos])) < tol, (dtype, pos)


def test_softcap():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(2)
    hq, hkv, dk, n = 4, 2, 64, 20
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32) * 3
    want = oracle_run(rows, hq, hkv, dk, 32, 0, 0, 30.0)
    kv = cai.KVCache(1, hkv, dk, 32)
    for pos in range(n):
        assert np.max(np.abs(kv.attn_decode(0, rows[pos], hq, 0, 30.0) - want[pos])) < 1e-5 * max(1.0, np.max(np.abs(want[pos])))


def test_truncate_snapshot_restore_reset():
    # tests/TestNeuralFusedSDPA.pas:228-454: truncate/rollback, capture/restore are bit-identical
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(3)
    hq, hkv, dk, n = 6, 2, 64, 40
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    kv = cai.KVCache(1, hkv, dk, 64)
    first = [kv.attn_decode(0, rows[p], hq) for p in range(n)]
    kv.truncate(25)
    assert kv.len() == 25
    again = [kv.attn_decode(0, rows[p], hq) for p in range(25, n)]
    assert all(np.array_equal(a, b) for a, b in zip(again, first[25:]))
    kv.truncate(10); snap = kv.snapshot()
    other = rng.standard_normal((5, rows.shape[1])).astype(np.float32)
    for p in range(5):
        kv.attn_decode(0, other[p], hq)
    kv.restore(snap)
    assert kv.len() == 10
    replay = [kv.attn_decode(0, rows[p], hq) for p in range(10, 20)]
    assert all(np.array_equal(a, b) for a, b in zip(replay, first[10:20]))
    cai.load().cai_kv_snap_destroy(snap)
    kv.reset()
    assert kv.len() == 0
    assert np.array_equal(kv.attn_decode(0, rows[0], hq), first[0])


def test_cache_full_is_an_error_not_a_fault():
    from helpers.device import dev
    cai = dev()
    kv = cai.KVCache(1, 1, 32, 3)
    row = np.ones(3 * 32, np.float32)
    for _ in range(3):
        kv.attn_decode(0, row, 1)
    with pytest.raises(cai.CaiError) as e:
        kv.attn_decode(0, row, 1)
    assert e.value.code == -5
