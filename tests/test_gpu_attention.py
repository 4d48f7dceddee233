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


def oracle_run_i8(rows, hq, hkv, dk, ctx, window=0, softcap=0.0):
    kq = np.zeros((hkv, ctx, dk), np.int8); vq = np.zeros_like(kq)
    ks = np.zeros((hkv, ctx), np.float32); vs = np.zeros_like(ks)
    outs = []
    for pos in range(rows.shape[0]):
        out = np.zeros(hq * dk, np.float32)
        O.lib().orc_attn_decode_i8(rows[pos].ctypes.data, hq, hkv, dk, kq.ctypes.data, ks.ctypes.data, vq.ctypes.data, vs.ctypes.data,
                                   ctx, pos, window, softcap, out.ctypes.data)
        outs.append(out)
    n = rows.shape[0]
    return np.array(outs), (kq[:, :n], vq[:, :n], ks[:, :n], vs[:, :n])


def stress_rows(rng, n, hq, hkv, dk):
    """Random rows, with the quantiser stress rows of the reference's append test in the K and V slices of the first
    steps (tests/TestNeuralNumerical.pas:69760-69800): all zeros, one outlier, flat, exact midpoints."""
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    kv = rows[:, hq * dk:].reshape(n, 2 * hkv, dk)
    kv[1] = 0
    kv[2] = 1e-4; kv[2, :, 0] = 100
    kv[3] = 0.75
    mid = np.full(dk, 0.5, np.float32); mid[dk - 1] = 1; d = 0
    for cand in range(127):
        v = np.float32(cand + 0.5) / np.float32(127)
        if d < dk - 1 and np.float32(v * np.float32(127)) == np.float32(cand + 0.5):
            mid[d] = v; d += 1
    kv[4] = mid; kv[5] = -mid
    return rows


@pytest.mark.parametrize("hq,hkv,dk", [(2, 1, 4), (9, 3, 64), (28, 4, 128), (16, 16, 128), (8, 1, 32), (6, 2, 80)])
@pytest.mark.parametrize("window", [0, 5])
def test_int8_cache_codes_bit_exact_and_decode_matches_oracle(hq, hkv, dk, window):
    """neural/neural.cl:2501-2687: the appended codes and row scales equal the oracle's bit for bit (the reference's own
    OpenCL-vs-host test allows one step / one ulp); outputs within 1e-5 (the reference allows 1e-3)."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(hq * 100 + dk + 7)
    n, ctx = 45, 80
    rows = stress_rows(rng, n, hq, hkv, dk)
    want, (kq, vq, ks, vs) = oracle_run_i8(rows, hq, hkv, dk, ctx, window)
    kv = cai.KVCache(2, hkv, dk, ctx, cai.KV_I8)
    for pos in range(n):
        got = kv.attn_decode(1, rows[pos], hq, window)
        assert np.max(np.abs(got - want[pos])) < 1e-5 * max(1.0, np.max(np.abs(want[pos]))), pos
    k, v, s_k, s_v = kv.export_layer(1)
    np.testing.assert_array_equal(k, kq); np.testing.assert_array_equal(v, vq)
    np.testing.assert_array_equal(s_k.view(np.uint32), ks.view(np.uint32))
    np.testing.assert_array_equal(s_v.view(np.uint32), vs.view(np.uint32))
    assert kv.len(0) == 0 and kv.export_layer(0)[0].shape == (hkv, 0, dk)


def test_int8_cache_long_context_softcap_and_non_finite_rows():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(21)
    hq, hkv, dk, n, ctx = 10, 2, 128, 600, 4096
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    want, (kq, vq, ks, vs) = oracle_run_i8(rows, hq, hkv, dk, ctx, 0, 20.0)
    kv = cai.KVCache(1, hkv, dk, ctx, cai.KV_I8)
    for pos in range(n):
        got = kv.attn_decode(0, rows[pos], hq, 0, 20.0)
        if pos % 97 == 0 or pos == n - 1:
            assert np.max(np.abs(got - want[pos])) < 1e-5, pos
    k, v, s_k, s_v = kv.export_layer(0)
    np.testing.assert_array_equal(k, kq); np.testing.assert_array_equal(v, vq)
    np.testing.assert_array_equal(s_k, ks); np.testing.assert_array_equal(s_v, vs)
    # NaN -> code 0, +/-Inf -> +/-127, neither enters the row maximum; a denormal row is unusable (unit scale, zero codes)
    kv2 = cai.KVCache(1, 1, 32, 8, cai.KV_I8)
    row = np.zeros(3 * 32, np.float32); row[:32] = 0.1
    row[32:64] = np.linspace(-1, 1, 32); row[33] = np.nan; row[34] = np.inf; row[35] = -np.inf
    row[64:] = 1e-41
    kv2.attn_decode(0, row, 1)
    k, v, s_k, s_v = kv2.export_layer(0)
    codes = np.zeros(32, np.int8); sc = np.zeros(1, np.float32)
    kr = np.ascontiguousarray(row[32:64])
    O.lib().orc_kv_quant_row(kr.ctypes.data, 32, codes.ctypes.data, sc.ctypes.data)
    np.testing.assert_array_equal(k[0, 0], codes)
    assert k[0, 0, 1] == 0 and k[0, 0, 2] == 127 and k[0, 0, 3] == -127 and s_k[0, 0] == sc[0] == np.float32(1) / np.float32(127)
    assert not v.any() and s_v[0, 0] == 1.0


def test_int8_cache_snapshot_restore_and_layer_import_export():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(33)
    hq, hkv, dk, n = 6, 2, 64, 40
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    kv = cai.KVCache(2, hkv, dk, 64, cai.KV_I8)
    first = [kv.attn_decode(1, rows[p], hq) for p in range(n)]
    kv.truncate(10); snap = kv.snapshot()
    for p in range(5):
        kv.attn_decode(1, rows[30 + p], hq)
    kv.restore(snap)
    assert kv.len(1) == 10
    again = [kv.attn_decode(1, rows[p], hq) for p in range(10, n)]
    assert all(np.array_equal(a, b) for a, b in zip(again, first[10:]))
    with pytest.raises(cai.CaiError):
        cai.KVCache(2, hkv, dk, 64, cai.KV_F32).restore(snap)       # the element type must match
    cai.load().cai_kv_snap_destroy(snap)
    # a cache rebuilt from exported rows continues identically (the hand-off of a prefix built elsewhere)
    kv.truncate(25)
    state = kv.export_layer(1)
    other = cai.KVCache(2, hkv, dk, 64, cai.KV_I8)
    other.import_layer(1, *state)
    assert other.len(1) == 25
    for p in range(25, n):
        assert np.array_equal(other.attn_decode(1, rows[p], hq), first[p])
    # the float and half caches round-trip through the same two calls
    for dtype in (cai.KV_F32, cai.KV_F16):
        a = cai.KVCache(1, hkv, dk, 64, dtype)
        ref = [a.attn_decode(0, rows[p], hq) for p in range(n)]
        a.truncate(12)
        b = cai.KVCache(1, hkv, dk, 64, dtype)
        b.import_layer(0, *a.export_layer(0)[:2])
        for p in range(12, 20):
            assert np.array_equal(b.attn_decode(0, rows[p], hq), ref[p])


def oracle_run_evict(rows, hq, hkv, dk, sinks, recent, kv_f16=0):
    n = rows.shape[0]
    kc = np.zeros((hkv, n, dk), np.float32); vc = np.zeros_like(kc)
    outs = []
    for pos in range(n):
        out = np.zeros(hq * dk, np.float32)
        O.lib().orc_attn_decode_evict(rows[pos].ctypes.data, hq, hkv, dk, kc.ctypes.data, vc.ctypes.data, n, pos, sinks, recent, 0.0, kv_f16, out.ctypes.data)
        outs.append(out)
    return np.array(outs)


@pytest.mark.parametrize("hq,hkv,dk,ctx,sinks,recent", [(4, 2, 64, 16, 2, 4), (28, 4, 128, 128, 4, 90), (32, 16, 128, 1024, 3, 300), (6, 2, 4, 64, 0, 33)])
def test_sink_and_window_eviction_matches_oracle_past_max_ctx(hq, hkv, dk, ctx, sinks, recent):
    """EnableEviction (neural/neuraldecode.pas:1257-1276, tests/TestNeuralDecode.pas:3863-3990): bit-identical to the
    unbounded cache up to the cap, rows pinned at the cap beyond it, and the stream runs past max_ctx.  The third shape
    takes the one-work-group-per-KV-head kernel, the others the per-query-head kernel."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(ctx + sinks)
    cap = sinks + recent
    n = max(ctx + 40, 2 * cap + 7) if ctx <= 128 else cap + 150
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    want = oracle_run_evict(rows, hq, hkv, dk, sinks, recent)
    plain = cai.KVCache(1, hkv, dk, ctx); ev = cai.KVCache(1, hkv, dk, ctx); ev.set_eviction(sinks, recent)
    for pos in range(n):
        got = ev.attn_decode(0, rows[pos], hq)
        if pos < cap:
            assert np.array_equal(got, plain.attn_decode(0, rows[pos], hq)), pos
        assert np.max(np.abs(got - want[pos])) < 1e-5, pos
        assert ev.rows(0) == min(pos + 1, cap) and ev.len(0) == pos + 1
    with pytest.raises(cai.CaiError):
        ev.truncate(cap)                     # the evicted middle cannot come back
    with pytest.raises(cai.CaiError):
        ev.set_eviction(0, 0)                # nor can the policy change once the stream is past the cap
    with pytest.raises(cai.CaiError):
        plain.set_eviction(ctx, 1)           # sinks + recent must fit the cache
    # snapshot / restore keeps the ring: the continuation replays exactly
    snap = ev.snapshot()
    more = rng.standard_normal((9, rows.shape[1])).astype(np.float32)
    a = [ev.attn_decode(0, r, hq) for r in more]
    ev.restore(snap)
    assert ev.len(0) == n
    b = [ev.attn_decode(0, r, hq) for r in more]
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    with pytest.raises(cai.CaiError):
        plain.restore(snap)                  # a snapshot taken under another policy
    cai.load().cai_kv_snap_destroy(snap)


def test_eviction_int8_cache_tracks_fp32_cache():
    # tests/TestNeuralDecode.pas:3980-4060: both evict the same positions, so the outputs differ by int8 drift only
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(8)
    hq, hkv, dk, sinks, recent, n = 8, 2, 64, 2, 12, 90
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    f = cai.KVCache(1, hkv, dk, 32); q = cai.KVCache(1, hkv, dk, 32, cai.KV_I8)
    f.set_eviction(sinks, recent); q.set_eviction(sinks, recent)
    drift = 0.0
    for pos in range(n):
        a = f.attn_decode(0, rows[pos], hq); b = q.attn_decode(0, rows[pos], hq)
        drift = max(drift, float(np.max(np.abs(a - b))))
    assert 0 < drift < 5e-2
    assert q.rows(0) == sinks + recent


@pytest.mark.parametrize("hq,hkv,ctx", [(40, 8, 8192), (56, 8, 8192), (32, 16, 1024), (8, 8, 8192)])
@pytest.mark.parametrize("kv", ["f16", "i8"])
def test_grouped_decode_attention_fp16_int8(hq, hkv, ctx, kv):
    """Grids that fill the chip (KV heads x slices >= 256) take the one-work-group-per-KV-head slice kernel (groups of
    5, 7, 2 and 1 query heads here) with fp16 and int8 caches: same bar as the per-head kernel, int8 codes and scales
    still exact, with a sliding window and a soft cap."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(hq + ctx)
    dk, n = 128, 150
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    for window, softcap in ((0, 0.0), (70, 25.0)):
        if kv == "i8":
            want, (kq, vq, ks, vs) = oracle_run_i8(rows, hq, hkv, dk, n, window, softcap)
        else:
            want = oracle_run(rows, hq, hkv, dk, n, window, 1, softcap)
        cache = cai.KVCache(1, hkv, dk, ctx, cai.KV_I8 if kv == "i8" else cai.KV_F16)
        for pos in range(n):
            got = cache.attn_decode(0, rows[pos], hq, window, softcap)
            assert np.max(np.abs(got - want[pos])) < 1e-5 * max(1.0, np.max(np.abs(want[pos]))), (window, pos)
        if kv == "i8":
            k, v, s_k, s_v = cache.export_layer(0)
            np.testing.assert_array_equal(k, kq); np.testing.assert_array_equal(v, vq)
            np.testing.assert_array_equal(s_k, ks); np.testing.assert_array_equal(s_v, vs)


@pytest.mark.parametrize("hq,hkv", [(8, 2), (16, 8)])
def test_context_beyond_64_slices(hq, hkv):
    """20k cached rows = 80 slices of 256: more than the 64 the merge stage once held (per-head kernel for 2 KV heads, the
    per-KV-head kernel for 8).  The cache is filled through the layer import; two decode steps against a float64 soft-max."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(hq)
    dk, n, ctx = 128, 20000, 20480
    k = rng.standard_normal((hkv, n, dk)).astype(np.float16); v = rng.standard_normal((hkv, n, dk)).astype(np.float16)
    cache = cai.KVCache(1, hkv, dk, ctx, cai.KV_F16)
    cache.import_layer(0, k, v)
    assert cache.len(0) == n
    kk = [k[h].astype(np.float64) for h in range(hkv)]; vv = [v[h].astype(np.float64) for h in range(hkv)]
    G = hq // hkv
    for step in range(2):
        row = rng.standard_normal((hq + 2 * hkv) * dk).astype(np.float32)
        got = cache.attn_decode(0, row, hq)
        q = row[: hq * dk].reshape(hq, dk).astype(np.float64)
        kn = row[hq * dk: (hq + hkv) * dk].reshape(hkv, dk).astype(np.float16).astype(np.float64)
        vn = row[(hq + hkv) * dk:].reshape(hkv, dk).astype(np.float16).astype(np.float64)
        for h in range(hkv):
            kk[h] = np.vstack([kk[h], kn[h]]); vv[h] = np.vstack([vv[h], vn[h]])
        want = np.zeros((hq, dk))
        for qh in range(hq):
            s = kk[qh // G] @ q[qh] / np.sqrt(dk)
            w = np.exp(s - s.max()); w /= w.sum()
            want[qh] = w @ vv[qh // G]
        assert np.max(np.abs(got.reshape(hq, dk) - want)) < 1e-5, step
    assert cache.len(0) == n + 2


@pytest.mark.parametrize("kvt,hq,hkv,ctx,n", [("f16", 10, 2, 131072, 100003), ("f32", 4, 1, 65536, 65530), ("i8", 8, 8, 40000, 39000),
                                             ("f16", 4, 1, 12000, 11990), ("f32", 6, 2, 9000, 8990)])   # (few KV heads from 8192 rows: slices halved for the grouped kernel)
def test_very_long_caches_many_slices(kvt, hq, hkv, ctx, n):
    """Long caches (up to 512 slices of 256 rows; 64- and 128-row slices where few KV heads would leave the grouped kernel short of work-groups): the cache is filled from the host (cai_kv_import_layer), then
    three tokens are decoded on top of it and compared with the oracle's kernel over the same rows.  One KV head with 256 slices
    takes the per-head kernels and their in-kernel merge, the others the grouped kernel and the merge launch."""
    from helpers.device import dev
    cai = dev()
    dk = 128
    rng = np.random.default_rng(ctx)
    dtype = {"f32": cai.KV_F32, "f16": cai.KV_F16, "i8": cai.KV_I8}[kvt]
    kv = cai.KVCache(1, hkv, dk, ctx, dtype)
    k = rng.standard_normal((hkv, n, dk)).astype(np.float32); v = rng.standard_normal((hkv, n, dk)).astype(np.float32)
    rows = rng.standard_normal((3, (hq + 2 * hkv) * dk)).astype(np.float32)
    if kvt == "i8":
        kq = np.zeros((hkv, ctx, dk), np.int8); vq = np.zeros_like(kq); ks = np.zeros((hkv, ctx), np.float32); vs = np.zeros_like(ks)
        for g in range(hkv):        # per-row codes and scales as the append kernel makes them (neural/neural.cl:2501-2580)
            for src, q, s in ((k[g], kq[g], ks[g]), (v[g], vq[g], vs[g])):
                m = np.max(np.abs(src), axis=1); sc = np.where(m > 0, m / 127.0, 1.0).astype(np.float32)
                q[:n] = np.clip(np.rint(src / sc[:, None]), -127, 127).astype(np.int8); s[:n] = np.where(m > 0, sc, 0.0)
        kv.import_layer(0, kq[:, :n], vq[:, :n], ks[:, :n], vs[:, :n])
        for i in range(3):
            out = np.zeros(hq * dk, np.float32)
            O.lib().orc_attn_decode_i8(rows[i].ctypes.data, hq, hkv, dk, kq.ctypes.data, ks.ctypes.data, vq.ctypes.data, vs.ctypes.data,
                                       ctx, n + i, 0, 0.0, out.ctypes.data)
            got = kv.attn_decode(0, rows[i], hq)
            assert np.max(np.abs(got - out)) < 2e-5 * max(1.0, np.max(np.abs(out))), i
    else:
        f16 = kvt == "f16"
        if f16:
            k = k.astype(np.float16).astype(np.float32); v = v.astype(np.float16).astype(np.float32)
        kc = np.zeros((hkv, ctx, dk), np.float32); vc = np.zeros_like(kc); kc[:, :n] = k; vc[:, :n] = v
        kv.import_layer(0, k.astype(np.float16) if f16 else k, v.astype(np.float16) if f16 else v)
        for i in range(3):
            out = np.zeros(hq * dk, np.float32)
            O.lib().orc_attn_decode(rows[i].ctypes.data, hq, hkv, dk, kc.ctypes.data, vc.ctypes.data, ctx, n + i, 0, 0.0, 1 if f16 else 0, out.ctypes.data)
            got = kv.attn_decode(0, rows[i], hq)
            assert np.max(np.abs(got - out)) < 2e-5 * max(1.0, np.max(np.abs(out))), i
    assert kv.len(0) == n + 3
    with pytest.raises(cai.CaiError, match="limit 512"):
        cai.KVCache(1, 1, 128, 131072 + 256, cai.KV_F16)


def _quantise_rows_i8(src):
    """per-row codes and scales as the append kernel makes them (neural/neural.cl:2501-2580)"""
    m = np.max(np.abs(src), axis=1); sc = np.where(m > 0, m / 127.0, 1.0).astype(np.float32)
    return np.clip(np.rint(src / sc[:, None]), -127, 127).astype(np.int8), np.where(m > 0, sc, 0.0).astype(np.float32)


@pytest.mark.parametrize("seed", range(12))
def test_grouped_matrix_core_attention_random_geometry(seed):
    """The one-work-group-per-KV-head kernel on the matrix cores (fp16 and int8 caches of 128-wide heads) over random geometries:
    8 / 16 / 32 KV heads, 1..8 query heads per KV head, caches of 1024..12000 rows filled to a random length from the host (so the
    live range ends anywhere inside a slice, in any of its 16-row tiles), window, soft cap; a few tokens decoded on top against the
    oracle's kernel over the same rows."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(5000 + seed)
    dk = 128
    hkv = int(rng.choice([8, 16, 32])); G = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8])); hq = hkv * G
    need = (256 + hkv - 1) // hkv                       # slices for a grid that takes this kernel
    ctx = int(rng.choice([c for c in (1024, 2048, 4096, 8192, 8448, 12000) if (c + 255) // 256 >= need or (c <= 4096 and 16 >= need)]))
    kvt = "i8" if seed % 2 else "f16"
    n0, steps = int(rng.integers(0, ctx - 30)), int(rng.integers(2, 6))
    window, softcap = int(rng.choice([0, 0, 70, 300])), float(rng.choice([0.0, 0.0, 25.0]))
    k = rng.standard_normal((hkv, n0, dk)).astype(np.float32); v = rng.standard_normal((hkv, n0, dk)).astype(np.float32)
    rows = rng.standard_normal((steps, (hq + 2 * hkv) * dk)).astype(np.float32)
    kv = cai.KVCache(1, hkv, dk, ctx, cai.KV_I8 if kvt == "i8" else cai.KV_F16)
    what = (hq, hkv, ctx, kvt, n0, window, softcap)
    if kvt == "i8":
        kq = np.zeros((hkv, ctx, dk), np.int8); vq = np.zeros_like(kq); ks = np.zeros((hkv, ctx), np.float32); vs = np.zeros_like(ks)
        for g in range(hkv):
            if n0:
                kq[g, :n0], ks[g, :n0] = _quantise_rows_i8(k[g]); vq[g, :n0], vs[g, :n0] = _quantise_rows_i8(v[g])
        if n0:
            kv.import_layer(0, kq[:, :n0], vq[:, :n0], ks[:, :n0], vs[:, :n0])
    else:
        k = k.astype(np.float16).astype(np.float32); v = v.astype(np.float16).astype(np.float32)
        kc = np.zeros((hkv, ctx, dk), np.float32); vc = np.zeros_like(kc); kc[:, :n0] = k; vc[:, :n0] = v
        if n0:
            kv.import_layer(0, k.astype(np.float16), v.astype(np.float16))
    for i in range(steps):
        out = np.zeros(hq * dk, np.float32)
        if kvt == "i8":
            O.lib().orc_attn_decode_i8(rows[i].ctypes.data, hq, hkv, dk, kq.ctypes.data, ks.ctypes.data, vq.ctypes.data, vs.ctypes.data,
                                       ctx, n0 + i, window, softcap, out.ctypes.data)
        else:
            O.lib().orc_attn_decode(rows[i].ctypes.data, hq, hkv, dk, kc.ctypes.data, vc.ctypes.data, ctx, n0 + i, window, softcap, 1, out.ctypes.data)
        got = kv.attn_decode(0, rows[i], hq, window, softcap)
        assert np.max(np.abs(got - out)) < 2e-5 * max(1.0, np.max(np.abs(out))), (i,) + what


@pytest.mark.parametrize("hkv,G,sinks,recent", [(16, 2, 3, 130), (32, 1, 0, 300), (16, 3, 17, 40)])
def test_grouped_matrix_core_attention_rolling_eviction(hkv, G, sinks, recent):
    """Sink + recent-window eviction on a half-precision cache through the same kernel: the appended row's slot lies in the middle of the
    ring, every cached row stays live."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(hkv + sinks)
    dk, ctx, hq = 128, 1024, hkv * G
    n = sinks + recent + 40
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    want = oracle_run_evict(rows, hq, hkv, dk, sinks, recent, 1)
    kv = cai.KVCache(1, hkv, dk, ctx, cai.KV_F16); kv.set_eviction(sinks, recent)
    for pos in range(n):
        got = kv.attn_decode(0, rows[pos], hq)
        assert np.max(np.abs(got - want[pos])) < 2e-5 * max(1.0, np.max(np.abs(want[pos]))), pos

