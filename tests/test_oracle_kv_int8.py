"""Pins the oracle's int8 KV-cache restatement (append rule neural/neural.cl:2501-2580, decode 2582-2687).

Known answers are the rows the reference's own tests build: the MaxAbsFinite cases of
tests/TestNeuralVolume.pas:2864-2903 and the zero / one-outlier / flat / exact-midpoint rows of
FusedSDPAInt8AppendOpenCLParity (tests/TestNeuralNumerical.pas:69740-69800), whose codes follow from the rule in closed
form.  The decode is pinned against the fp32 attention on caches whose rows quantise without error."""
import numpy as np

from helpers import oracle_lib as O


def max_abs_finite(x):
    x = np.ascontiguousarray(x, np.float32)
    return O.lib().orc_max_abs_finite(x.ctypes.data, x.size)


def quant_row(x):
    x = np.ascontiguousarray(x, np.float32)
    codes = np.zeros(x.size, np.int8); scale = np.zeros(1, np.float32)
    O.lib().orc_kv_quant_row(x.ctypes.data, x.size, codes.ctypes.data, scale.ctypes.data)
    return codes, scale[0]


def test_max_abs_finite_reference_cases():
    n = 37
    v = np.zeros(n, np.float32)
    assert max_abs_finite(v) == 0.0
    v[:] = 0.5; v[20] = -3.25
    assert max_abs_finite(v) == 3.25
    v[35] = -9.5
    assert max_abs_finite(v) == 9.5
    v[3] = np.nan; v[9] = np.inf; v[34] = -np.inf
    assert max_abs_finite(v) == 9.5
    v[:] = np.nan
    assert max_abs_finite(v) == 0.0
    v[:] = 0; v[5] = -2
    assert max_abs_finite(v[:8]) == 2.0


def test_quantiser_stress_rows_of_the_reference():
    dk = 64
    codes, scale = quant_row(np.zeros(dk))
    assert scale == 1.0 and not codes.any()                      # all-zero row: unit scale, zero codes
    row = np.full(dk, 1e-4, np.float32); row[0] = 100
    codes, scale = quant_row(row)
    assert scale == np.float32(100) / np.float32(127) and codes[0] == 127 and not codes[1:].any()
    codes, scale = quant_row(np.full(dk, 0.75, np.float32))
    assert scale == np.float32(0.75) / np.float32(127) and (codes == 127).all()
    # exact midpoints: row maximum 1, elements (c + 0.5)/127 that scale back to exactly c + 0.5 -> half-to-even
    row = np.full(dk, 0.5, np.float32); row[dk - 1] = 1
    want = np.zeros(dk, np.int64); d = 0; n_mid = 0
    for cand in range(127):
        if d >= dk - 1: break
        v = np.float32(cand + 0.5) / np.float32(127)
        if np.float32(v * np.float32(127)) == np.float32(cand + 0.5):
            row[d] = v; want[d] = cand if cand % 2 == 0 else cand + 1; d += 1; n_mid += 1
    assert n_mid >= 2
    want[d:dk - 1] = 64                                          # 0.5 * 127 = 63.5 -> 64 (even)
    want[dk - 1] = 127
    codes, scale = quant_row(row)
    assert scale == np.float32(1) / np.float32(127)
    np.testing.assert_array_equal(codes, want)
    # the negated row mirrors exactly (symmetric quantiser)
    codes_n, _ = quant_row(-row)
    np.testing.assert_array_equal(codes_n, -want)


def test_quantiser_non_finite_and_denormal_rows():
    row = np.array([1.0, np.nan, np.inf, -np.inf, -0.25, 0.5], np.float32)
    codes, scale = quant_row(row)
    assert scale == np.float32(1) / np.float32(127)
    np.testing.assert_array_equal(codes, [127, 0, 127, -127, -32, 64])   # -31.75 -> -32, 63.5 -> 64
    codes, scale = quant_row(np.array([1e-40, -1e-41], np.float32))       # denormal maximum: unusable
    assert scale == 1.0 and not codes.any()
    codes, scale = quant_row(np.array([2.0 ** 120, -2.0 ** 119, 1.0], np.float32))  # 1/max first, then *127: no overflow
    np.testing.assert_array_equal(codes, [127, -64, 0])                   # -63.5 -> -64 (even)
    # random rows: |x - scale*code| <= scale/2 (+ rounding of the two multiplies), codes reach +/-127
    rng = np.random.default_rng(5)
    for _ in range(20):
        x = (rng.standard_normal(128) * rng.uniform(1e-3, 1e3)).astype(np.float32)
        codes, scale = quant_row(x)
        assert np.abs(codes).max() == 127
        assert np.abs(x - scale * codes.astype(np.float32)).max() <= 0.5 * scale * (1 + 1e-5)


def test_int8_decode_equals_fp32_decode_when_rows_quantise_exactly():
    # rows of integers in [-127,127] times 2^e with a +/-127 entry: max = 127 * 2^e, scale = 2^e, and v * (1/max) * 127
    # lands within an ulp of the integer it came from, so codes = x / 2^e and scale * code reproduces x exactly
    rng = np.random.default_rng(11)
    hq, hkv, dk, ctx = 4, 2, 32, 24
    kw = hkv * dk
    kc = np.zeros((hkv, ctx, dk), np.float32); vc = np.zeros_like(kc)
    kq = np.zeros((hkv, ctx, dk), np.int8); vq = np.zeros_like(kq)
    ks = np.zeros((hkv, ctx), np.float32); vs = np.zeros_like(ks)
    for window in (0, 5):
        for pos in range(ctx):
            row = np.zeros(hq * dk + 2 * kw, np.float32)
            row[:hq * dk] = rng.standard_normal(hq * dk) * 0.3
            for part in range(2 * hkv):
                e = float(2.0 ** rng.integers(-9, -4))
                ints = rng.integers(-127, 128, dk); ints[rng.integers(dk)] = 127 if rng.random() < 0.5 else -127
                row[hq * dk + part * dk: hq * dk + (part + 1) * dk] = ints * e
            a = np.zeros(hq * dk, np.float32); b = np.zeros_like(a)
            O.lib().orc_attn_decode(row.ctypes.data, hq, hkv, dk, kc.ctypes.data, vc.ctypes.data, ctx, pos, window, 0.0, 0, a.ctypes.data)
            O.lib().orc_attn_decode_i8(row.ctypes.data, hq, hkv, dk, kq.ctypes.data, ks.ctypes.data, vq.ctypes.data, vs.ctypes.data, ctx, pos, window, 0.0, b.ctypes.data)
            # same real numbers, different association of the (exact, power-of-two) scale: a few ulps
            np.testing.assert_allclose(b, a, rtol=2e-5, atol=1e-6)
        np.testing.assert_array_equal(kq.astype(np.float32) * ks[..., None], kc)
        np.testing.assert_array_equal(vq.astype(np.float32) * vs[..., None], vc)


def test_int8_decode_brute_force_softmax():
    rng = np.random.default_rng(3)
    hq, hkv, dk, ctx = 6, 3, 16, 9
    kw = hkv * dk
    kq = np.zeros((hkv, ctx, dk), np.int8); vq = np.zeros_like(kq)
    ks = np.zeros((hkv, ctx), np.float32); vs = np.zeros_like(ks)
    for pos in range(ctx):
        row = rng.standard_normal(hq * dk + 2 * kw).astype(np.float32)
        out = np.zeros(hq * dk, np.float32)
        O.lib().orc_attn_decode_i8(row.ctypes.data, hq, hkv, dk, kq.ctypes.data, ks.ctypes.data, vq.ctypes.data, vs.ctypes.data, ctx, pos, 0, 0.0, out.ctypes.data)
        K = kq[:, :pos + 1].astype(np.float64) * ks[:, :pos + 1, None]; V = vq[:, :pos + 1].astype(np.float64) * vs[:, :pos + 1, None]
        for h in range(hq):
            g = h // (hq // hkv)
            s = K[g] @ row[h * dk:(h + 1) * dk].astype(np.float64) / np.sqrt(dk)
            w = np.exp(s - s.max()); w /= w.sum()
            np.testing.assert_allclose(out[h * dk:(h + 1) * dk], w @ V[g], rtol=1e-4, atol=1e-5)


def test_eviction_mask_within_cap_identical_and_past_cap_brute_force():
    """Sink + recent-window eviction as the oracle states it (neural/neuraldecode.pas:1257-1276): up to the cap the run
    is bit-identical to the unbounded one (tests/TestNeuralDecode.pas:3863-3915); past it the output is the softmax over
    positions [0, sinks) and the latest `recent`."""
    rng = np.random.default_rng(17)
    hq, hkv, dk, n, sinks, recent = 4, 2, 8, 20, 2, 4
    rows = rng.standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
    kc = np.zeros((hkv, n, dk), np.float32); vc = np.zeros_like(kc)
    ke = np.zeros_like(kc); ve = np.zeros_like(kc)
    for pos in range(n):
        a = np.zeros(hq * dk, np.float32); b = np.zeros_like(a)
        O.lib().orc_attn_decode(rows[pos].ctypes.data, hq, hkv, dk, kc.ctypes.data, vc.ctypes.data, n, pos, 0, 0.0, 0, a.ctypes.data)
        O.lib().orc_attn_decode_evict(rows[pos].ctypes.data, hq, hkv, dk, ke.ctypes.data, ve.ctypes.data, n, pos, sinks, recent, 0.0, 0, b.ctypes.data)
        if pos + 1 <= sinks + recent:
            assert np.array_equal(a, b), pos
        else:
            live = list(range(sinks)) + list(range(pos + 1 - recent, pos + 1))
            assert len(live) == sinks + recent
            for h in range(hq):
                g = h // (hq // hkv)
                s = ke[g, live].astype(np.float64) @ rows[pos, h * dk:(h + 1) * dk].astype(np.float64) / np.sqrt(dk)
                w = np.exp(s - s.max()); w /= w.sum()
                np.testing.assert_allclose(b[h * dk:(h + 1) * dk], w @ ve[g, live].astype(np.float64), rtol=1e-5, atol=1e-6)
            assert not np.allclose(a, b)
