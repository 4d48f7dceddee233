"""Pins the oracle's decoders of the less common GGUF types the reference also reads (Q5_K, Q2_K, Q3_K, Q4_1, Q5_0, Q5_1):
the reference's golden vectors where it holds them (Q5_K, Q2_K: gguf-py values in tiny_kquant_ref.json, demanded
bit-for-bit: every product in these formulas is exact in binary32 and at most one addition rounds), the hand-built blocks
of the reference's own test for the others (tests/TestNeuralPretrained.pas:6024-6299), and for all six an independent
restatement on random bytes written the way ggml describes the layouts (whole-array reshapes and shifts, no per-element
index arithmetic), so that a wrong shift, plane or nibble order in the scalar oracle fails."""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.fixtures_io import GGUFFile, load_json, ref_path


def f16(v):
    return np.array([np.float16(v)]).view(np.uint8)


@pytest.mark.parametrize("name,qt,bb", [("Q5_K", O.Q5_K, 176), ("Q2_K", O.Q2_K, 84)])
def test_bit_exact_vs_reference_golden(name, qt, bb):
    g = GGUFFile(ref_path("tiny_kquant.gguf"))
    t, shape, raw = g.raw("kq.%s.weight" % name)
    assert t == qt and shape == [1024] and raw.size == 4 * bb
    ref = load_json("tiny_kquant_ref.json")
    want = np.array(ref["dequant"][name], np.float32)
    got = O.dequant(qt, raw, 1024)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    src = np.array(ref["ref_f32"], np.float32).reshape(-1)
    assert np.max(np.abs(got - src)) < (0.6 if name == "Q5_K" else 2.5)   # it approximates the fp32 source it was quantised from


def test_legacy_handbuilt_blocks_of_the_reference_test():
    # Q4_1: d = 0.25, m = -1.5, nibble(e) = e mod 16 (tests/TestNeuralPretrained.pas:6145-6171)
    blk = np.zeros(20, np.uint8); blk[0:2] = f16(0.25); blk[2:4] = f16(-1.5)
    for e in range(32):
        blk[4 + e % 16] |= (e % 16) << (0 if e < 16 else 4)
    assert np.array_equal(O.dequant(O.Q4_1, blk, 32), np.array([0.25 * (e % 16) - 1.5 for e in range(32)], np.float32))
    # Q5_0: d = 0.3 (as stored: the half nearest 0.3), 5-bit code e, fifth bit in qh bit e (6173-6204)
    d = float(np.float16(0.3))
    blk = np.zeros(22, np.uint8); blk[0:2] = f16(0.3)
    for e in range(32):
        if e >> 4:
            blk[2 + e // 8] |= 1 << (e % 8)
        blk[6 + e % 16] |= (e & 15) << (0 if e < 16 else 4)
    assert np.array_equal(O.dequant(O.Q5_0, blk, 32), np.array([np.float32(d) * np.float32(e - 16) for e in range(32)], np.float32))
    # Q5_1: d = 0.2, m = 2.0 (6206-6236)
    d = float(np.float16(0.2))
    blk = np.zeros(24, np.uint8); blk[0:2] = f16(0.2); blk[2:4] = f16(2.0)
    for e in range(32):
        if e >> 4:
            blk[4 + e // 8] |= 1 << (e % 8)
        blk[8 + e % 16] |= (e & 15) << (0 if e < 16 else 4)
    assert np.array_equal(O.dequant(O.Q5_1, blk, 32), np.array([np.float32(d * e + 2.0) for e in range(32)], np.float32))


def test_q3_k_handbuilt_super_block_of_the_reference_test():
    # tests/TestNeuralPretrained.pas:6238-6299: packed scale sb + 24 (signed -8..7), qcode = e mod 4, hbit = (e mod 3) & 1
    d = float(np.float16(0.1))
    blk = np.zeros(110, np.uint8); blk[108:110] = f16(0.1)
    scales = [sb + 24 for sb in range(16)]
    for e in range(256):
        blk[32 + (e // 128) * 32 + e % 32] |= (e % 4) << (2 * ((e % 128) // 32))
        if (e % 3) & 1:
            blk[e % 32] |= 1 << (e // 32)
    for j in range(16):
        blk[96 + j % 8] |= (scales[j] & 15) << (0 if j < 8 else 4)
        blk[96 + 8 + j % 4] |= ((scales[j] >> 4) & 3) << (2 * (j // 4))
    got = O.dequant(O.Q3_K, blk, 256)
    want = np.array([np.float32(d) * np.float32(scales[e // 16] - 32) * np.float32((e % 4) - ((1 ^ ((e % 3) & 1)) << 2)) for e in range(256)], np.float32)
    assert np.array_equal(got, want)


def random_blocks(qt, n, seed):
    """n blocks of random bytes whose f16 fields are finite (the quant codes and packed scales take every value)"""
    rng = np.random.default_rng(seed)
    bb = {O.Q5_K: 176, O.Q2_K: 84, O.Q3_K: 110, O.Q4_1: 20, O.Q5_0: 22, O.Q5_1: 24}[qt]
    raw = rng.integers(0, 256, (n, bb), dtype=np.uint8)
    halfs = {O.Q5_K: [0, 2], O.Q2_K: [80, 82], O.Q3_K: [108], O.Q4_1: [0, 2], O.Q5_0: [0], O.Q5_1: [0, 2]}[qt]
    for off in halfs:
        v = (rng.uniform(1e-4, 0.3, n) * rng.choice([-1.0, 1.0], n)).astype(np.float16)
        raw[:, off:off + 2] = v.view(np.uint8).reshape(n, 2)
    return raw


def vectorised_reference(qt, raw):
    """The ggml layouts stated as whole-array reshapes and shifts (float64 arithmetic, rounded once)."""
    n = raw.shape[0]
    h = lambda off: raw[:, off:off + 2].copy().view(np.float16).astype(np.float64)      # [n, 1]
    if qt in (O.Q4_1, O.Q5_0, O.Q5_1):
        qs_off = {O.Q4_1: 4, O.Q5_0: 6, O.Q5_1: 8}[qt]
        qs = raw[:, qs_off:qs_off + 16]
        nib = np.concatenate([qs & 15, qs >> 4], 1).astype(np.int64)                     # qs.reshape(-1, 2, 16) >> [0, 4]
        if qt == O.Q4_1:
            return (h(0) * nib + h(2)).astype(np.float32)
        qh_off = 2 if qt == O.Q5_0 else 4
        qh = raw[:, qh_off:qh_off + 4].copy().view("<u4").astype(np.int64)               # [n, 1]
        q5 = nib | (((qh >> np.arange(32)) & 1) << 4)
        return (h(0) * (q5 - 16)).astype(np.float32) if qt == O.Q5_0 else (h(0) * q5 + h(2)).astype(np.float32)
    if qt == O.Q5_K:
        p = raw[:, 4:16].astype(np.int64)
        sc = np.concatenate([p[:, 0:4] & 63, (p[:, 8:12] & 15) | ((p[:, 0:4] >> 6) << 4)], 1)
        mn = np.concatenate([p[:, 4:8] & 63, (p[:, 8:12] >> 4) | ((p[:, 4:8] >> 6) << 4)], 1)
        ql = raw[:, 48:176].reshape(n, 4, 1, 32) >> np.array([0, 4], np.uint8).reshape(1, 1, 2, 1)
        ql = (ql & 15).reshape(n, 8, 32).astype(np.int64)
        qhb = (raw[:, 16:48].reshape(n, 1, 32) >> np.arange(8, dtype=np.uint8).reshape(1, 8, 1)) & 1
        q = ql | (qhb.astype(np.int64) << 4)
        x = (h(0) * sc)[:, :, None] * q - (h(2) * mn)[:, :, None]
        return x.reshape(n, 256).astype(np.float32)
    if qt == O.Q2_K:
        scb = raw[:, 0:16].astype(np.int64)
        dl = h(80) * (scb & 15); ml = h(82) * (scb >> 4)                                  # [n, 16]
        q = (raw[:, 16:80].reshape(n, 2, 1, 32) >> np.array([0, 2, 4, 6], np.uint8).reshape(1, 1, 4, 1)) & 3
        q = q.reshape(n, 16, 16).astype(np.int64)
        return (dl[:, :, None] * q - ml[:, :, None]).reshape(n, 256).astype(np.float32)
    if qt == O.Q3_K:
        sp = raw[:, 96:108].astype(np.int64)
        low = np.concatenate([sp[:, 0:8] & 15, sp[:, 0:8] >> 4], 1)                       # scales 0..7, 8..15
        high = ((sp[:, 8:12].reshape(n, 1, 4) >> np.array([0, 2, 4, 6]).reshape(1, 4, 1)) & 3).reshape(n, 16)
        scale = (low | (high << 4)) - 32
        ql = (raw[:, 32:96].reshape(n, 2, 1, 32) >> np.array([0, 2, 4, 6], np.uint8).reshape(1, 1, 4, 1)) & 3
        hb = (raw[:, 0:32].reshape(n, 1, 32) >> np.arange(8, dtype=np.uint8).reshape(1, 8, 1)) & 1
        q = ql.reshape(n, 256).astype(np.int64) - ((hb.reshape(n, 256).astype(np.int64) ^ 1) << 2)
        return ((h(108) * scale)[:, :, None] * q.reshape(n, 16, 16)).reshape(n, 256).astype(np.float32)
    raise AssertionError(qt)


@pytest.mark.parametrize("qt", [O.Q5_K, O.Q2_K, O.Q3_K, O.Q4_1, O.Q5_0, O.Q5_1])
def test_random_bytes_against_the_vectorised_restatement(qt):
    raw = random_blocks(qt, 64, seed=qt)
    be = 256 if qt in (O.Q5_K, O.Q2_K, O.Q3_K) else 32
    got = O.dequant(qt, raw.reshape(-1), 64 * be).reshape(64, be)
    want = vectorised_reference(qt, raw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_row_bytes_of_every_type():
    for qt, be, bb in [(O.Q4_1, 32, 20), (O.Q5_0, 32, 22), (O.Q5_1, 32, 24), (O.Q2_K, 256, 84), (O.Q3_K, 256, 110), (O.Q5_K, 256, 176)]:
        assert O.row_bytes(qt, 4 * be) == 4 * bb and O.row_bytes(qt, be + 1) == -1


@pytest.mark.parametrize("qt,rel", [(O.Q5_K, 0.04), (O.Q2_K, 0.4), (O.Q3_K, 0.2), (O.Q4_1, 0.08), (O.Q5_0, 0.05), (O.Q5_1, 0.04)])
def test_test_side_packers_round_trip_through_the_oracle(qt, rel):
    """quantize (numpy packers of tests/helpers/quant_other.py) -> oracle decode stays within a format-sized error of the
    source: pins the packers the model-level tests build their weights with (a wrong plane or shift gives errors ~ 1)."""
    rng = np.random.default_rng(qt)
    x = rng.standard_normal((8, 512)).astype(np.float32)
    raw = O.quantize(qt, x)
    back = O.dequant(qt, raw, x.size).reshape(x.shape)
    err = np.sqrt(np.mean((back - x) ** 2)) / np.sqrt(np.mean(x ** 2))
    assert err < rel, err
    assert np.array_equal(back.reshape(-1, 256 if qt in (O.Q5_K, O.Q2_K, O.Q3_K) else 32),
                          vectorised_reference(qt, raw.reshape(-1, O.row_bytes(qt, 512) // (2 if qt in (O.Q5_K, O.Q2_K, O.Q3_K) else 16))))
