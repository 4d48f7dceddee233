"""Pins the oracle's codecs against the reference's own golden vectors and against closed forms.

Exactness note for Q4_K: d*sc (<= 17 significant bits), (d*sc)*q (<= 21 bits) and dmin*mn (<= 17 bits) are
exactly representable in binary32 and both lie on a 2^-24 grid below 2^26, so their difference is exact in
double and rounds once; any evaluation order (FMA or not) yields the same binary32 value.  That is why the
comparison with the gguf-py reference values can be demanded bit-for-bit.
"""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.fixtures_io import GGUFFile, load_json, load_safetensors, ref_path

L = O.lib()

# tests/TestNeuralVolume.pas:3223-3246 known answers
F16_BITS = [0x3C00, 0xBC00, 0x0000, 0x8000, 0x4000, 0xC000, 0x3800, 0xB800, 0x7BFF, 0xFBFF, 0x0001, 0x8001, 0x03FF,
            0x0400, 0x3555, 0x4248, 0x5140, 0xD140, 0x1400, 0x6400, 0xE400]
F16_VALS = [1.0, -1.0, 0.0, -0.0, 2.0, -2.0, 0.5, -0.5, 65504.0, -65504.0, 5.9604644775390625e-8,
            -5.9604644775390625e-8, 6.0975551605224609e-5, 6.103515625e-5, 0.333251953125, 3.140625, 42.0, -42.0,
            0.0009765625, 1024.0, -1024.0]


def test_f16_known_answers():
    for b, v in zip(F16_BITS, F16_VALS):
        got = L.orc_f16_to_f32(b)
        assert got == v and np.signbit(got) == np.signbit(v), hex(b)


def test_f16_special_values():
    # tests/TestNeuralVolume.pas:3264-3294
    assert L.orc_f16_to_f32(0x7C00) == np.inf and L.orc_f16_to_f32(0xFC00) == -np.inf
    assert np.isnan(L.orc_f16_to_f32(0x7E00)) and np.isnan(L.orc_f16_to_f32(0x7DAB))


def test_f16_exhaustive_vs_numpy_half():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.orc_f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_encode_roundtrip_and_rne():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    for b, v in zip(bits.tolist(), vals.tolist()):
        if np.isnan(v):
            continue
        assert L.orc_f32_to_f16(v) == b
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(20000) * 10.0 ** rng.integers(-4, 4, 20000)).astype(np.float32)
    x = x[np.abs(x) >= 6.2e-5]  # normal half range: round-to-nearest-even like IEEE
    want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f32_to_f16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)


def test_q4k_bit_exact_vs_reference_golden():
    g = GGUFFile(ref_path("tiny_kquant.gguf"))
    t, shape, raw = g.raw("kq.Q4_K.weight")
    assert t == O.Q4_K and shape == [1024] and raw.size == 4 * 144
    want = np.array(load_json("tiny_kquant_ref.json")["dequant"]["Q4_K"], np.float32)
    got = O.dequant(O.Q4_K, raw, 1024)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and it approximates the fp32 source the fixture was quantised from
    src = np.array(load_json("tiny_kquant_ref.json")["ref_f32"], np.float32)
    assert np.max(np.abs(got - src)) < 0.6


def test_q4k_scale_min_bruteforce():
    rng = np.random.default_rng(7)
    for _ in range(500):
        sc = rng.integers(0, 64, 8); mn = rng.integers(0, 64, 8)
        p = np.zeros(12, np.uint8)
        for j in range(4):  # 6-bit field definition (neuralgguf.pas:440-447)
            p[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
            p[j + 4] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
            p[j + 8] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
        s8 = np.zeros(8, np.uint8); m8 = np.zeros(8, np.uint8)
        L.orc_q4k_scale_min(p.ctypes.data, s8.ctypes.data, m8.ctypes.data)
        assert np.array_equal(s8, sc) and np.array_equal(m8, mn)


def test_q4k_closed_form_all_sc_q():
    # every (sc, q) pair with mn sweeping, random half d/dmin: x == (d*sc)*q - dmin*mn evaluated in double
    rng = np.random.default_rng(3)
    for trial in range(8):
        d = np.float16(rng.uniform(1e-4, 0.1)); dm = np.float16(rng.uniform(1e-4, 0.1))
        blk = np.zeros(144, np.uint8)
        blk[0:2] = np.array([d]).view(np.uint8); blk[2:4] = np.array([dm]).view(np.uint8)
        sc = rng.integers(0, 64, 8); mn = rng.integers(0, 64, 8)
        for j in range(4):
            blk[4 + j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
            blk[8 + j] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
            blk[12 + j] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
        q = rng.integers(0, 16, 256)
        for c in range(4):
            blk[16 + 32 * c:16 + 32 * c + 32] = q[64 * c:64 * c + 32] | (q[64 * c + 32:64 * c + 64] << 4)
        got = O.dequant(O.Q4_K, blk, 256)
        want = np.empty(256, np.float32)
        for j in range(8):
            want[32 * j:32 * j + 32] = (float(d) * sc[j] * q[32 * j:32 * j + 32].astype(np.float64) - float(dm) * mn[j]).astype(np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q4_0_reference_handbuilt_block():
    # tests/TestNeuralPretrained.pas:6116-6143: d = 0.5, nibble(e) = e mod 16 -> x = d*((e mod 16) - 8)
    blk = np.zeros(18, np.uint8)
    blk[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
    for e in range(16):
        blk[2 + e] = (e % 16) | (((e + 16) % 16) << 4)
    got = O.dequant(O.Q4_0, blk, 32)
    want = np.array([0.5 * ((e % 16) - 8) for e in range(32)], np.float32)
    assert np.array_equal(got, want)
    # asymmetric nibbles catch a swapped low/high half
    blk[2:18] = np.arange(16, dtype=np.uint8) | ((15 - np.arange(16, dtype=np.uint8)) << 4)
    got = O.dequant(O.Q4_0, blk, 32)
    want = np.concatenate([0.5 * (np.arange(16) - 8), 0.5 * ((15 - np.arange(16)) - 8)]).astype(np.float32)
    assert np.array_equal(got, want)


def test_q8_0_closed_form_and_reference_gguf_twin():
    rng = np.random.default_rng(5)
    q = rng.integers(-127, 128, (10, 32)).astype(np.int8)
    d = rng.uniform(1e-5, 0.2, 10).astype(np.float16)
    raw = np.zeros((10, 34), np.uint8)
    raw[:, 0:2] = d.view(np.uint8).reshape(10, 2); raw[:, 2:] = q.view(np.uint8)
    got = O.dequant(O.Q8_0, raw.reshape(-1), 320).reshape(10, 32)
    want = d.astype(np.float32)[:, None] * q.astype(np.float32)
    assert np.array_equal(got, want)
    # reference-held Q8_0 GGUF against its fp32 twin (tests/TestNeuralPretrained.pas:5891-5917)
    g = GGUFFile(ref_path("tiny_llama_q8.gguf"))
    st = load_safetensors(ref_path("tiny_llama_q8.safetensors"))
    t, shape, raw = g.raw("blk.0.attn_v.weight")
    assert t == O.Q8_0
    deq = O.dequant(t, raw, shape[0] * shape[1]).reshape(shape)
    twin = st["model.layers.0.self_attn.v_proj.weight"]
    err = np.max(np.abs(deq - twin))
    assert 1e-6 < err < 0.01


def test_gguf_qk_deinterleave_matches_safetensors():
    # tests/TestNeuralPretrained.pas:5861-5869: de-interleaved GGUF q rows == HF rows exactly (F32 file)
    g = GGUFFile(ref_path("tiny_llama_f32.gguf"))
    st = load_safetensors(ref_path("tiny_llama.safetensors"))
    t, shape, raw = g.raw("blk.0.attn_q.weight")
    w = O.dequant(t, raw, shape[0] * shape[1]).reshape(shape)
    hd = 4
    hf = np.stack([w[L.orc_gguf_deinterleaved_src_row(r, hd)] for r in range(shape[0])])
    assert np.array_equal(hf, st["model.layers.0.self_attn.q_proj.weight"])
    # composing with MapTargetNeuron is the identity on stored rows
    for hd in (4, 64, 128):
        for r in range(2 * hd):
            assert L.orc_map_target_neuron(r, hd) == L.orc_gguf_deinterleaved_src_row(r, hd)


@pytest.mark.parametrize("qt,tol", [(O.Q8_0, 0.5), (O.Q4_0, 1.0), (O.Q4_K, 1.0)])
def test_quantizer_roundtrip(qt, tol):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((8, 512)) * 0.02).astype(np.float32)
    raw = O.quantize(qt, x)
    assert raw.size == 8 * O.row_bytes(qt, 512)
    y = O.dequant(qt, raw, x.size).reshape(x.shape)
    if qt == O.Q8_0:
        step = np.abs(x.reshape(-1, 32)).max(1) / 127
    elif qt == O.Q4_0:
        step = np.abs(x.reshape(-1, 32)).max(1) / 8
    else:
        step = (x.reshape(-1, 32).max(1) - np.minimum(x.reshape(-1, 32).min(1), 0)) / 15
    err = np.abs(x - y).reshape(-1, 32).max(1)
    assert np.all(err <= tol * step * 1.3 + 1e-6)


def test_int8_row_roundtrip():
    # tests/TestNeuralPretrained.pas:3592: round trip within scale/2
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((4, 100)) * 0.05).astype(np.float32)
    codes, scales = O.quant_int8_rows(x)
    assert np.all(np.abs(codes.astype(np.float32) * scales[:, None] - x) <= scales[:, None] * 0.5 + 1e-7)
    assert np.all(np.abs(codes).max(1) == 127)


def test_q6_k_dequant_matches_reference_vectors_bit_for_bit():
    """tiny_kquant.gguf / tiny_kquant_ref.json (gguf-py values): d*scale and its product with q are exact in binary32."""
    g = GGUFFile(ref_path("tiny_kquant.gguf"))
    t, shape, raw = g.raw("kq.Q6_K.weight")
    assert t == O.Q6_K and shape == [1024] and raw.size == 4 * 210
    want = np.array(load_json("tiny_kquant_ref.json")["dequant"]["Q6_K"], np.float32)
    got = O.dequant(O.Q6_K, raw, 1024)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q6_k_closed_form_on_random_bytes_and_packer_round_trip():
    rng = np.random.default_rng(5)
    blk = rng.integers(0, 256, 210, dtype=np.uint8)
    blk[208:210] = np.array([0.0123], np.float16).view(np.uint8)
    got = O.dequant(O.Q6_K, blk, 256)
    d = np.float32(np.array([0.0123], np.float16)[0]); sc = blk[192:208].view(np.int8)
    for i in (0, 15, 16, 63, 64, 100, 127, 128, 191, 200, 255):
        lo = int(blk[(i // 128) * 64 + i % 64]); nib = (lo & 15) if (i % 128) < 64 else (lo >> 4)
        h2 = (int(blk[128 + (i // 128) * 32 + i % 32]) >> (2 * ((i % 128) // 32))) & 3
        assert got[i] == np.float32(np.float32(d * np.float32(sc[i // 16])) * np.float32((nib | (h2 << 4)) - 32))
    x = (rng.standard_normal(512) * 0.02).astype(np.float32)
    back = O.dequant(O.Q6_K, O.quantize(O.Q6_K, x), 512)
    assert np.max(np.abs(back - x)) < np.max(np.abs(x)) / 31 * 0.75      # half a step of the coarsest group, plus scale rounding
