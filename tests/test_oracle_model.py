"""Pins the oracle's whole-decoder restatement against the logits the reference's own tests hold
(tests/TestNeuralPretrained.pas:5684-5757 and siblings; gate 1e-4, never looser than 1e-3)."""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.fixtures_io import load_json, ref_path
from helpers.model_build import oracle_model, spec_from_gguf_llama, spec_from_ref_fixture

FAMILIES = ["tiny_llama", "tiny_smollm2", "tiny_qwen2", "tiny_mistral", "tiny_olmoe"]


def run_sequences(model, seqs):
    out = []
    for s in seqs:
        model.reset()
        out.append([model.step(t, p)[1] for p, t in enumerate(s)])
    return np.array(out, np.float32)


@pytest.mark.parametrize("name", FAMILIES)
def test_oracle_decoder_matches_reference_logits(name):
    ref = load_json(name + "_logits.json")
    spec = spec_from_ref_fixture(name, O.F32, max_ctx=32)
    m = oracle_model(spec, acc64=1)
    got = run_sequences(m, ref["sequences"])
    want = np.array(ref["logits"], np.float32)
    assert got.shape == want.shape
    assert np.max(np.abs(got - want)) < 1e-4


def test_oracle_fp32_accumulation_close_to_acc64():
    ref = load_json("tiny_qwen2_logits.json")
    spec = spec_from_ref_fixture("tiny_qwen2", O.F32, max_ctx=32)
    a = run_sequences(oracle_model(spec, acc64=1), ref["sequences"])
    b = run_sequences(oracle_model(spec, acc64=0), ref["sequences"])
    assert np.max(np.abs(a - b)) < 1e-5


def test_oracle_gguf_f32_import_matches_reference_logits():
    # tests/TestNeuralPretrained.pas:6312 (TestGGUFLlamaLogitParity): GGUF F32 import end to end, stored row order
    ref = load_json("tiny_llama_logits.json")
    spec = spec_from_gguf_llama(ref_path("tiny_llama_f32.gguf"), max_ctx=32)
    got = run_sequences(oracle_model(spec, acc64=1), ref["sequences"])
    assert np.max(np.abs(got - np.array(ref["logits"], np.float32))) < 1e-4


def test_oracle_gguf_q8_import_drift_window():
    # tests/TestNeuralPretrained.pas:6343-6417: Q8_0 import drifts from the fp32 twin by (1e-3, 1.5e-1) relative
    q8 = oracle_model(spec_from_gguf_llama(ref_path("tiny_llama_q8.gguf"), max_ctx=32))
    f32 = oracle_model(spec_from_ref_fixture("tiny_llama_q8", O.F32, max_ctx=32))
    seq = [1, 5, 2, 7, 3, 0, 6, 4]
    a = run_sequences(q8, [seq]); b = run_sequences(f32, [seq])
    rel = np.max(np.abs(a - b)) / np.max(np.abs(b))
    assert 1e-3 < rel < 1.5e-1


def test_oracle_truncate_replays_identically():
    spec = spec_from_ref_fixture("tiny_llama", O.F32, max_ctx=32)
    m = oracle_model(spec)
    seq = [1, 2, 3, 4, 5, 6]
    full = run_sequences(m, [seq])[0]
    m.truncate(3)
    again = [m.step(t, p)[1] for p, t in list(enumerate(seq))[3:]]
    assert np.array_equal(np.array(again), full[3:])


def test_topk_gate_known_answer():
    # tests/TestNeuralNumerical.pas:74997-75042
    p = np.array([0.5, 0.1, 0.3, 0.1], np.float32); g = np.zeros(4, np.float32); idx = np.zeros(2, np.int32)
    O.lib().orc_topk_gate(p.ctypes.data, 4, 2, 1, g.ctypes.data, idx.ctypes.data)
    assert np.allclose(g, [0.625, 0, 0.375, 0], atol=1e-6) and list(idx) == [0, 2]


def test_argmax_lowest_index_wins_ties():
    x = np.array([1, 3, 3, 2, 3], np.float32)
    assert O.lib().orc_argmax(x.ctypes.data, 5) == 1


def test_attention_matches_bruteforce_softmax():
    rng = np.random.default_rng(0)
    hq, hkv, dk, ctx = 4, 2, 8, 11
    kc = np.zeros((hkv, ctx, dk), np.float32); vc = np.zeros_like(kc)
    rows = rng.standard_normal((ctx, (hq + 2 * hkv) * dk)).astype(np.float32)
    for window in (0, 4):
        kc[:] = 0; vc[:] = 0
        for pos in range(ctx):
            out = np.zeros(hq * dk, np.float32)
            O.lib().orc_attn_decode(rows[pos].ctypes.data, hq, hkv, dk, kc.ctypes.data, vc.ctypes.data, ctx, pos, window, 0.0, 0, out.ctypes.data)
            j0 = max(0, pos + 1 - window) if window else 0
            for h in range(hq):
                g = h // (hq // hkv)
                q = rows[pos, h * dk:(h + 1) * dk].astype(np.float64)
                K = rows[j0:pos + 1, hq * dk + g * dk: hq * dk + (g + 1) * dk].astype(np.float64)
                V = rows[j0:pos + 1, (hq + hkv) * dk + g * dk: (hq + hkv) * dk + (g + 1) * dk].astype(np.float64)
                s = K @ q / np.sqrt(dk); p = np.exp(s - s.max()); p /= p.sum()
                assert np.allclose(out[h * dk:(h + 1) * dk], p @ V, atol=2e-6)


def test_avx_baseline_kernels_match_scalar():
    rng = np.random.default_rng(4)
    for n in (1, 3, 4, 31, 32, 33, 67, 576, 3584):
        a = rng.standard_normal(n).astype(np.float32); b = rng.standard_normal(n).astype(np.float32)
        c = rng.integers(-127, 128, n).astype(np.int8)
        assert abs(O.lib().cpu_avx_dot_f32(a.ctypes.data, b.ctypes.data, n) - float(a.astype(np.float64) @ b)) < 1e-4 * max(1, n ** 0.5)
        assert abs(O.lib().cpu_avx_dot_int8(c.ctypes.data, b.ctypes.data, n) - float(c.astype(np.float64) @ b)) < 1e-3 * max(1, n ** 0.5)


def _scaled(base, hd, mode, factor, orig=0, low=1.0, high=4.0):
    import ctypes as C
    th = np.empty(hd // 2, np.float32)
    assert O.lib().orc_rope_thetas_scaled(C.c_float(base), hd, mode, C.c_float(factor), orig, C.c_float(low), C.c_float(high), th.ctypes.data) == 0
    return th


def test_rope_scaling_tables():
    """Long-context frequency rules (neural/neuralpretrained.pas:633-668).  Known answers: the saturating case the reference's
    own test describes (tests/TestNeuralNumerical.pas:16008-16028: d = 8, base 1e4, original 512, low 1, high 4 - pairs 0, 1
    keep their frequency, pairs 2, 3 are fully interpolated); linear = theta / factor; and the published Llama-3.1 rule
    written a second way (numpy float64, wavelength masks) on a 128-wide head with the Llama-3.1 constants."""
    base = np.array([1e4 ** (-2.0 * k / 8) for k in range(4)])
    th = _scaled(1e4, 8, 2, 8.0, 512, 1.0, 4.0)
    assert np.array_equal(th, np.array([base[0], base[1], base[2] / 8, base[3] / 8]).astype(np.float32))
    assert np.array_equal(_scaled(1e4, 8, 1, 4.0), (base / 4).astype(np.float32))
    assert np.array_equal(_scaled(1e4, 8, 0, 1.0), base.astype(np.float32))
    # Llama-3.1: rope_theta 5e5, factor 8, original 8192, low 1, high 4
    hd, factor, orig, low, high = 128, 8.0, 8192, 1.0, 4.0
    inv = 5e5 ** (-np.arange(0, hd, 2, dtype=np.float64) / hd)
    wavelen = 2 * np.pi / inv
    out = np.where(wavelen > orig / low, inv / factor, inv)
    smooth = (orig / wavelen - low) / (high - low)
    mid = ~(wavelen < orig / high) & ~(wavelen > orig / low)
    out = np.where(mid, (1 - smooth) * inv / factor + smooth * inv, out)
    th = _scaled(5e5, hd, 2, factor, orig, low, high)
    assert np.array_equal(th, out.astype(np.float32))
    assert mid.sum() >= 5 and (wavelen < orig / high).sum() >= 20 and (wavelen > orig / low).sum() >= 20   # all three regimes present
    # between the two limits everywhere, non-increasing in k like the unscaled table
    assert np.all(th <= inv.astype(np.float32)) and np.all(th >= (inv / factor).astype(np.float32) * (1 - 1e-7))
    assert np.all(np.diff(th) <= 0)
    # refused arguments
    import ctypes as C
    buf = np.empty(4, np.float32)
    assert O.lib().orc_rope_thetas_scaled(C.c_float(1e4), 8, 1, C.c_float(0.5), 0, C.c_float(1), C.c_float(4), buf.ctypes.data) != 0
    assert O.lib().orc_rope_thetas_scaled(C.c_float(1e4), 8, 2, C.c_float(8), 512, C.c_float(4), C.c_float(4), buf.ctypes.data) != 0


def test_rope_scaling_ntk_and_yarn_known_answers():
    """NTK: theta'_k = (base * s^(d/(d-2)))^(-2k/d) (tests/TestNeuralNumerical.pas:15869-15880, d = 8, s = 4).  YaRN: the band case
    of tests/TestNeuralNumerical.pas:15890-15990 (d = 8, base 1e4, original 512, s = 2, alpha 1, beta 32): pair 0 keeps its
    frequency, pair 1 is the half-way blend 0.075, pairs 2 and 3 are fully interpolated; temperature 0.1 ln 2 + 1."""
    import ctypes as C
    nb = 1e4 * 4.0 ** (8 / 6)
    assert np.array_equal(_scaled(1e4, 8, 3, 4.0), np.array([nb ** (-2.0 * k / 8) for k in range(4)]).astype(np.float32))
    th = _scaled(1e4, 8, 4, 2.0, 512, 1.0, 32.0)
    assert np.allclose(th, [1.0, 0.075, 0.005, 0.0005], rtol=1e-6, atol=0)
    assert th[0] == np.float32(1.0) and th[2] == np.float32(0.01 / 2) and th[3] == np.float32(0.001 / 2)
    L = O.lib()
    assert abs(L.orc_rope_out_scale(4, C.c_float(2.0)) - (0.1 * np.log(2.0) + 1.0)) < 1e-7
    assert L.orc_rope_out_scale(2, C.c_float(8.0)) == 1.0 and L.orc_rope_out_scale(0, C.c_float(1.0)) == 1.0
    # the published YaRN rule written a second way (numpy, the way HF states it) on a 128-wide head: Qwen2.5 long-context constants
    hd, base, factor, orig, bslow, bfast = 128, 1e6, 4.0, 32768, 1.0, 32.0
    pos_freqs = base ** (np.arange(0, hd, 2, dtype=np.float64) / hd)
    corr = lambda rot: hd * np.log(orig / (rot * 2 * np.pi)) / (2 * np.log(base))
    low, high = max(np.floor(corr(bfast)), 0), min(np.ceil(corr(bslow)), hd - 1)
    ramp = np.clip((np.arange(hd // 2) - low) / (high - low), 0, 1)
    extrap_factor = 1 - ramp
    inv = (1 / (factor * pos_freqs)) * (1 - extrap_factor) + (1 / pos_freqs) * extrap_factor
    assert np.allclose(_scaled(base, hd, 4, factor, orig, bslow, bfast), inv.astype(np.float32), rtol=3e-7, atol=0)
    assert 0 < low < high < hd // 2          # a genuine band inside the table
