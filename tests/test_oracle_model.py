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
