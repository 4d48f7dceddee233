"""cai_decoder_load_gguf: the library reads a llama / qwen2 file itself and must reproduce the reference's logits
(tests/fixtures/tiny_llama_logits.json, < 1e-4 as in tests/TestNeuralPretrained.pas:5819-5917) and the oracle."""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.fixtures_io import load_json, ref_path
from helpers.gguf_write import spec_to_gguf, write_gguf
from helpers.model_build import oracle_model, spec_from_gguf_llama, synthetic_spec

pytestmark = pytest.mark.gpu


def run(dec, seqs):
    out = []
    for seq in seqs:
        dec.reset()
        out.append(np.stack([dec.step(t, p)[1][0] for p, t in enumerate(seq)]))
    return np.array(out)


def test_reference_llama_files_reproduce_reference_logits():
    from helpers.device import dev, rel_err
    cai = dev()
    ref = load_json("tiny_llama_logits.json")
    want = np.array(ref["logits"], np.float32)
    dec = cai.Decoder.from_gguf(ref_path("tiny_llama_f32.gguf"), max_ctx=32)
    assert (dec.cfg.n_layers, dec.cfg.d_model, dec.cfg.n_q_heads, dec.cfg.n_kv_heads, dec.cfg.vocab) == (2, 8, 2, 1, 11)
    assert np.max(np.abs(run(dec, ref["sequences"]) - want)) < 1e-4
    dec16 = cai.Decoder.from_gguf(ref_path("tiny_llama_f16.gguf"), max_ctx=32)     # half weights: drift of the rounding only
    assert np.max(np.abs(run(dec16, ref["sequences"]) - want)) < 2e-2
    # Q8_0 file: same blocks through the oracle
    spec = spec_from_gguf_llama(ref_path("tiny_llama_q8.gguf"), max_ctx=32)
    seq = [1, 5, 2, 7, 3, 0, 6, 4, 1, 1]
    om = oracle_model(spec, acc64=1)
    want8 = np.array([om.step(t, p)[1] for p, t in enumerate(seq)])
    got8 = run(cai.Decoder.from_gguf(ref_path("tiny_llama_q8.gguf"), max_ctx=32), [seq])[0]
    assert rel_err(got8, want8) < 1e-5


def test_context_length_defaults_to_the_file(tmp_path):
    from helpers.device import dev
    cai = dev()
    dec = cai.Decoder.from_gguf(ref_path("tiny_llama_f32.gguf"))
    assert dec.cfg.max_ctx == 16


def test_qwen2_style_q4k_file_with_biases_and_untied_q8_head(tmp_path):
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=2, d_model=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=768, vocab=640, max_ctx=64, eps=1e-6, rope_theta=1e6)
    spec = synthetic_spec(cfg, O.Q4_K, head_qtype=O.Q8_0, seed=7, qkv_bias=True)
    path = str(tmp_path / "q.gguf")
    spec_to_gguf(path, spec, "qwen2")
    dec = cai.Decoder.from_gguf(path)
    om = oracle_model(spec, acc64=1)
    seq = [3, 600, 17, 17, 250, 9, 1, 0, 638, 77, 5, 5]
    want = np.array([om.step(t, p)[1] for p, t in enumerate(seq)])
    got = run(dec, [seq])[0]
    assert rel_err(got, want) < 1e-3
    assert np.array_equal(got.argmax(1), want.argmax(1))


def test_mixed_q4k_q6k_file_like_a_q4_k_m_export(tmp_path):
    """A Q4_K body whose output.weight, attn_v and ffn_down are Q6_K, the mix llama.cpp's Q4_K_M preset writes."""
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=2, head_dim=64, ffn=512, vocab=300, max_ctx=48, eps=1e-5, rope_theta=1e4)
    spec = synthetic_spec(cfg, O.Q4_K, head_qtype=O.Q6_K, seed=11)
    rng = np.random.default_rng(3)
    for l in range(cfg["n_layers"]):           # re-quantise attn_v and ffn_down as Q6_K
        for slot in (O.W_V, O.W_DOWN):
            t = spec["tensors"][(l, slot)]
            w = (rng.standard_normal((t["rows"], t["cols"])) * 0.02).astype(np.float32)
            t.update(type=O.Q6_K, raw=O.quantize(O.Q6_K, w))
    path = str(tmp_path / "m.gguf")
    spec_to_gguf(path, spec, "llama")
    dec = cai.Decoder.from_gguf(path)
    om = oracle_model(spec, acc64=1)
    seq = [3, 299, 17, 17, 250, 9, 1, 0]
    want = np.array([om.step(t, p)[1] for p, t in enumerate(seq)])
    got = run(dec, [seq])[0]
    assert rel_err(got, want) < 1e-3 and np.array_equal(got.argmax(1), want.argmax(1))


def test_loader_refuses_what_it_cannot_run(tmp_path):
    from helpers.device import dev
    cai = dev()
    base = {"general.architecture": "llama", "llama.block_count": 1, "llama.embedding_length": 32, "llama.feed_forward_length": 64,
            "llama.attention.head_count": 2, "llama.context_length": 16}
    z = lambda r, c: np.zeros((r, c), np.float32).tobytes()
    tens = [("token_embd.weight", [10, 32], 0, z(10, 32)), ("output_norm.weight", [32], 0, z(1, 32))]
    cases = []
    m = dict(base); m["general.architecture"] = "gemma2"; cases.append((m, tens, "supported: llama, qwen2"))
    m = dict(base); del m["llama.block_count"]; cases.append((m, tens, "llama.block_count"))
    cases.append((dict(base), tens, "missing tensor \"blk.0.attn_q.weight\""))
    m = dict(base); m["llama.rope.scaling.type"] = "yarn"; cases.append((m, tens, "rope.scaling.type"))
    # a BF16 embedding: sized by the container, refused by the loader (the reference has no decoder for it either)
    cases.append((dict(base), [("token_embd.weight", [10, 32], 30, bytes(10 * 64))], "ggml type 30"))
    for i, (meta, tensors, needle) in enumerate(cases):
        p = str(tmp_path / ("c%d.gguf" % i))
        write_gguf(p, meta, tensors)
        with pytest.raises(cai.CaiError) as e:
            cai.Decoder.from_gguf(p)
        assert needle in str(e.value), (needle, str(e.value))
