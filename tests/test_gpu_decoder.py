"""Step-resident decoder on the device: reference-held logits, oracle parity on quantized synthetic models,
greedy-token identity, session management.  All calls go through the C ABI."""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.device_model import run_sequences_device
from helpers.fixtures_io import load_json, ref_path
from helpers.model_build import oracle_model, spec_from_gguf_llama, spec_from_ref_fixture, synthetic_spec

pytestmark = pytest.mark.gpu
FAMILIES = ["tiny_llama", "tiny_smollm2", "tiny_qwen2", "tiny_mistral", "tiny_olmoe"]


@pytest.mark.parametrize("name", FAMILIES)
def test_device_decoder_matches_reference_logits(name):
    # the reference's own gate (tests/TestNeuralPretrained.pas:5739-5743): max |diff| < 1e-4
    from helpers.device import dev
    cai = dev()
    ref = load_json(name + "_logits.json")
    dec = cai.Decoder(spec_from_ref_fixture(name, O.F32, max_ctx=32))
    got = run_sequences_device(dec, ref["sequences"])
    assert np.max(np.abs(got - np.array(ref["logits"], np.float32))) < 1e-4


def test_device_gguf_imports_match():
    from helpers.device import dev, rel_err
    cai = dev()
    ref = load_json("tiny_llama_logits.json")
    dec = cai.Decoder(spec_from_gguf_llama(ref_path("tiny_llama_f32.gguf"), max_ctx=32))
    got = run_sequences_device(dec, ref["sequences"])
    assert np.max(np.abs(got - np.array(ref["logits"], np.float32))) < 1e-4
    # Q8_0 GGUF (hidden 32): device == oracle on the same blocks, tightly
    spec = spec_from_gguf_llama(ref_path("tiny_llama_q8.gguf"), max_ctx=32)
    seq = [1, 5, 2, 7, 3, 0, 6, 4, 1, 1]
    om = oracle_model(spec, acc64=1)
    want = np.array([om.step(t, p)[1] for p, t in enumerate(seq)])
    got = run_sequences_device(cai.Decoder(spec), [seq])[0]
    assert rel_err(got, want) < 1e-5


SHAPES = {
    # scaled-down twins of the BASELINE shapes (same head grouping / bias / MoE structure)
    "qwen7b_like_q4k": dict(cfg=dict(n_layers=3, d_model=512, n_q_heads=14, n_kv_heads=2, head_dim=128, ffn=1024, vocab=2048, max_ctx=128,
                                     eps=1e-6, rope_theta=1e6), qtype=O.Q4_K, head=O.Q8_0, bias=True),
    "smollm_like_q8": dict(cfg=dict(n_layers=3, d_model=576, n_q_heads=9, n_kv_heads=3, head_dim=64, ffn=1536, vocab=3000, max_ctx=160,
                                    eps=1e-5, rope_theta=1e4, tied=True), qtype=O.Q8_0, head=None, bias=False),
    "llama_like_q4_0": dict(cfg=dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=4, head_dim=64, ffn=512, vocab=1000, max_ctx=96,
                                     eps=1e-5, rope_theta=1e4), qtype=O.Q4_0, head=None, bias=False),
    "olmoe_like_q8": dict(cfg=dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=4, head_dim=64, ffn=128, vocab=1500, max_ctx=96,
                                   eps=1e-5, rope_theta=1e4, n_experts=16, top_k=4, norm_topk=0, qk_norm_full=1), qtype=O.Q8_0, head=None, bias=False),
    # expert banks in Q6_K (records, scales and d planes gathered per slot) and a dense Q6_K model on the integer-dot kernel
    "moe_like_q6k": dict(cfg=dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=2, head_dim=64, ffn=256, vocab=900, max_ctx=96,
                                  eps=1e-5, rope_theta=1e4, n_experts=8, top_k=2, norm_topk=1), qtype=O.Q6_K, head=None, bias=False),
    "llama_like_q6k": dict(cfg=dict(n_layers=2, d_model=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=768, vocab=1100, max_ctx=96,
                                    eps=1e-5, rope_theta=1e4), qtype=O.Q6_K, head=O.Q6_K, bias=True),
}


@pytest.mark.parametrize("name", list(SHAPES))
def test_quantized_decoder_logits_and_greedy_tokens(name):
    """Logits within 1e-3 relative of the oracle and the greedy token sequence identical for 64 tokens."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = SHAPES[name]
    spec = synthetic_spec(s["cfg"], s["qtype"], head_qtype=s["head"], qkv_bias=s["bias"], std=0.05)
    rng = np.random.default_rng(424242)
    prompt = rng.integers(0, spec["cfg"]["vocab"], 16).tolist()
    om = oracle_model(spec, acc64=1)
    dec = cai.Decoder(spec)
    worst = 0.0
    tok_o, tok_d = None, None
    for p, t in enumerate(prompt):
        tok_o, lo = om.step(t, p); am, ld = dec.step(t, p); tok_d = int(am[0])
        worst = max(worst, rel_err(ld[0], lo))
    assert worst < 1e-3
    seq_o, seq_d = [], []
    for i in range(64):
        p = len(prompt) + i
        seq_o.append(tok_o); seq_d.append(tok_d)
        n_o, lo = om.step(tok_o, p); am, ld = dec.step(tok_d, p)
        if tok_o == tok_d:
            worst = max(worst, rel_err(ld[0], lo))
        tok_o, tok_d = n_o, int(am[0])
    assert seq_o == seq_d
    assert worst < 1e-3


def test_generate_equals_step_loop_and_batch_equals_single():
    from helpers.device import dev
    cai = dev()
    s = SHAPES["qwen7b_like_q4k"]
    spec = synthetic_spec(s["cfg"], s["qtype"], head_qtype=s["head"], qkv_bias=True, std=0.05)
    dec = cai.Decoder(spec, max_batch=4)
    prompt = [5, 17, 900, 3]
    for p, t in enumerate(prompt[:-1]):
        dec.step(t, p, want_logits=False)
    snap = dec.snapshot()
    gen = dec.generate(prompt[-1], 3, 24)
    assert dec.len() == 27
    dec.restore(snap)
    assert dec.len() == 3
    tok, seq = prompt[-1], []
    for i in range(24):
        am, _ = dec.step(tok, 3 + i, want_logits=False)
        tok = int(am[0]); seq.append(tok)
    assert seq == gen.tolist()
    cai.load().cai_kv_snap_destroy(snap)
    # four independent sequences stepped together == each stepped alone
    rng = np.random.default_rng(3)
    toks = rng.integers(0, spec["cfg"]["vocab"], (4, 10))
    singles = []
    for b in range(4):
        dec.reset(0)
        singles.append([dec.step(int(toks[b, p]), p)[1][0].copy() for p in range(10)])
    for b in range(4):
        dec.reset(b)
    for p in range(10):
        _, lg = dec.step(toks[:, p], np.full(4, p))
        for b in range(4):
            assert np.max(np.abs(lg[b] - singles[b][p])) <= 1e-5 * np.max(np.abs(singles[b][p]))


@pytest.mark.parametrize("name", ["smollm_like_q8", "llama_like_q4_0"])
def test_batched_decode_of_32_weight_block_models_equals_single(name):
    """Q8_0 / Q4_0 models stepped as a batch run every linear layer on the matrix cores (width 576 ends in a short block group)."""
    from helpers.device import dev
    cai = dev()
    s = SHAPES[name]
    spec = synthetic_spec(s["cfg"], s["qtype"], head_qtype=s["head"], qkv_bias=s["bias"], std=0.05)
    dec = cai.Decoder(spec, max_batch=5)
    rng = np.random.default_rng(11)
    toks = rng.integers(0, spec["cfg"]["vocab"], (5, 12))
    singles = []
    for b in range(5):
        dec.reset(0)
        singles.append([dec.step(int(toks[b, p]), p)[1][0].copy() for p in range(12)])
    for b in range(5):
        dec.reset(b)
    for p in range(12):
        am, lg = dec.step(toks[:, p], np.full(5, p))
        for b in range(5):
            assert np.max(np.abs(lg[b] - singles[b][p])) <= 2e-5 * np.max(np.abs(singles[b][p]))
            assert int(am[b]) == int(np.argmax(singles[b][p]))


def test_batched_decode_and_prompt_of_a_q4k_q6k_mix_equal_single_steps():
    """The Q4_K_M mix (attn_v and ffn_down of every other block and the head in Q6_K, the rest Q4_K): a batch steps every
    linear layer on the matrix cores, q | k of one type and v of another sharing the partial buffer; the prompt path takes
    the Q6_K matrices through the small-batch kernels.  Both equal single-token steps."""
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=4, d_model=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=1024, vocab=600, max_ctx=64, eps=1e-5, rope_theta=1e4)
    spec = synthetic_spec(cfg, O.Q4_K, head_qtype=O.Q6_K, seed=5, std=0.05)
    rng = np.random.default_rng(4)
    for l in (0, 2):
        for slot in (O.W_V, O.W_DOWN):
            t = spec["tensors"][(l, slot)]
            w = (rng.standard_normal((t["rows"], t["cols"])) * 0.05).astype(np.float32)
            t.update(type=O.Q6_K, raw=O.quantize(O.Q6_K, w))
    dec = cai.Decoder(spec, max_batch=4)
    toks = rng.integers(0, cfg["vocab"], (4, 10))
    singles = []
    for b in range(4):
        dec.reset(0)
        singles.append([dec.step(int(toks[b, p]), p)[1][0].copy() for p in range(10)])
    om = oracle_model(spec, acc64=1)
    want0 = np.array([om.step(int(t), p)[1] for p, t in enumerate(toks[0])])
    assert rel_err(np.array(singles[0]), want0) < 1e-3
    for b in range(4):
        dec.reset(b)
    for p in range(10):
        am, lg = dec.step(toks[:, p], np.full(4, p))
        for b in range(4):
            assert rel_err(lg[b], singles[b][p]) < 1e-3
    dec.reset(1)
    am, lg = dec.prefill([int(t) for t in toks[2]], 0, seq=1)
    assert rel_err(lg, singles[2][9]) < 1e-3 and am == int(np.argmax(singles[2][9]))
    # a prompt of more than 16 tokens: the Q6_K matrices go through the prompt GEMM with split scales
    long = [int(t) for t in rng.integers(0, cfg["vocab"], 45)]
    dec.reset(0)
    last = None
    for p, t in enumerate(long):
        last = dec.step(t, p)[1][0].copy()
    dec.reset(1)
    am, lg = dec.prefill(long, 0, seq=1)
    assert rel_err(lg, last) < 1e-3 and am == int(np.argmax(last))


@pytest.mark.parametrize("name,n", [("olmoe_like_q8", 11), ("olmoe_like_q8", 45), ("moe_like_q6k", 29)])
def test_moe_prefill_equals_sequential_steps(name, n):
    """Mixture-of-experts prompts: attention half on the whole chunk, routed half per group of rows (router and top-k once
    per group, the gathered expert products per token) == token-at-a-time steps."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = SHAPES[name]
    spec = synthetic_spec(s["cfg"], s["qtype"], head_qtype=s["head"], qkv_bias=s["bias"], std=0.05)
    dec = cai.Decoder(spec, max_batch=3)
    rng = np.random.default_rng(n)
    toks = [int(t) for t in rng.integers(0, spec["cfg"]["vocab"], n)]
    last = None
    for p, t in enumerate(toks):
        _, last = dec.step(t, p)
    am, lg = dec.prefill(toks, 0, seq=1)
    assert rel_err(lg, last[0]) < 1e-3 and am == int(np.argmax(last[0]))
    assert dec.len(1) == n
    # the ingested cache continues like the stepped one
    a0, l0 = dec.step(7, n)
    dec2 = cai.Decoder(spec, max_batch=1)
    dec2.prefill(toks, 0)
    a1, l1 = dec2.step(7, n)
    assert rel_err(l1[0], l0[0]) < 1e-3


def test_prefill_equals_sequential_steps():
    from helpers.device import dev, rel_err
    cai = dev()
    s = SHAPES["smollm_like_q8"]
    spec = synthetic_spec(s["cfg"], s["qtype"], std=0.05)
    dec = cai.Decoder(spec, max_batch=2)
    toks = [3, 14, 15, 92, 65, 35, 89, 79, 32, 38, 46]
    last = None
    for p, t in enumerate(toks):
        _, last = dec.step(t, p)
    am, lg = dec.prefill(toks, 0, seq=1)
    assert rel_err(lg, last[0]) < 1e-3 and am == int(np.argmax(last[0]))
    assert dec.len(1) == len(toks)


def test_truncate_and_error_paths():
    from helpers.device import dev
    cai = dev()
    spec = spec_from_ref_fixture("tiny_llama", O.F32, max_ctx=8)
    dec = cai.Decoder(spec)
    seq = [1, 2, 3, 4, 5, 6]
    full = [dec.step(t, p)[1][0].copy() for p, t in enumerate(seq)]
    dec.truncate(3)                       # prefix reuse (neuralchatengine.pas:1434-1439)
    again = [dec.step(t, p)[1][0].copy() for p, t in list(enumerate(seq))[3:]]
    assert all(np.array_equal(a, b) for a, b in zip(again, full[3:]))
    with pytest.raises(cai.CaiError):     # wrong position
        dec.step(1, 2)
    with pytest.raises(cai.CaiError):     # token outside the vocabulary
        dec.step(9999, dec.len())
    dec.step(1, 6); dec.step(1, 7)
    with pytest.raises(cai.CaiError):     # context exhausted: refused on the host, nothing launched
        dec.step(1, 8)
    dec.reset()                           # always safe after a failed step (neuralchatengine.pas:1630-1636)
    assert np.array_equal(dec.step(seq[0], 0)[1][0], full[0])


def test_matrix_core_prefill_equals_steps_and_feeds_decode():
    """Q4_K decoder: multi-token prompt ingestion (MFMA GEMM + prompt attention) == token-at-a-time steps; a 600-token
    prompt crosses the 512-token chunk boundary; decode continues identically from either cache."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = SHAPES["qwen7b_like_q4k"]
    cfg = dict(s["cfg"]); cfg["max_ctx"] = 700
    spec = synthetic_spec(cfg, s["qtype"], head_qtype=s["head"], qkv_bias=True, std=0.05)
    dec = cai.Decoder(spec, max_batch=2)
    rng = np.random.default_rng(5)
    for n in (7, 130, 600):
        toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
        dec.reset(0); dec.reset(1)
        last = None
        for p, t in enumerate(toks):
            am_s, last = dec.step(int(t), p)
        am_p, lg = dec.prefill(toks, 0, seq=1)
        assert rel_err(lg, last[0]) < 1e-4, n
        assert am_p == int(am_s[0])
        assert dec.len(1) == n
    # continue decoding on sequence 0 after a prefill there: same tokens as after the stepped prompt
    toks = rng.integers(0, cfg["vocab"], 40).astype(np.int32)
    dec.reset(0)
    for p, t in enumerate(toks[:-1]):
        dec.step(int(t), p, want_logits=False)
    a = dec.generate(int(toks[-1]), 39, 16)
    dec.reset(0)
    dec.prefill(toks[:-1], 0, seq=0, want_logits=False)
    b = dec.generate(int(toks[-1]), 39, 16)
    assert a.tolist() == b.tolist()


def test_int8_kv_cache_decoder():
    """Session over an int8 KV cache (TNNetStreamingDecoder with pInt8KV, neural/neuraldecode.pas:5775-5840): close to
    the oracle run with the same cache model (codes may differ by one step where the two K,V rows differ in the last
    bits), prompt ingestion and batch stepping agree with single steps, snapshot/restore replays exactly."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = SHAPES["qwen7b_like_q4k"]
    spec = synthetic_spec(s["cfg"], s["qtype"], head_qtype=s["head"], qkv_bias=True, std=0.05)
    rng = np.random.default_rng(77)
    toks = rng.integers(0, spec["cfg"]["vocab"], 40).tolist()
    om = oracle_model(spec, acc64=1, kv_f16=2)
    of = oracle_model(spec, acc64=1)
    dec = cai.Decoder(spec, max_batch=2, kv_dtype=cai.KV_I8)
    worst, drift, steps = 0.0, 0.0, []
    for p, t in enumerate(toks):
        _, lo = om.step(t, p); _, lf = of.step(t, p); _, ld = dec.step(t, p)
        steps.append(ld[0].copy())
        worst = max(worst, rel_err(ld[0], lo)); drift = max(drift, rel_err(ld[0], lf))
    assert worst < 5e-3, worst            # device int8 cache vs oracle int8 cache
    assert drift < 5e-2, drift            # int8 cache vs fp32 cache: the quantisation itself
    am, lg = dec.prefill(toks, 0, seq=1)  # prompt path: rows quantised by the append kernel, attention over codes
    assert rel_err(lg, steps[-1]) < 2e-3 and dec.len(1) == len(toks)
    dec.truncate(20); snap = dec.snapshot()
    a = [dec.step(t, 20 + i)[1][0].copy() for i, t in enumerate(toks[20:30])]
    dec.restore(snap)
    b = [dec.step(t, 20 + i)[1][0].copy() for i, t in enumerate(toks[20:30])]
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    assert all(np.array_equal(x, y) for x, y in zip(a, steps[20:30]))
    cai.load().cai_kv_snap_destroy(snap)


def test_streaming_eviction_session_runs_past_max_ctx():
    """TNNetStreamingDecoder.EnableEviction (neural/neuraldecode.pas:1257-1276): logits follow the oracle's position
    mask while the stream runs to three times max_ctx; generate, prefill and the int8 cache work under it."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = SHAPES["llama_like_q4_0"]
    cfg = dict(s["cfg"]); cfg["max_ctx"] = 48
    spec = synthetic_spec(cfg, s["qtype"], std=0.05)
    sinks, recent, n = 4, 36, 150
    rng = np.random.default_rng(99)
    toks = rng.integers(0, cfg["vocab"], n).tolist()
    om = oracle_model(spec, acc64=1, max_ctx=n + 8, evict_sinks=sinks, evict_recent=recent)
    dec = cai.Decoder(spec, max_batch=2)
    dec.set_eviction(sinks, recent)
    worst = 0.0
    for p, t in enumerate(toks):
        _, lo = om.step(t, p); _, ld = dec.step(t, p)
        worst = max(worst, rel_err(ld[0], lo))
        assert dec.cache_rows(0, 1) == min(p + 1, sinks + recent) and dec.len() == p + 1
    assert worst < 1e-3, worst
    # chained greedy generation under eviction == step loop
    snap = dec.snapshot()
    gen = dec.generate(toks[-1] % cfg["vocab"], n, 30)
    dec.restore(snap)
    tok, seq = toks[-1] % cfg["vocab"], []
    for i in range(30):
        am, _ = dec.step(tok, n + i, want_logits=False)
        tok = int(am[0]); seq.append(tok)
    assert seq == gen.tolist()
    cai.load().cai_kv_snap_destroy(snap)
    # a prompt longer than the cap is ingested token by token and lands on the same logits
    _, last = dec.prefill(toks[:100], 0, seq=1)
    om2 = oracle_model(spec, acc64=1, max_ctx=n + 8, evict_sinks=sinks, evict_recent=recent)
    for p, t in enumerate(toks[:100]):
        _, lo = om2.step(t, p)
    assert rel_err(last, lo) < 1e-3
    # storage mode switch on a fresh session only (EnableInt8KVCache)
    with pytest.raises(cai.CaiError):
        dec.set_kv_dtype(cai.KV_I8)
    dec.reset(0); dec.reset(1)
    dec.set_kv_dtype(cai.KV_I8)
    drift = 0.0
    om3 = oracle_model(spec, acc64=1, max_ctx=n + 8, evict_sinks=sinks, evict_recent=recent)
    for p, t in enumerate(toks[:80]):
        _, lo = om3.step(t, p); _, ld = dec.step(t, p)
        drift = max(drift, rel_err(ld[0], lo))
    assert drift < 5e-2, drift


@pytest.mark.parametrize("kv,window", [("f32", 0), ("f16", 0), ("f32", 40), ("f16", 70), ("i8", 0), ("i8", 50)])
def test_prompt_attention_on_matrix_cores_equals_steps(kv, window):
    """Prompt ingestion over a 128-wide cache runs the matrix-core attention kernel (32 tokens x 4 heads per
    work-group): the last token's logits equal token-at-a-time ingestion for fp32, fp16 and int8 caches, under a sliding
    window, for prompt lengths that are not multiples of the tile and for a continuation from position > 0."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = SHAPES["qwen7b_like_q4k"]
    cfg = dict(s["cfg"]); cfg["max_ctx"] = 200; cfg["window"] = window
    spec = synthetic_spec(cfg, s["qtype"], head_qtype=s["head"], qkv_bias=True, std=0.05)
    dec = cai.Decoder(spec, max_batch=2, kv_dtype={"f32": cai.KV_F32, "f16": cai.KV_F16, "i8": cai.KV_I8}[kv])
    rng = np.random.default_rng(11)
    # int8: the two routes compute K and V rows that differ in the last bits, so now and then a code lands one step apart
    tol = 5e-3 if kv == "i8" else 2e-4
    for n in (33, 97, 160):
        toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
        dec.reset(0); dec.reset(1)
        for p, t in enumerate(toks):
            am_s, last = dec.step(int(t), p)
        am_p, lg = dec.prefill(toks, 0, seq=1)
        assert rel_err(lg, last[0]) < tol, (n, rel_err(lg, last[0]))
        if kv != "i8":
            assert am_p == int(am_s[0])
    # a second piece appended at position 50: attends over the rows of the first
    toks = rng.integers(0, cfg["vocab"], 120).astype(np.int32)
    dec.reset(0); dec.reset(1)
    for p, t in enumerate(toks):
        _, last = dec.step(int(t), p)
    dec.prefill(toks[:50], 0, seq=1, want_logits=False)
    _, lg = dec.prefill(toks[50:], 50, seq=1)
    assert rel_err(lg, last[0]) < tol


@pytest.mark.parametrize("name", ["qwen7b_like_q4k", "olmoe_like_q8"])
def test_per_class_timing_leaves_the_session_as_it_found_it(name):
    """cai_decoder_profile (a measurement aid without a counterpart in the reference) replays whole steps and steps without one
    class of launches at the current position.  It must not advance the session, and the step that follows must give what it
    gives without the timing pass in between; the classes it reports are finite and the large ones positive."""
    from helpers.device import dev
    cai = dev()
    s = SHAPES[name]
    spec = synthetic_spec(s["cfg"], s["qtype"], head_qtype=s["head"], qkv_bias=s["bias"], std=0.05)
    dec = cai.Decoder(spec)
    toks = [3, 17, 256, 9, 41, 5]
    for p, t in enumerate(toks[:-1]):
        dec.step(t, p, want_logits=False)
    _, want = dec.step(toks[-1], 5)
    dec.truncate(5)
    us = dec.profile(toks[-1], reps=4)
    assert dec.len() == 5
    assert np.isfinite(us).all() and us[4] > 0 and us[1] > 0 and us.sum() > 0
    _, got = dec.step(toks[-1], 5)
    assert np.array_equal(got, want)


def test_session_beyond_32768_rows_prompt_pass_and_decode_step_agree():
    """A 66 000-token session (258 cache slices): the prompt pass ingests the history through the matrix-core attention kernel,
    the decode step then walks the 66 000 cached rows with the split kernels; the same last token taken both ways must give the
    same logits.  (The stand-alone attention test pins such caches to the oracle; this covers the session plumbing: chunked
    ingestion, positions, captured step graph at that length.)"""
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=1, d_model=256, n_q_heads=2, n_kv_heads=1, head_dim=128, ffn=256, vocab=300, max_ctx=66100, eps=1e-5, rope_theta=1e6)
    spec = synthetic_spec(cfg, O.Q8_0, std=0.05)
    dec = cai.Decoder(spec, max_batch=2, kv_dtype=cai.KV_F16)
    rng = np.random.default_rng(66)
    toks = rng.integers(0, cfg["vocab"], 66000).astype(np.int32)
    dec.prefill(toks[:-1], 0, seq=0, want_logits=False)
    am_a, la = dec.step_window([int(toks[-1])], 65999, seq=0)
    am_b, lb = dec.prefill(toks, 0, seq=1)
    assert dec.len(0) == 66000 and dec.len(1) == 66000
    assert rel_err(la[0], lb) < 2e-4 and int(am_a[0]) == am_b
    g = dec.generate(int(am_a[0]), 66000, 4)
    assert dec.len(0) == 66004 and len(g) == 4
    dec.close()


@pytest.mark.parametrize("kv", [0, 1])
def test_attention_geometry_follows_the_session_length_across_bucket_boundaries(kv):
    """The slice geometry of the decode attention follows the rows in use (buckets of 1024 * 2^b rows, one captured graph per
    bucket), not max_ctx.  A session created for 5000 rows is walked across the 1024- and 2048-row boundaries by single steps,
    by the eight-step generation graph, by windows and by a batch whose sequences sit in different buckets; every logits row
    against the oracle."""
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=2, head_dim=64, ffn=256, vocab=400, max_ctx=5000, eps=1e-5, rope_theta=1e4)
    spec = synthetic_spec(cfg, O.Q8_0, std=0.05)
    om = oracle_model(spec, acc64=1, kv_f16=kv)
    dec = cai.Decoder(spec, max_batch=2, kv_dtype=kv)
    rng = np.random.default_rng(12)
    toks = rng.integers(0, cfg["vocab"], 2100).tolist()
    ref = [om.step(t, p) for p, t in enumerate(toks)]
    # 1010 tokens by a prompt pass, then single steps over the first boundary
    dec.prefill(toks[:1010], 0, want_logits=False)
    for p in range(1010, 1030):
        _, lg = dec.step(toks[p], p)
        assert rel_err(lg[0], ref[p][1]) < 1e-3, p
    # back to 1018 and on with the generation graph (eight steps per launch straddle row 1024)
    dec.truncate(1018)
    g = dec.generate(toks[1018], 1018, 20).tolist()
    cur, p = toks[1018], 1018
    om.truncate(1018)
    for t in g:
        am, lg = om.step(cur, p)
        if am != t:
            top2 = np.sort(lg)[-2:]; assert top2[1] - top2[0] < 2e-3 * np.max(np.abs(lg)), p
        cur, p = t, p + 1
    # windows over the boundary, on fresh history
    dec.truncate(1010); om.truncate(1010)
    for p in range(1010, 1018): om.step(toks[p], p)
    dec.step_window(toks[1010:1018], 1010, want_logits=False)
    am, lg = dec.step_window(toks[1018:1026], 1018)
    for r in range(8):
        assert rel_err(lg[r], ref[1018 + r][1]) < 1e-3, r
    # second boundary by a prompt pass that ends behind it, then steps
    dec.prefill(toks[1026:2060], 1026, want_logits=False)
    for p in range(2060, 2070):
        _, lg = dec.step(toks[p], p)
        assert rel_err(lg[0], ref[p][1]) < 1e-3, p
    # a batch whose sequences are in different buckets: the longer one decides the geometry
    dec.prefill(toks[:300], 0, seq=1, want_logits=False)
    _, lg = dec.step([toks[2070], toks[300]], [2070, 300])
    assert rel_err(lg[0], ref[2070][1]) < 1e-3 and rel_err(lg[1], ref[300][1]) < 1e-3
    dec.close()


def test_rotary_positions_far_beyond_32768_in_a_rolling_session():
    """Positions up to 70 000 through the kernels that rotate q and k inside attention (a session with eviction keeps only sinks +
    recent rows, so the stream runs far past max_ctx): the device generates 70 000 greedy tokens, the oracle is fed the same tokens
    and the logits of steps at positions 40 000, 69 990.. are compared (angle = fp32 position x frequency as in
    neural/neural.cl:1517-1542; an inaccurate sine / cosine at large arguments would show here)."""
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=1, d_model=256, n_q_heads=2, n_kv_heads=1, head_dim=128, ffn=256, vocab=300, max_ctx=64, eps=1e-5, rope_theta=1e4)
    spec = synthetic_spec(cfg, O.Q8_0, std=0.05)
    dec = cai.Decoder(spec)
    dec.set_eviction(2, 30)
    om = oracle_model(spec, acc64=1, max_ctx=70100, evict_sinks=2, evict_recent=30)
    toks = [7]
    pos = 0
    for target in (40000, 69990):
        out = []
        while pos + len(out) < target:                    # cai_decoder_generate takes at most max_ctx tokens per call
            n = min(64, target - pos - len(out))
            out += dec.generate(toks[-1] if not out else out[-1], pos + len(out), n).tolist()
        # the oracle takes the device's tokens as inputs (greedy ties would otherwise fork the two histories)
        for i, t in enumerate([toks[-1]] + out[:-1]):
            om.step(t, pos + i, want_logits=False)
        pos += len(out); toks.append(out[-1])
        for i in range(5):
            t = int(toks[-1])
            _, lo = om.step(t, pos); am, ld = dec.step(t, pos)
            assert rel_err(ld[0], lo) < 1e-3, (pos, rel_err(ld[0], lo))
            pos += 1; toks.append(int(am[0]))
    dec.close()
