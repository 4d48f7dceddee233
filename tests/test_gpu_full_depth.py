"""Full-depth parity of the headline model: all 28 blocks of the Qwen2.5-7B shape at full width against the oracle.

The weights are the benchmark's (bench.py: seed 424242, N(0, 0.02), Q4_K body with q|k|v bias, Q8_0 embedding and head), made on
the device; their block bytes are downloaded so that the oracle and the library consume identical bytes.  An 8-token prompt
and 64 greedy tokens are stepped through both: every logits row within 1e-3 of the oracle's (relative to the row's largest
logit, the stated tolerance) and the greedy tokens identical (first index wins a tie: neural/neuralchatengine.pas:683-697).
With N(0, 0.02) weights the logits of a 152064-row head are nearly flat, so the margin between the oracle's best and second
best logit is reported per token next to the largest deviation: a token can only differ where the margin is below it.
Two more checks at the benchmarked widths sit here: the 64 tokens once more through the captured eight-step graph (the path the
benchmark times), and the large-tile forms of the prompt pass (merged q | k | v launch, gate|up product with the SwiGLU
epilogue) on one full-width block, directly against the oracle.
"""
import importlib
import time

import numpy as np
import pytest

from helpers import oracle_lib as O

pytestmark = pytest.mark.gpu
TOL = 1e-3

CFG_7B = dict(n_layers=28, d_model=3584, n_q_heads=28, n_kv_heads=4, head_dim=128, ffn=18944, vocab=152064, max_ctx=128,
              eps=1e-6, rope_theta=1e6)


def test_qwen7b_all_28_blocks_64_greedy_tokens_against_the_oracle():
    import torch
    from helpers.device import dev, rel_err
    cai = dev()
    synth = importlib.import_module("neural-api_amd.synth")
    t0 = time.time()
    spec = synth.random_decoder_spec(CFG_7B, cai.Q4_K, cai.Q8_0, seed=424242, qkv_bias=True, keep_bytes=True)
    dec = cai.Decoder(spec)
    # the oracle's copy: the very bytes the device holds (embedding and head are separate matrices here, as in the benchmark)
    ocfg = dict(CFG_7B)
    for k, v in dict(window=0, qk_norm_full=0, n_experts=0, top_k=0, norm_topk=0, kv_f16=0, acc64=1).items():
        ocfg.setdefault(k, v)
    om = O.OracleModel(O.OrcConfig(**ocfg))
    for (layer, slot), t in spec["tensors"].items():
        raw = t["raw_dev"].cpu().numpy()
        t["raw_dev"] = None
        om.set_tensor(layer, slot, t["type"], t["rows"], t["cols"], raw, None, t["bias"])
    for (layer, slot), v in spec["vecs"].items():
        om.set_vec(layer, slot, v)
    torch.cuda.empty_cache()
    t_build = time.time() - t0

    rng = np.random.default_rng(424242)
    prompt = rng.integers(0, CFG_7B["vocab"], 8).tolist()
    worst, tok_o, tok_d = 0.0, None, None
    t0 = time.time()
    for p, t in enumerate(prompt):
        tok_o, lo = om.step(t, p); am, ld = dec.step(t, p); tok_d = int(am[0])
        worst = max(worst, rel_err(ld[0], lo))
    assert worst < TOL, "prompt rows: %g" % worst
    assert tok_o == tok_d
    first = tok_d
    seq_o, seq_d, margins, devs = [], [], [], []
    for i in range(64):
        p = len(prompt) + i
        n_o, lo = om.step(tok_o, p); am, ld = dec.step(tok_d, p)
        top2 = np.partition(lo, -2)[-2:]
        scale = float(np.max(np.abs(lo)))
        margins.append(float(top2[1] - top2[0]) / scale)
        devs.append(rel_err(ld[0], lo))
        tok_o, tok_d = n_o, int(am[0])
        seq_o.append(tok_o); seq_d.append(tok_d)
        if tok_o != tok_d:
            break
    t_steps = time.time() - t0
    print("full depth: build %.0f s, 72 oracle + device steps %.0f s; largest logit deviation %.2e of the row maximum; smallest "
          "margin between the oracle's two best logits %.2e of the row maximum (token %d); per token (deviation, margin): %s"
          % (t_build, t_steps, max(devs), min(margins), int(np.argmin(margins)),
             " ".join("%.1e/%.1e" % (a, b) for a, b in zip(devs, margins))))
    assert max(devs) < TOL
    assert seq_d == seq_o, "greedy tokens differ at generated token %d (margin %.2e, deviation %.2e)" % (len(seq_o) - 1, margins[-1], devs[-1])
    # the same 64 tokens through the captured eight-step graph (cai_decoder_generate)
    dec.truncate(len(prompt))
    assert dec.generate(first, len(prompt), 64).tolist() == seq_o
    dec.close()


def test_large_tile_prompt_pass_of_one_full_width_block_against_the_oracle():
    """A 256-token prompt through ONE block of the 7B width (vocabulary cut to 1024 rows so that the oracle's 257 steps stay
    short): the prompt pass takes its large-tile forms - q | k | v as one launch with biases, the gate|up product with two row
    tiles per wave and SwiGLU in its epilogue (engaged from 193 tokens at 37888 rows), the register-resident pre-pass of the
    18944-wide row, matrix-core prompt attention - and is compared DIRECTLY with the oracle stepping token by token: last-token
    logits within 1e-3 of the row's largest logit, same arg-max, and the decode step that follows (it reads the cache rows the
    prompt pass wrote) as well."""
    from helpers.device import dev, rel_err
    from helpers.model_build import oracle_model, synthetic_spec
    cai = dev()
    cfg = dict(CFG_7B, n_layers=1, vocab=1024, max_ctx=320)
    spec = synthetic_spec(cfg, O.Q4_K, head_qtype=O.Q8_0, seed=256, qkv_bias=True, std=0.02)
    om = oracle_model(spec, acc64=1)
    dec = cai.Decoder(spec)
    rng = np.random.default_rng(256)
    prompt = rng.integers(0, cfg["vocab"], 256).tolist()
    tok_o, lo = None, None
    for p, t in enumerate(prompt):
        tok_o, lo = om.step(t, p, want_logits=(p == len(prompt) - 1))
    am, ld = dec.prefill(prompt, 0)
    assert rel_err(ld, lo) < TOL and am == tok_o
    n_o, lo = om.step(tok_o, len(prompt)); a, ld = dec.step(am, len(prompt))
    assert rel_err(ld[0], lo) < TOL and int(a[0]) == n_o
    dec.close()
