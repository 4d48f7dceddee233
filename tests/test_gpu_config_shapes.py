"""Oracle parity at the shapes the published figures are measured on (BASELINE configs 2-5 at their real widths).

The kernels choose their geometry (waves per row, rows per group, K slices, ring depth) from the shape, so a scaled-down
twin does not exercise the instance a benchmark times.  Each case here runs the real width through the C ABI and compares
with the oracle's dequantise-then-dot definition accumulated in double (TIGHT = 2e-5 of the largest output; the north-star
bar for logits is 1e-3).  Matrices are built in row chunks so the float copy never exists whole.
"""
import ctypes as C

import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.model_build import oracle_model, synthetic_spec

pytestmark = pytest.mark.gpu
TIGHT = 2e-5
TOL = 1e-3


def big_matrix(qt, rows, cols, seed, std=0.02, chunk=8192):
    rng = np.random.default_rng(seed)
    rb = O.row_bytes(qt, cols)
    raw = np.empty(rows * rb, np.uint8)
    for r0 in range(0, rows, chunk):
        n = min(chunk, rows - r0)
        raw[r0 * rb:(r0 + n) * rb] = O.quantize(qt, rng.standard_normal((n, cols), dtype=np.float32) * np.float32(std))
    return raw, rng


def oracle_gateup(raw, rows, cols, x, gain, eps):
    """TokenRMSNorm -> gate|up projection -> SwiGLU with the oracle's own pieces (up = rows 0..I-1, gate = rows I..2I-1)."""
    L = O.lib()
    out = np.empty((x.shape[0], rows // 2), np.float32)
    for b in range(x.shape[0]):
        h = x[b].copy()
        if gain is not None:
            L.orc_rmsnorm(C.c_void_p(x[b].ctypes.data), C.c_void_p(gain.ctypes.data), cols, C.c_float(eps), C.c_void_p(h.ctypes.data))
        ug = O.gemv(O.Q4_K, raw, rows, cols, h, None, 0, 1)[0]
        L.orc_swiglu(C.c_void_p(ug.ctypes.data), rows // 2, C.c_void_p(out[b].ctypes.data))
    return out


@pytest.mark.parametrize("rows,cols", [(37888, 3584), (55296, 5120)])
def test_ffn_gateup_at_the_benchmarked_shapes(rows, cols):
    """cai_ffn_gateup on the 7B (the launch the roofline figure times) and 32B gate|up matrices, with and without the fused
    RMSNorm, batch 1; the SwiGLU output is compared (its scale is that of up * gate, so the floor is the typical product)."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = big_matrix(O.Q4_K, rows, cols, rows + cols)
    w = cai.QWeight(O.Q4_K, rows, cols, raw)
    x = (rng.standard_normal((1, cols)) * 1.7).astype(np.float32)
    gain = (1.0 + 0.2 * rng.standard_normal(cols)).astype(np.float32)
    for g in (gain, None):
        got = w.ffn_gateup(x, g, 1e-6)
        want = oracle_gateup(raw, rows, cols, x, g, 1e-6)
        assert got.shape == want.shape
        assert rel_err(got, want) < TIGHT, "gain" if g is not None else "no gain"
    # the plain product of the same matrix (both halves as rows), which shares the geometry choice but not the epilogue
    got = w.gemv(x)
    assert rel_err(got, O.gemv(O.Q4_K, raw, rows, cols, x, None, 0, 1), floor=0.02 * cols ** 0.5) < TIGHT
    w.close()


@pytest.mark.parametrize("rows,cols", [(5120, 5120), (1024, 5120), (5120, 27648), (152064, 5120)])
def test_q4_k_gemv_at_the_32b_shapes(rows, cols):
    """Qwen2.5-32B widths: 5120 columns = 20 super-blocks (five waves of 4 super-blocks x 4 rows), 27648 = 108; batch 1 (integer-dot
    kernel) and batch 8 (matrix-core small-batch kernel); bias included."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = big_matrix(O.Q4_K, rows, cols, rows * 3 + cols)
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(O.Q4_K, rows, cols, raw, bias)
    x = rng.standard_normal((8, cols)).astype(np.float32)
    want = O.gemv(O.Q4_K, raw, rows, cols, x, bias, 0, 1)
    got1 = w.gemv(x[:1])
    assert rel_err(got1, want[:1], floor=0.02 * cols ** 0.5) < TIGHT
    got8 = w.gemv(x)
    for b in range(8):
        assert rel_err(got8[b], want[b], floor=0.02 * cols ** 0.5) < TIGHT, b
    w.close()


@pytest.mark.parametrize("rows,cols", [(38864, 768), (6864, 4352), (3152, 9472), (17456, 1792)])
def test_q4_k_one_launch_small_batch_form_on_awkward_shapes(rows, cols):
    """The one-launch small-batch form of Q4_K (a batch of cai_qgemv on a matrix of 16 MiB or more) where its geometry has
    remainders: an odd number of super-blocks (768 = 3: the last wave of a work-group covers one, not two), widths cut into
    column slices that the last work-group to arrive adds up (4352 = 17 super-blocks: two slices, 9472 = 37: three), row counts
    that are an odd number of 16-row sets (units of 16 rows), 2, 3, 5 and 8 tokens; against the float64-accumulated oracle,
    with bias."""
    from helpers.device import dev, rel_err
    cai = dev()
    assert rows % 16 == 0 and (rows // 16) % 2 == 1 and rows * cols * 144 // 256 >= 16 << 20
    raw, rng = big_matrix(O.Q4_K, rows, cols, rows + 7 * cols)
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(O.Q4_K, rows, cols, raw, bias)
    x = rng.standard_normal((8, cols)).astype(np.float32)
    x[3] *= 40.0                       # tokens of different magnitude: the block scales are per token
    x[5, : cols // 2] = 0.0            # whole zero blocks
    want = O.gemv(O.Q4_K, raw, rows, cols, x, bias, 0, 1)
    for nb in (2, 3, 5, 8):
        got = w.gemv(x[:nb])
        for b in range(nb):
            assert rel_err(got[b], want[b], floor=0.02 * cols ** 0.5 * (40.0 if b == 3 else 1.0)) < TIGHT, (nb, b)
    w.close()


@pytest.mark.parametrize("qt", [O.Q8_0, O.Q4_0])
@pytest.mark.parametrize("rows,cols", [(18944, 3584), (152064, 3584)])
def test_q8_0_q4_0_gemv_at_the_large_sweep_shapes(qt, rows, cols):
    """The two large shapes of the isolated GEMV sweep at batch 1 and 4 for both 32-weight block types."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = big_matrix(qt, rows, cols, rows + cols + qt)
    w = cai.QWeight(qt, rows, cols, raw)
    x = rng.standard_normal((4, cols)).astype(np.float32)
    want = O.gemv(qt, raw, rows, cols, x, None, 0, 1)
    assert rel_err(w.gemv(x[:1]), want[:1], floor=0.02 * cols ** 0.5) < TIGHT
    got4 = w.gemv(x)
    for b in range(4):
        assert rel_err(got4[b], want[b], floor=0.02 * cols ** 0.5) < TIGHT, b
    w.close()


def full_width_spec(cfg, qtype, head_qtype, qkv_bias, seed):
    """synthetic_spec with the embedding sharing the head's bytes: two vocab-sized matrices need only be built once."""
    c = dict(cfg, tied=True)
    spec = synthetic_spec(c, qtype, head_qtype=head_qtype, seed=seed, qkv_bias=qkv_bias, std=0.02)
    spec["tensors"][(-1, O.W_HEAD)] = dict(spec["tensors"][(-1, O.W_EMBED)])    # untied slot, same bytes
    return spec


TWINS = {
    # two blocks at the full widths of BASELINE configs 3, 5 and 4
    "qwen2.5-7b": dict(cfg=dict(n_layers=2, d_model=3584, n_q_heads=28, n_kv_heads=4, head_dim=128, ffn=18944, vocab=152064, max_ctx=64,
                                eps=1e-6, rope_theta=1e6), qtype=O.Q4_K, head=O.Q8_0, bias=True, kv_f16=0),
    "qwen2.5-32b": dict(cfg=dict(n_layers=2, d_model=5120, n_q_heads=40, n_kv_heads=8, head_dim=128, ffn=27648, vocab=152064, max_ctx=64,
                                 eps=1e-6, rope_theta=1e6), qtype=O.Q4_K, head=O.Q4_K, bias=True, kv_f16=1),
    "olmoe-1b-7b": dict(cfg=dict(n_layers=2, d_model=2048, n_q_heads=16, n_kv_heads=16, head_dim=128, ffn=1024, vocab=50304, max_ctx=64,
                                 eps=1e-5, rope_theta=1e4, n_experts=64, top_k=8, norm_topk=0, qk_norm_full=1), qtype=O.Q8_0, head=O.Q8_0, bias=False, kv_f16=0),
}


@pytest.mark.parametrize("name", list(TWINS))
def test_full_width_two_block_decoder_against_the_oracle(name):
    """8 prompt tokens + 16 greedy tokens, one step at a time: every logits row within 1e-3 of the oracle's (relative to the
    row's largest logit) and the greedy tokens identical; then the same 16 tokens once more through cai_decoder_generate
    (the captured-graph path the benchmark times)."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = TWINS[name]
    spec = full_width_spec(s["cfg"], s["qtype"], s["head"], s["bias"], seed=424242)
    om = oracle_model(spec, acc64=1, kv_f16=s["kv_f16"])
    dec = cai.Decoder(spec, kv_dtype=cai.KV_F16 if s["kv_f16"] else cai.KV_F32)
    rng = np.random.default_rng(424242)
    prompt = rng.integers(0, s["cfg"]["vocab"], 8).tolist()
    worst, tok_o, tok_d = 0.0, None, None
    for p, t in enumerate(prompt):
        tok_o, lo = om.step(t, p); am, ld = dec.step(t, p); tok_d = int(am[0])
        worst = max(worst, rel_err(ld[0], lo))
    assert worst < TOL
    first = tok_d
    seq_o, seq_d = [], []
    for i in range(16):
        p = len(prompt) + i
        n_o, lo = om.step(tok_o, p); am, ld = dec.step(tok_d, p)
        if tok_o == tok_d:
            worst = max(worst, rel_err(ld[0], lo))
        tok_o, tok_d = n_o, int(am[0])
        seq_o.append(tok_o); seq_d.append(tok_d)
    assert seq_o == seq_d
    assert worst < TOL
    dec.truncate(len(prompt))
    assert dec.generate(first, len(prompt), 16).tolist() == seq_o
    dec.close()


def test_olmoe_width_prompt_grouped_by_expert_against_the_oracle():
    """A 40-token prompt through two OLMoE-width blocks (64 experts, top-8, I = 1024, H = 2048, Q8_0): the prompt path sorts the
    320 (token, rank) slots by expert and runs gate|up and down as one launch each over the bank; last-token logits within
    1e-3 of the oracle stepping token by token, same arg-max, and decoding continues from the ingested cache like the oracle."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = TWINS["olmoe-1b-7b"]
    spec = full_width_spec(s["cfg"], s["qtype"], s["head"], s["bias"], seed=77)
    om = oracle_model(spec, acc64=1)
    dec = cai.Decoder(spec)
    rng = np.random.default_rng(77)
    prompt = rng.integers(0, s["cfg"]["vocab"], 40).tolist()
    tok_o, lo = None, None
    for p, t in enumerate(prompt):
        tok_o, lo = om.step(t, p)
    am, ld = dec.prefill(prompt, 0)
    assert rel_err(ld, lo) < TOL and am == tok_o
    for i in range(4):
        p = len(prompt) + i
        n_o, lo = om.step(tok_o, p); a, ld = dec.step(am, p)
        assert rel_err(ld[0], lo) < TOL and int(a[0]) == n_o
        tok_o, am = n_o, int(a[0])
    dec.close()


@pytest.mark.parametrize("name,n_tok", [("qwen2.5-7b", 230), ("qwen2.5-32b", 150)])
def test_full_width_prompt_pass_equals_token_at_a_time(name, n_tok):
    """A prompt long enough for the full-width prompt pass to take its large-tile forms (q | k | v as one launch with biases,
    SwiGLU in the epilogue of the gate|up product - engaged from 193 tokens at 37888 rows, from 129 at 55296 -, the
    register-resident pre-pass of the 18944- / 27648-wide row) against the same tokens ingested one step at a time, whose
    kernels the test above pins to the oracle at these widths: last-token logits within 2e-4 of the row's largest logit, same
    arg-max, and the decode step that follows agrees too (the caches hold the same rows)."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = TWINS[name]
    cfg = dict(s["cfg"], max_ctx=256)
    spec = full_width_spec(cfg, s["qtype"], s["head"], s["bias"], seed=99)
    kvd = cai.KV_F16 if s["kv_f16"] else cai.KV_F32
    rng = np.random.default_rng(99)
    prompt = rng.integers(0, cfg["vocab"], n_tok).tolist()
    a = cai.Decoder(spec, kv_dtype=kvd)
    am_s, l_s = None, None
    for p, t in enumerate(prompt):
        am_s, l_s = a.step(t, p)
    nxt_s, l2_s = a.step(int(am_s[0]), n_tok)
    a.close()
    b = cai.Decoder(spec, kv_dtype=kvd)
    am_p, l_p = b.prefill(prompt, 0)
    assert rel_err(l_p, l_s[0]) < 2e-4 and am_p == int(am_s[0])
    nxt_p, l2_p = b.step(am_p, n_tok)
    assert rel_err(l2_p[0], l2_s[0]) < 2e-4 and int(nxt_p[0]) == int(nxt_s[0])
    b.close()


@pytest.mark.parametrize("name", ["qwen2.5-7b", "qwen2.5-32b"])
def test_full_width_window_step_equals_token_at_a_time(name):
    """A width-8 window of one sequence (the verify pass of speculative decoding, neural/neuraldecode.pas:1151-1183) on the
    full-width twins, over a cache long enough (4096 rows) for the window's attention to take the grouped multi-slice form:
    every row within 2e-4 of the width-1 step at the same position (whose kernels the tests above pin to the oracle), same
    arg-max, and after committing five of the eight rows the next width-1 step agrees as well."""
    from helpers.device import dev, rel_err
    cai = dev()
    s = TWINS[name]
    cfg = dict(s["cfg"], max_ctx=4096)
    spec = full_width_spec(cfg, s["qtype"], s["head"], s["bias"], seed=123)
    rng = np.random.default_rng(123)
    toks = rng.integers(0, cfg["vocab"], 40).tolist()
    dec = cai.Decoder(spec, kv_dtype=cai.KV_F16 if s["kv_f16"] else cai.KV_F32)
    dec.prefill(toks[:24], 0, want_logits=False)
    single = [dec.step(t, 24 + i) for i, t in enumerate(toks[24:33])]
    dec.truncate(24)
    am, lg = dec.step_window(toks[24:32], 24)
    for r in range(8):
        assert rel_err(lg[r], single[r][1][0]) < 2e-4, r
        assert int(am[r]) == int(single[r][0][0]), r
    dec.truncate(29)
    nxt, l1 = dec.step(toks[29], 29)
    assert rel_err(l1[0], single[5][1][0]) < 2e-4 and int(nxt[0]) == int(single[5][0][0])
    dec.close()
