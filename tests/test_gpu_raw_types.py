"""The GGUF block types that stay resident as the stored stream (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K) through the C ABI:
dequantisation bit-exact (golden vectors and arbitrary bytes), the matrix-vector kernel against the oracle's
dequantise-then-dot in double, and a decoder whose file mixes Q5_K and Q6_K the way llama.cpp's Q5_K_M preset does."""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.fixtures_io import GGUFFile, load_json, ref_path
from helpers.model_build import oracle_model, synthetic_spec

pytestmark = pytest.mark.gpu
TIGHT = 2e-5
TOL = 1e-3
RAW = [O.Q5_K, O.Q2_K, O.Q3_K, O.Q4_1, O.Q5_0, O.Q5_1]


@pytest.mark.parametrize("name,qt", [("Q5_K", O.Q5_K), ("Q2_K", O.Q2_K)])
def test_reference_golden_bit_exact_on_device(name, qt):
    from helpers.device import dev
    cai = dev()
    t, shape, raw = GGUFFile(ref_path("tiny_kquant.gguf")).raw("kq.%s.weight" % name)
    w = cai.QWeight(qt, 4, 256, raw)
    want = np.array(load_json("tiny_kquant_ref.json")["dequant"][name], np.float32)
    assert np.array_equal(w.dequant_rows().reshape(-1).view(np.uint32), want.view(np.uint32))
    w.close()


@pytest.mark.parametrize("qt", RAW)
def test_random_bytes_bit_exact(qt):
    """Arbitrary block bytes: every code, packed scale and plane bit; the half fields kept finite."""
    from helpers.device import dev
    from test_oracle_codecs_other import random_blocks
    cai = dev()
    rows, cols = 37, 1024
    be = 256 if qt in (O.Q5_K, O.Q2_K, O.Q3_K) else 32
    raw = random_blocks(qt, rows * cols // be, seed=900 + qt).reshape(-1)
    w = cai.QWeight(qt, rows, cols, raw)
    got = w.dequant_rows()
    want = O.dequant(qt, raw, rows * cols).reshape(rows, cols)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # a window of rows, as the row-streaming loader asks for
    assert np.array_equal(w.dequant_rows(5, 9).view(np.uint32), want[5:14].view(np.uint32))
    w.close()


@pytest.mark.parametrize("qt", RAW)
@pytest.mark.parametrize("rows,cols", [(2048, 2048), (3, 256), (1, 9728), (1000, 3584), (64, 18944), (1001, 5120), (77, 4352)])
def test_gemv_matches_oracle(qt, rows, cols):
    from helpers.device import dev, rel_err
    cai = dev()
    rng = np.random.default_rng(rows * 7 + cols + qt)
    raw = O.quantize(qt, (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(qt, rows, cols, raw, bias)
    for nb in (1, 3, 8):
        x = rng.standard_normal((nb, cols)).astype(np.float32)
        got = w.gemv(x)
        want = O.gemv(qt, raw, rows, cols, x, bias, 0, 1)
        assert got.shape == want.shape
        assert rel_err(got, want, floor=0.02 * cols ** 0.5) < TIGHT, nb
    w.close()


@pytest.mark.parametrize("qt,rows,cols", [(O.Q4_1, 96, 160), (O.Q5_0, 576, 576), (O.Q5_1, 5, 32), (O.Q5_0, 192, 1536)])
def test_gemv_widths_that_are_not_whole_super_blocks(qt, rows, cols):
    from helpers.device import dev, rel_err
    cai = dev()
    rng = np.random.default_rng(cols + qt)
    raw = O.quantize(qt, (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32))
    w = cai.QWeight(qt, rows, cols, raw)
    for nb in (1, 2, 5):
        x = rng.standard_normal((nb, cols)).astype(np.float32)
        assert rel_err(w.gemv(x, act=cai.ACT_TANH if nb == 2 else 0), O.gemv(qt, raw, rows, cols, x, None, 3 if nb == 2 else 0, 1)) < TIGHT
    w.close()


def test_width_that_splits_a_block_is_refused():
    from helpers.device import dev
    cai = dev()
    with pytest.raises(cai.CaiError):
        cai.QWeight(O.Q5_K, 2, 384, np.zeros(2 * 264, np.uint8))
    with pytest.raises(cai.CaiError):
        cai.QWeight(O.Q5_0, 2, 48, np.zeros(2 * 33, np.uint8))


def q5_k_m_spec(cfg, seed):
    """Q5_K body; attn_v and ffn_down of every other block and the head in Q6_K (the Q5_K_M preset)."""
    spec = synthetic_spec(cfg, O.Q5_K, head_qtype=O.Q6_K, seed=seed, std=0.05, qkv_bias=True)
    rng = np.random.default_rng(seed + 1)
    for l in range(0, cfg["n_layers"], 2):
        for slot in (O.W_V, O.W_DOWN):
            t = spec["tensors"][(l, slot)]
            w = (rng.standard_normal((t["rows"], t["cols"])) * 0.05).astype(np.float32)
            t.update(type=O.Q6_K, raw=O.quantize(O.Q6_K, w))
    return spec


def test_q5_k_m_like_decoder_logits_greedy_tokens_batch_and_prompt():
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=4, d_model=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=1024, vocab=600, max_ctx=96, eps=1e-5, rope_theta=1e4)
    spec = q5_k_m_spec(cfg, 21)
    om = oracle_model(spec, acc64=1)
    dec = cai.Decoder(spec, max_batch=4)
    rng = np.random.default_rng(8)
    prompt = [int(t) for t in rng.integers(0, cfg["vocab"], 6)]
    tok_o = tok_d = None
    worst = 0.0
    singles = []
    for p, t in enumerate(prompt):
        tok_o, lo = om.step(t, p); am, ld = dec.step(t, p); tok_d = int(am[0])
        worst = max(worst, rel_err(ld[0], lo)); singles.append(ld[0].copy())
    first = tok_d
    seq_o, seq_d = [], []
    for i in range(64):                          # 64 greedy tokens identical (the north-star bar)
        p = len(prompt) + i
        n_o, lo = om.step(tok_o, p); am, ld = dec.step(tok_d, p)
        if tok_o == tok_d:
            worst = max(worst, rel_err(ld[0], lo))
        tok_o, tok_d = n_o, int(am[0])
        seq_o.append(tok_o); seq_d.append(tok_d)
    assert worst < TOL and seq_o == seq_d
    dec.truncate(len(prompt))
    assert dec.generate(first, len(prompt), 64).tolist() == seq_o        # the captured-graph path
    # the prompt path and a batch of 4 equal the single steps
    dec.reset(1)
    am, lg = dec.prefill(prompt, 0, seq=1)
    assert rel_err(lg, singles[-1]) < TOL and am == int(np.argmax(singles[-1]))
    for b in range(4):
        dec.reset(b)
    for p, t in enumerate(prompt):
        am, lg = dec.step(np.full(4, t), np.full(4, p))
        for b in range(4):
            assert rel_err(lg[b], singles[p]) < TOL
    # and as a window of one sequence, followed by lookup generation over the greedy continuation
    dec.reset(0)
    am, lg = dec.step_window(prompt, 0)
    for r in range(len(prompt)):
        assert rel_err(lg[r], singles[r]) < TOL
    dec.truncate(len(prompt) - 1)
    got, passes = dec.generate_lookup(prompt, 65, 1, 5)
    assert got.tolist() == [first] + seq_o[:64] and passes <= 65
    dec.close()


@pytest.mark.parametrize("qt", [O.Q2_K, O.Q3_K, O.Q4_1, O.Q5_0, O.Q5_1])
def test_decoder_of_each_other_type_against_the_oracle(qt):
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=2, head_dim=64, ffn=512, vocab=300, max_ctx=48, eps=1e-5, rope_theta=1e4)
    spec = synthetic_spec(cfg, qt, seed=30 + qt, std=0.05)
    om = oracle_model(spec, acc64=1)
    dec = cai.Decoder(spec)
    seq = [3, 299, 17, 17, 250, 9, 1, 0, 44, 120]
    rows = []
    for p, t in enumerate(seq):
        n_o, lo = om.step(t, p); am, ld = dec.step(t, p)
        assert rel_err(ld[0], lo) < TOL and int(am[0]) == n_o
        rows.append(lo)
    # the same tokens as one window of five after the first five (the verify pass of speculative decoding)
    dec.truncate(5)
    am, lg = dec.step_window(seq[5:], 5)
    for r in range(5):
        assert rel_err(lg[r], rows[5 + r]) < TOL and int(am[r]) == int(np.argmax(rows[5 + r]))
    dec.close()


def test_q5_k_largest_codes_on_equal_activations_do_not_overflow_the_integer_sums():
    """Every code 31, every scale 63, all activations equal: the integer sum of a 32-block is 32 * 31 * (2^22 - 1), past
    32 bits, which is why the batch-1 kernel combines its three digit sums in float."""
    from helpers.device import dev, rel_err
    cai = dev()
    rows, cols = 64, 2048
    blk = np.full(176, 0xff, np.uint8)
    blk[0:2] = np.array([np.float16(0.01)]).view(np.uint8); blk[2:4] = np.array([np.float16(0.0)]).view(np.uint8)
    raw = np.tile(blk, rows * cols // 256)
    w = cai.QWeight(O.Q5_K, rows, cols, raw)
    for x in (np.ones((1, cols), np.float32), -np.ones((1, cols), np.float32), np.full((1, cols), 3.7e3, np.float32)):
        assert rel_err(w.gemv(x), O.gemv(O.Q5_K, raw, rows, cols, x, None, 0, 1)) < TIGHT
    w.close()


@pytest.mark.parametrize("rows,cols", [(2048, 512), (37888, 3584), (1024, 5120)])
def test_q5_k_fused_feed_forward_front_half(rows, cols):
    """cai_ffn_gateup (RMSNorm -> gate|up -> SwiGLU in one launch) on Q5_K at batch 1, with and without the gain."""
    import ctypes as C
    from helpers.device import dev, rel_err
    cai = dev()
    rng = np.random.default_rng(rows + cols)
    raw = O.quantize(O.Q5_K, (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    w = cai.QWeight(O.Q5_K, rows, cols, raw)
    x = (rng.standard_normal((1, cols)) * 1.7).astype(np.float32)
    gain = (1.0 + 0.2 * rng.standard_normal(cols)).astype(np.float32)
    L = O.lib()
    for g in (gain, None):
        h = x[0].copy()
        if g is not None:
            L.orc_rmsnorm(C.c_void_p(x[0].ctypes.data), C.c_void_p(g.ctypes.data), cols, C.c_float(1e-6), C.c_void_p(h.ctypes.data))
        ug = O.gemv(O.Q5_K, raw, rows, cols, h, None, 0, 1)[0]
        want = np.empty(rows // 2, np.float32)
        L.orc_swiglu(C.c_void_p(ug.ctypes.data), rows // 2, C.c_void_p(want.ctypes.data))
        assert rel_err(w.ffn_gateup(x, g, 1e-6)[0], want) < TIGHT
    w.close()


@pytest.mark.parametrize("rows,cols,T", [(128, 256, 2), (33, 512, 3), (1000, 1024, 8), (3584, 3584, 8), (512, 18944, 4), (5000, 768, 13),
                                         (1000, 1024, 40), (3584, 3584, 77), (512, 18944, 33), (130, 512, 64), (4099, 256, 129), (9000, 2048, 300)])
def test_q5_k_on_the_matrix_cores(rows, cols, T):
    """Q5_K through the small-batch kernel (up to 16 tokens) and the prompt kernel (more): the Q4_K walks with the fifth-bit plane
    merged into the codes, sc * (nibble | bit << 4) exact in f16; == T single-token layers of the oracle, bias included."""
    from helpers.device import dev, rel_err
    cai = dev()
    rng = np.random.default_rng(rows + cols + T)
    raw = O.quantize(O.Q5_K, (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    x = (rng.standard_normal((T, cols)) * rng.uniform(0.01, 30.0, (T, 1))).astype(np.float32)
    x[0, : cols // 2] = 0.0
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(O.Q5_K, rows, cols, raw, bias)
    got = w.gemm(x, matrix_cores=True)
    want = O.gemv(O.Q5_K, raw, rows, cols, x, bias, 0, 1)
    for t in range(T):
        assert rel_err(got[t], want[t], floor=0.02 * cols ** 0.5 * float(np.abs(x[t]).mean())) < TIGHT, t
    w.close()


def test_q5_k_largest_codes_and_scales_on_the_matrix_cores():
    """Every code 31 and every scale 63 (the f16 weight operand at its largest, 1953) on both matrix-core kernels."""
    from helpers.device import dev, rel_err
    cai = dev()
    rows, cols = 96, 1024
    blk = np.full(176, 0xff, np.uint8)
    blk[0:2] = np.array([np.float16(0.01)]).view(np.uint8); blk[2:4] = np.array([np.float16(0.02)]).view(np.uint8)
    raw = np.tile(blk, rows * cols // 256)
    w = cai.QWeight(O.Q5_K, rows, cols, raw)
    rng = np.random.default_rng(3)
    for T in (5, 40):
        x = rng.standard_normal((T, cols)).astype(np.float32)
        assert rel_err(w.gemm(x, matrix_cores=True), O.gemv(O.Q5_K, raw, rows, cols, x, None, 0, 1)) < TIGHT
    w.close()


def test_q5_k_m_like_decoder_long_prompt_and_batched_generation():
    """A 45-token prompt (prompt kernels for Q5_K and Q6_K) == token-at-a-time steps == the oracle; then a batch of 3 sequences
    decodes (small-batch kernels) like the single sequence."""
    from helpers.device import dev, rel_err
    cai = dev()
    cfg = dict(n_layers=2, d_model=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=1024, vocab=600, max_ctx=96, eps=1e-5, rope_theta=1e4)
    spec = q5_k_m_spec(cfg, 31)
    om = oracle_model(spec, acc64=1)
    dec = cai.Decoder(spec, max_batch=3)
    rng = np.random.default_rng(9)
    prompt = [int(t) for t in rng.integers(0, cfg["vocab"], 45)]
    lo = None
    for p, t in enumerate(prompt):
        _, lo = om.step(t, p)
    for b in range(3):
        am, lg = dec.prefill(prompt, 0, seq=b)
        assert rel_err(lg, lo) < TOL and am == int(np.argmax(lo))
    tok = np.full(3, am)
    for i in range(6):
        n_o, lo = om.step(int(tok[0]), len(prompt) + i)
        tok, lg = dec.step(tok, np.full(3, len(prompt) + i))
        for b in range(3):
            assert rel_err(lg[b], lo) < TOL and int(tok[b]) == n_o
    dec.close()
