"""Block-fused GEMV / small-batch kernels against the oracle's dequantize-then-dot definition.

Tolerance: max |y - y_ref| / max |y_ref| <= 1e-3 (north-star bar for fp32 logits); measured values are ~1e-6.
y_ref accumulates in double over the bit-exact dequantized weights.
"""
import numpy as np
import pytest

from helpers import oracle_lib as O

pytestmark = pytest.mark.gpu
TOL = 1e-3
TIGHT = 2e-5


def make(qt, rows, cols, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    return O.quantize(qt, w), rng


@pytest.mark.parametrize("qt", [O.Q4_K, O.Q8_0, O.Q4_0])
@pytest.mark.parametrize("rows,cols", [(2048, 2048), (5632, 2048), (2048, 5632), (3, 256), (1, 9728), (1000, 3584), (64, 18944), (40000, 512),
                                       (1001, 4352), (77, 6144), (3, 5120), (4099, 5120)])   # 17..24 super-blocks: four rows packed per wave
@pytest.mark.parametrize("nb", [1, 4])
def test_gemv_matches_oracle(qt, rows, cols, nb):
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(qt, rows, cols, rows * 7 + cols)
    x = rng.standard_normal((nb, cols)).astype(np.float32)
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(qt, rows, cols, raw, bias)
    got = w.gemv(x)
    want = O.gemv(qt, raw, rows, cols, x, bias, 0, 1)
    assert got.shape == want.shape
    assert rel_err(got, want, floor=0.02 * cols ** 0.5) < TIGHT


@pytest.mark.parametrize("qt,rows,cols", [(O.Q8_0, 576, 576), (O.Q8_0, 192, 576), (O.Q8_0, 576, 1536), (O.Q4_0, 96, 160), (O.Q8_0, 5, 32)])
def test_gemv_non_256_multiple_widths(qt, rows, cols):
    # SmolLM2-135M widths: 576 = 18 blocks of 32 (not a multiple of 256)
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(qt, rows, cols, 5)
    for nb in (1, 2, 3, 5, 8):
        x = rng.standard_normal((nb, cols)).astype(np.float32)
        got = cai.QWeight(qt, rows, cols, raw).gemv(x)
        assert rel_err(got, O.gemv(qt, raw, rows, cols, x, None, 0, 1)) < TIGHT


@pytest.mark.parametrize("nb", [1, 2, 3, 4, 5, 6, 7, 8])
def test_all_batch_widths_q4k(nb):
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(O.Q4_K, 777, 1024, nb)
    x = rng.standard_normal((nb, 1024)).astype(np.float32)
    got = cai.QWeight(O.Q4_K, 777, 1024, raw).gemv(x)
    assert rel_err(got, O.gemv(O.Q4_K, raw, 777, 1024, x, None, 0, 1)) < TIGHT


@pytest.mark.parametrize("act", [0, 1, 2, 3])
def test_fused_bias_and_activation_order(act):
    # y = act(dot + bias): bias before activation (neural.cl:111-146)
    from helpers.device import dev
    cai = dev()
    raw, rng = make(O.Q8_0, 300, 512, 77)
    x = rng.standard_normal((2, 512)).astype(np.float32) * 3
    bias = rng.standard_normal(300).astype(np.float32)
    got = cai.QWeight(O.Q8_0, 300, 512, raw, bias).gemv(x, act)
    want = O.gemv(O.Q8_0, raw, 300, 512, x, bias, act, 1)
    assert np.max(np.abs(got - want)) < 1e-5


@pytest.mark.parametrize("qt", [O.F32, O.F16])
@pytest.mark.parametrize("rows,cols", [(11, 8), (8, 12), (8, 5), (300, 1000)])
def test_float_weight_types_any_width(qt, rows, cols):
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(qt, rows, cols, 3)
    x = rng.standard_normal((3, cols)).astype(np.float32)
    got = cai.QWeight(qt, rows, cols, raw).gemv(x)
    assert rel_err(got, O.gemv(qt, raw, rows, cols, x, None, 0, 1)) < TIGHT


@pytest.mark.parametrize("rows,cols,nb", [(37, 256, 1), (512, 3584, 1), (300, 2048, 3), (9001, 512, 1), (33001, 256, 1), (70, 18944, 1),
                                          (66, 18944, 2), (41, 1024, 8), (18000, 256, 5)])
def test_q6_k_gemv_matches_oracle(rows, cols, nb):
    """Q6_K (the type real Q4_K_M files use for output.weight and part of ffn_down) on the vector kernel: 16 lanes per
    210-byte super-block, unaligned dword requests; 1, 2 and 4 rows per wave, several activation panels, batches."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(O.Q6_K, rows, cols, rows + cols)
    x = rng.standard_normal((nb, cols)).astype(np.float32)
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    got = cai.QWeight(O.Q6_K, rows, cols, raw, bias).gemv(x)
    want = O.gemv(O.Q6_K, raw, rows, cols, x, bias, 0, 1)
    assert rel_err(got, want, floor=0.02 * cols ** 0.5) < TIGHT


def test_q6_k_largest_codes_on_equal_activations_do_not_overflow_the_integer_sums():
    """16 codes of 63 against 16 activations at the top of the 23-bit range: 16 * 63 * (2^22 - 1) exceeds 32 bits, so the
    batch-1 kernel combines its three digit sums in floating point."""
    from helpers.device import dev, rel_err
    cai = dev()
    rows, cols = 6, 512
    blk = np.zeros(210, np.uint8)
    blk[:192] = 0xFF                                   # every code 63
    blk[192:208] = np.array([1, 2, 3, 127, 1, 1, 5, 1, 9, 1, 1, 1, 77, 1, 1, 1], np.int8).view(np.uint8)
    blk[208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    raw = np.tile(blk, rows * cols // 256)
    for x in (np.ones((1, cols), np.float32), -np.ones((1, cols), np.float32), np.full((1, cols), 3.0e4, np.float32)):
        got = cai.QWeight(O.Q6_K, rows, cols, raw).gemv(x)
        want = O.gemv(O.Q6_K, raw, rows, cols, x, None, 0, 1)
        assert rel_err(got, want) < TIGHT


def test_int8_row_path_scale_then_bias():
    # the reference's own fused-quant format: y = scale_a * sum(code*x) + bias_a (neuralvolume.pas:12693-12745)
    from helpers.device import dev, rel_err
    cai = dev()
    rng = np.random.default_rng(9)
    wf = (rng.standard_normal((128, 515)) * 0.05).astype(np.float32)
    codes, scales = O.quant_int8_rows(wf)
    bias = rng.standard_normal(128).astype(np.float32)
    x = rng.standard_normal((2, 515)).astype(np.float32)
    got = cai.QWeight(cai.I8ROW, 128, 515, codes, bias, scales).gemv(x)
    want = O.gemv(O.I8ROW, codes.view(np.uint8), 128, 515, x, bias, 0, 1, scales)
    assert rel_err(got, want) < TIGHT


@pytest.mark.parametrize("rows,cols", [(128, 512), (1000, 3584), (3, 32), (577, 576), (4096, 18944), (37, 2080)])
@pytest.mark.parametrize("nb", [1, 3, 8])
def test_int8_row_widths_of_whole_32_blocks_take_the_vector_kernel(rows, cols, nb):
    """Per-row int8 matrices whose width is a multiple of 32 run the 16-byte-per-lane kernel of the block types (the row scale
    applied to the finished sum, then the bias: neuralvolume.pas:12693-12745); same contract and tolerance as other widths."""
    from helpers.device import dev, rel_err
    cai = dev()
    rng = np.random.default_rng(rows + cols)
    wf = (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)
    codes, scales = O.quant_int8_rows(wf)
    bias = rng.standard_normal(rows).astype(np.float32)
    x = rng.standard_normal((nb, cols)).astype(np.float32)
    got = cai.QWeight(cai.I8ROW, rows, cols, codes, bias, scales).gemv(x)
    want = O.gemv(O.I8ROW, codes.view(np.uint8), rows, cols, x, bias, 0, 1, scales)
    assert rel_err(got, want, floor=0.05 * cols ** 0.5) < TIGHT


def test_linearity_and_zero_input():
    # size-independent properties at a full-size shape (18944 x 3584 Q4_K)
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(O.Q4_K, 18944, 3584, 42)
    w = cai.QWeight(O.Q4_K, 18944, 3584, raw)
    a = rng.standard_normal(3584).astype(np.float32); b = rng.standard_normal(3584).astype(np.float32)
    ya, yb, yab = w.gemv(a)[0], w.gemv(b)[0], w.gemv(a + b)[0]
    assert rel_err(yab, ya + yb) < 1e-5
    assert np.all(w.gemv(np.zeros(3584, np.float32)) == 0)
    # one-hot input reads one dequantized column exactly
    e = np.zeros(3584, np.float32); e[1234] = 1
    col = O.dequant(O.Q4_K, raw, 18944 * 3584).reshape(18944, 3584)[:, 1234]
    assert rel_err(w.gemv(e)[0], col) < 1e-6


def test_lm_head_shape_q8_0():
    # 152064 x 3584 Q8_0 (Qwen2.5-7B head) at batch 1
    from helpers.device import dev, rel_err
    cai = dev()
    rows, cols = 152064, 3584
    rng = np.random.default_rng(1)
    raw = np.empty(rows * O.row_bytes(O.Q8_0, cols), np.uint8)
    step = 19008
    for r0 in range(0, rows, step):
        blk = (rng.standard_normal((step, cols)) * 0.02).astype(np.float32)
        raw[r0 * O.row_bytes(O.Q8_0, cols):(r0 + step) * O.row_bytes(O.Q8_0, cols)] = O.quantize(O.Q8_0, blk)
    x = rng.standard_normal(cols).astype(np.float32)
    got = cai.QWeight(O.Q8_0, rows, cols, raw).gemv(x)
    want = O.gemv(O.Q8_0, raw, rows, cols, x, None, 0, 1)
    assert rel_err(got, want) < TIGHT
    assert int(np.argmax(got)) == int(np.argmax(want))


@pytest.mark.parametrize("rows,cols,T", [(128, 256, 1), (1000, 1024, 5), (300, 3584, 128), (777, 2048, 200), (4608, 3584, 64)])
def test_multi_token_gemm_on_matrix_cores_equals_gemv(rows, cols, T):
    """cai_qgemm (Q4_K: MFMA with exact integer blocks and hi/lo-split activations) == T single-token layers."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(O.Q4_K, rows, cols, T)
    x = (rng.standard_normal((T, cols)) * rng.uniform(0.01, 30.0, (T, 1))).astype(np.float32)   # very different scales per token
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(O.Q4_K, rows, cols, raw, bias)
    got = w.gemm(x)
    want = O.gemv(O.Q4_K, raw, rows, cols, x, bias, 0, 1)
    for t in range(T):
        assert rel_err(got[t], want[t], floor=0.02 * cols ** 0.5 * float(np.abs(x[t]).mean())) < TIGHT, t


@pytest.mark.parametrize("rows,cols,T", [(128, 256, 2), (33, 512, 3), (1000, 1024, 8), (3584, 3584, 8), (512, 18944, 4), (40000, 2048, 16), (5000, 768, 13)])
def test_small_batch_gemm_on_matrix_cores_equals_gemv(rows, cols, T):
    """2..16 tokens: the streaming matrix-core kernel (scales folded exactly into the f16 weight operand, block sums fed as one
    more reduction step, 1/2/4 super-block slices per row tile) == T single-token layers, bias included."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(O.Q4_K, rows, cols, T + 100)
    x = (rng.standard_normal((T, cols)) * rng.uniform(0.01, 30.0, (T, 1))).astype(np.float32)
    x[0, : cols // 2] = 0.0                          # all-zero blocks
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(O.Q4_K, rows, cols, raw, bias)
    got = w.gemm(x)
    want = O.gemv(O.Q4_K, raw, rows, cols, x, bias, 0, 1)
    for t in range(T):
        assert rel_err(got[t], want[t], floor=0.02 * cols ** 0.5 * float(np.abs(x[t]).mean())) < TIGHT, t


def test_multi_token_gemm_other_types_and_tokens_not_multiple_of_eight():
    from helpers.device import dev, rel_err
    cai = dev()
    for qt in (O.Q8_0, O.Q4_0):
        raw, rng = make(qt, 200, 576, 9)
        x = rng.standard_normal((13, 576)).astype(np.float32)
        got = cai.QWeight(qt, 200, 576, raw).gemm(x)
        assert rel_err(got, O.gemv(qt, raw, 200, 576, x, None, 0, 1)) < TIGHT


@pytest.mark.parametrize("qt", [O.Q8_0, O.Q4_0])
@pytest.mark.parametrize("rows,cols,T", [(128, 256, 2), (33, 512, 3), (1000, 1024, 8), (3584, 3584, 8), (512, 18944, 4), (40000, 2048, 16),
                                         (5000, 768, 13), (577, 576, 8), (192, 576, 40), (96, 160, 5), (5, 32, 2), (70, 1536, 7)])
def test_small_batch_gemm_q8_0_q4_0_on_matrix_cores(qt, rows, cols, T):
    """32-weight block types on the matrix cores: signed codes as exact f16 (activations the A operand, 16 weight rows the B
    operand, one MFMA per block, the block scale applied to its result) == T single-token layers, bias included.  Widths that
    are not a multiple of 256 end in a short group of blocks."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(qt, rows, cols, T + 200)
    x = (rng.standard_normal((T, cols)) * rng.uniform(0.01, 30.0, (T, 1))).astype(np.float32)
    x[0, : cols // 2] = 0.0
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(qt, rows, cols, raw, bias)
    got = w.gemm(x, matrix_cores=True)               # small matrices would otherwise stay on the vector-unit kernel
    want = O.gemv(qt, raw, rows, cols, x, bias, 0, 1)
    for t in range(T):
        assert rel_err(got[t], want[t], floor=0.02 * cols ** 0.5 * float(np.abs(x[t]).mean())) < TIGHT, t
    assert rel_err(w.gemm(x), want, floor=0.02 * cols ** 0.5 * float(np.abs(x).mean())) < TIGHT   # the dispatcher's own choice


@pytest.mark.parametrize("rows,cols,T", [(128, 256, 2), (33, 512, 3), (1000, 1024, 8), (3584, 3584, 8), (512, 18944, 4), (20000, 2048, 16), (5000, 768, 13), (70, 1536, 7),
                                         (1000, 1024, 40), (3584, 3584, 77), (512, 18944, 33), (130, 512, 64), (4099, 256, 129)])
def test_small_batch_gemm_q6_k_on_matrix_cores(rows, cols, T):
    """Q6_K on the matrix cores: one 16-deep MFMA per 16-weight scale group (codes q - 32 exact in f16, d * scale applied to
    the result by the lane that owns the weight row), 16-byte requests transposed over the four k lanes
    == T single-token layers, bias included.  More than 16 tokens take the prompt kernel: the scale split into
    16 * (s >> 4) and s & 15, two exact f16 operand slots per weight."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(O.Q6_K, rows, cols, T + 300)
    x = (rng.standard_normal((T, cols)) * rng.uniform(0.01, 30.0, (T, 1))).astype(np.float32)
    x[0, : cols // 2] = 0.0
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(O.Q6_K, rows, cols, raw, bias)
    got = w.gemm(x, matrix_cores=True)
    want = O.gemv(O.Q6_K, raw, rows, cols, x, bias, 0, 1)
    for t in range(T):
        assert rel_err(got[t], want[t], floor=0.02 * cols ** 0.5 * float(np.abs(x[t]).mean())) < TIGHT, t
    assert rel_err(w.gemm(x), want, floor=0.02 * cols ** 0.5 * float(np.abs(x).mean())) < TIGHT   # the dispatcher's own choice


@pytest.mark.parametrize("qt,rows,cols", [(O.Q8_0, 4101, 4096), (O.Q4_0, 8203, 4096), (O.Q4_K, 8203, 4096), (O.Q6_K, 5003, 4096), (O.I8ROW, 4101, 4096), (O.I8ROW, 7001, 2400)])
@pytest.mark.parametrize("nb", [2, 4, 8])
def test_gemv_batch_on_large_matrix_goes_to_matrix_cores(qt, rows, cols, nb):
    """cai_qgemv with a batch on a matrix of 16 MiB or more takes the matrix-core small-batch path; same contract as batch 1."""
    from helpers.device import dev, rel_err
    cai = dev()
    scales = None
    if qt == O.I8ROW:      # the reference's own per-row int8 format (width 2400: a short last block group)
        rng = np.random.default_rng(nb)
        raw, scales = O.quant_int8_rows((rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    else:
        raw, rng = make(qt, rows, cols, nb)
    x = rng.standard_normal((nb, cols)).astype(np.float32)
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(qt, rows, cols, raw, bias, scales)
    got = w.gemv(x)
    want = O.gemv(qt, raw.view(np.uint8) if qt == O.I8ROW else raw, rows, cols, x, bias, 0, 1, scales) if qt == O.I8ROW else O.gemv(qt, raw, rows, cols, x, bias, 0, 1)
    assert rel_err(got, want, floor=0.02 * cols ** 0.5) < TIGHT
    one = w.gemv(x[:1])
    assert rel_err(got[:1], one, floor=0.02 * cols ** 0.5) < TIGHT


@pytest.mark.parametrize("qt", [O.Q8_0, O.Q4_0])
@pytest.mark.parametrize("rows,cols,T", [(200, 576, 17), (577, 576, 40), (192, 576, 255), (1000, 1024, 33), (3584, 3584, 77), (512, 18944, 64), (130, 512, 129),
                                         (4099, 256, 96), (96, 160, 31), (5, 32, 100), (9000, 2048, 300), (64, 2048, 255)])
def test_prompt_gemm_q8_0_q4_0_on_matrix_cores(qt, rows, cols, T):
    """More than 16 tokens of a 32-weight block type go to the prompt kernel (weights as the B operand of 32x32x16 tiles, the
    block scale applied to each block's sums): == T single-token layers of the oracle, bias included; widths that end inside a
    256-column step, row counts that end inside a tile, token counts that end inside a token tile."""
    from helpers.device import dev, rel_err
    cai = dev()
    raw, rng = make(qt, rows, cols, T + 300)
    x = (rng.standard_normal((T, cols)) * rng.uniform(0.01, 30.0, (T, 1))).astype(np.float32)
    x[0, : cols // 2] = 0.0
    bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
    w = cai.QWeight(qt, rows, cols, raw, bias)
    got = w.gemm(x)
    want = O.gemv(qt, raw, rows, cols, x, bias, 0, 1)
    for t in range(T):
        assert rel_err(got[t], want[t], floor=0.02 * cols ** 0.5 * float(np.abs(x[t]).mean())) < TIGHT, t
    w.close()


@pytest.mark.parametrize("qt", [O.Q4_K, O.Q8_0, O.Q4_0, O.Q6_K])
@pytest.mark.parametrize("cols", [3584, 5120])
def test_a_nan_or_inf_activation_reaches_every_output(qt, cols):
    """The integer-dot kernels hold the activation in block-float form (a maximum and integers): a NaN or an infinity in x
    must still poison every output row, as it does in the float dot product of the reference (0 * inf = NaN, x + NaN = NaN),
    and must not leak into rows of a clean batch neighbour."""
    from helpers.device import dev
    cai = dev()
    rows = 300
    raw, rng = make(qt, rows, cols, cols + qt)
    w = cai.QWeight(qt, rows, cols, raw)
    for bad in (np.nan, np.inf, -np.inf):
        for at in (0, 7, cols - 1, cols // 2 + 33):
            x = rng.standard_normal((1, cols)).astype(np.float32)
            x[0, at] = bad
            got = w.gemv(x)
            assert not np.isfinite(got).any(), (bad, at, int(np.isfinite(got).sum()))
    x = rng.standard_normal((3, cols)).astype(np.float32)
    x[1, 100] = np.nan
    got = w.gemv(x)
    assert np.isfinite(got[0]).all() and np.isfinite(got[2]).all() and not np.isfinite(got[1]).any()
    w.close()


@pytest.mark.parametrize("qt,rows,cols", [(O.Q4_K, 8203, 4096), (O.Q8_0, 4101, 4096)])
def test_a_nan_token_poisons_only_its_own_row_on_the_matrix_cores(qt, rows, cols):
    """The same through the matrix-core kernels (a batch of 8 on a matrix of 16 MiB or more, and a 40-token prompt product):
    the poisoned token's outputs are all non-finite, every other token's outputs are finite."""
    from helpers.device import dev
    cai = dev()
    raw, rng = make(qt, rows, cols, 31)
    w = cai.QWeight(qt, rows, cols, raw)
    x = rng.standard_normal((8, cols)).astype(np.float32)
    x[5, 77] = np.nan; x[2, 4000] = np.inf
    got = w.gemv(x)
    for t in range(8):
        assert np.isfinite(got[t]).all() == (t not in (2, 5)), t
        if t in (2, 5):
            assert not np.isfinite(got[t]).any(), t
    x = rng.standard_normal((40, cols)).astype(np.float32)
    x[33, 1] = np.nan
    got = w.gemm(x)
    assert not np.isfinite(got[33]).any()
    assert np.isfinite(np.delete(got, 33, axis=0)).all()
    w.close()


@pytest.mark.parametrize("qt", [O.Q4_K, O.Q4_0, O.Q6_K])
def test_blocks_of_denormal_and_huge_activations(qt):
    """Block-float corner cases of the integer-dot kernels: a 32-block holding only denormals (its scale underflows: the block
    must count as zero, not as NaN), a block of values near 1e30, and a block with one huge and otherwise tiny values (the
    tiny ones round to zero integers, as 2^-23 of the maximum allows).  The kernels sum quant x activation over a 32-block
    BEFORE the block's scale (about 1e-3) multiplies it, so their range ends about four decades below the float maximum:
    activations beyond 1e33 may overflow where a dequantise-first product would not."""
    from helpers.device import dev, rel_err
    cai = dev()
    rows, cols = 200, 3584
    raw, rng = make(qt, rows, cols, 5 + qt)
    w = cai.QWeight(qt, rows, cols, raw)
    x = rng.standard_normal((1, cols)).astype(np.float32)
    x[0, 64:96] = np.float32(1e-40); x[0, 70] = 0.0; x[0, 71] = np.float32(-3e-41)
    x[0, 512:544] *= np.float32(1e30)
    x[0, 1024:1056] = np.float32(1e-12); x[0, 1030] = np.float32(5e6)
    got = w.gemv(x)
    want = O.gemv(qt, raw, rows, cols, x, None, 0, 1)
    assert np.isfinite(got).all()
    assert rel_err(got, want) < TIGHT
    w.close()
