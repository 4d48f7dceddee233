"""Device dequantization is bit-exact to the oracle / reference golden vectors (block formats are the contract)."""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.fixtures_io import GGUFFile, load_json, ref_path

pytestmark = pytest.mark.gpu


def bits_equal(a, b):
    a = np.ascontiguousarray(a, np.float32).reshape(-1); b = np.ascontiguousarray(b, np.float32).reshape(-1)
    nan = np.isnan(a) | np.isnan(b)
    return np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~nan].view(np.uint32), b[~nan].view(np.uint32))


def test_f16_decode_exhaustive_on_device():
    from helpers.device import dev
    cai = dev()
    bits = np.arange(65536, dtype=np.uint16)
    w = cai.QWeight(cai.F16, 1, 65536, bits.view(np.uint8))
    got = w.dequant_rows()[0]
    want = O.dequant(O.F16, bits.view(np.uint8), 65536)
    assert bits_equal(got, want)


def test_q4k_reference_golden_bit_exact_on_device():
    from helpers.device import dev
    cai = dev()
    g = GGUFFile(ref_path("tiny_kquant.gguf"))
    t, shape, raw = g.raw("kq.Q4_K.weight")
    w = cai.QWeight(cai.Q4_K, 4, 256, raw)
    got = w.dequant_rows().reshape(-1)
    want = np.array(load_json("tiny_kquant_ref.json")["dequant"]["Q4_K"], np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q6k_reference_golden_bit_exact_on_device():
    from helpers.device import dev
    cai = dev()
    g = GGUFFile(ref_path("tiny_kquant.gguf"))
    t, shape, raw = g.raw("kq.Q6_K.weight")
    w = cai.QWeight(cai.Q6_K, 4, 256, raw)
    want = np.array(load_json("tiny_kquant_ref.json")["dequant"]["Q6_K"], np.float32)
    assert np.array_equal(w.dequant_rows().reshape(-1).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("qt", [O.Q8_0, O.Q4_0, O.Q4_K, O.Q6_K])
def test_random_bytes_bit_exact(qt):
    """Arbitrary block bytes (every scale/min/nibble pattern, subnormal and huge half scales)."""
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(100 + qt)
    rows, cols = 37, 1024
    rb = O.row_bytes(qt, cols)
    raw = rng.integers(0, 256, rows * rb, dtype=np.uint8)
    # keep half scales finite so products are comparable bit for bit (Inf*0 = NaN is still checked as NaN)
    w = cai.QWeight(qt, rows, cols, raw)
    got = w.dequant_rows()
    want = O.dequant(qt, raw, rows * cols).reshape(rows, cols)
    assert bits_equal(got, want)
    # row window
    assert bits_equal(w.dequant_rows(5, 3), want[5:8])


@pytest.mark.parametrize("qt", [O.Q8_0, O.Q4_0, O.Q4_K, O.Q6_K, O.F32, O.F16])
def test_quantized_weights_bit_exact(qt):
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((64, 768)) * 0.02).astype(np.float32)
    raw = O.quantize(qt, x)
    w = cai.QWeight(qt, 64, 768, raw)
    assert bits_equal(w.dequant_rows(), O.dequant(qt, raw, x.size))


def test_int8_row_dequant():
    from helpers.device import dev
    cai = dev()
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((16, 100)) * 0.05).astype(np.float32)
    codes, scales = O.quant_int8_rows(x)
    w = cai.QWeight(cai.I8ROW, 16, 100, codes, scales=scales)
    assert np.array_equal(w.dequant_rows(), codes.astype(np.float32) * scales[:, None])


def test_bad_shapes_are_refused():
    from helpers.device import dev
    cai = dev()
    with pytest.raises(cai.CaiError) as e:
        cai.QWeight(cai.Q4_K, 4, 300, np.zeros(4 * 144 * 2, np.uint8))
    assert e.value.code == -1 and "blocks" in str(e.value)
    with pytest.raises(cai.CaiError):
        cai.QWeight(30, 4, 256, np.zeros(4 * 512, np.uint8))  # BF16: the container sizes it, nothing decodes it (nor does the reference)
