"""Long-context frequency rules on the device decoder (cai_decoder_set_rope_scaling / _set_rope_freq_factors and the GGUF
keys that select them) against the oracle stepping with the same table."""
import ctypes as C

import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.gguf_write import spec_to_gguf, write_gguf
from helpers.model_build import oracle_model, synthetic_spec

pytestmark = pytest.mark.gpu
TOL = 1e-3
CFG = dict(n_layers=2, d_model=256, n_q_heads=4, n_kv_heads=2, head_dim=64, ffn=512, vocab=300, max_ctx=96, eps=1e-5, rope_theta=1e4)


def scaled(base, hd, mode, factor, orig=0, low=1.0, high=4.0):
    th = np.empty(hd // 2, np.float32)
    assert O.lib().orc_rope_thetas_scaled(C.c_float(base), hd, mode, C.c_float(factor), orig, C.c_float(low), C.c_float(high), th.ctypes.data) == 0
    return th


def run_both(om, dec, seq, pos0=0):
    from helpers.device import rel_err
    worst = 0.0
    for i, t in enumerate(seq):
        n_o, lo = om.step(t, pos0 + i); am, ld = dec.step(t, pos0 + i)
        worst = max(worst, rel_err(ld[0], lo))
        assert int(am[0]) == n_o
    return worst


@pytest.mark.parametrize("mode,args", [("linear", (1, 4.0, 0, 1.0, 4.0)), ("llama3", (2, 8.0, 16, 1.0, 4.0)), ("ntk", (3, 4.0, 0, 1.0, 4.0)), ("yarn", (4, 4.0, 24, 1.0, 32.0))])
def test_scaled_decoder_matches_the_oracle_and_differs_from_the_unscaled_one(mode, args):
    from helpers.device import dev, rel_err
    cai = dev()
    spec = synthetic_spec(CFG, O.Q8_0, seed=77, std=0.08)
    th = scaled(CFG["rope_theta"], CFG["head_dim"], *args)
    om = oracle_model(spec, acc64=1); om.set_thetas(th)
    out_scale = O.lib().orc_rope_out_scale(args[0], C.c_float(args[1]))
    om.set_rope_out_scale(out_scale)          # the oracle scales the rotated q and k, the device the scores by its square
    dec = cai.Decoder(spec)
    seq = [int(t) for t in np.random.default_rng(5).integers(0, 300, 40)]
    plain = [dec.step(t, p)[1][0].copy() for p, t in enumerate(seq)]
    # a rule cannot change under cached keys
    with pytest.raises(cai.CaiError) as e:
        dec.set_rope_scaling(*args)
    assert e.value.code == -5
    dec.reset(0)
    dec.set_rope_scaling(*args)
    assert run_both(om, dec, seq) < TOL
    dec.reset(0)
    last = [dec.step(t, p)[1][0].copy() for p, t in enumerate(seq)][-1]
    assert rel_err(last, plain[-1]) > 1e-2          # the rule does something at these positions
    dec.reset(0)
    am, lg = dec.prefill(seq, 0)                     # the prompt kernels rotate and scale by the same rule
    assert rel_err(lg, last) < TOL
    # the same table as per-frequency divisors
    base = scaled(CFG["rope_theta"], CFG["head_dim"], 0, 1.0)
    dec.reset(0)
    dec.set_rope_freq_factors(base.astype(np.float64) / th.astype(np.float64))
    dec.set_rope_out_scale(out_scale)
    again = [dec.step(t, p)[1][0].copy() for p, t in enumerate(seq)][-1]
    assert rel_err(again, last) < 1e-4
    # back to none restores the unscaled logits bit for bit; the captured-graph path follows the table too
    dec.reset(0)
    dec.set_rope_scaling(cai.ROPE_NONE, 1.0)
    # (none also puts the output scale back to 1)
    back = [dec.step(t, p)[1][0].copy() for p, t in enumerate(seq)][-1]
    assert np.array_equal(back, plain[-1])
    dec.close()


def test_bad_rules_are_refused():
    from helpers.device import dev
    cai = dev()
    dec = cai.Decoder(synthetic_spec(CFG, O.Q8_0, seed=1))
    for args in [(1, 0.5, 0, 1.0, 4.0), (2, 8.0, 0, 1.0, 4.0), (2, 8.0, 512, 4.0, 4.0), (4, 2.0, 0, 1.0, 32.0), (7, 2.0, 0, 1.0, 4.0)]:
        with pytest.raises(cai.CaiError):
            dec.set_rope_scaling(*args)
    with pytest.raises(cai.CaiError):
        dec.set_rope_freq_factors(np.ones(5, np.float32))
    with pytest.raises(cai.CaiError):
        dec.set_rope_freq_factors(np.zeros(32, np.float32))
    dec.close()


def gguf_with(tmp_path, spec, arch, extra_meta=None, extra_tensors=()):
    """spec_to_gguf, then the same file again with extra metadata / tensors appended through the tests' writer."""
    import struct
    from helpers.fixtures_io import GGUFFile
    p0 = str(tmp_path / "base.gguf")
    spec_to_gguf(p0, spec, arch)
    g = GGUFFile(p0)
    meta = dict(g.meta)
    meta.update(extra_meta or {})
    tens = []
    for name in list(g.tensors):
        t, shape, raw = g.raw(name)
        tens.append((name, shape, t, raw.tobytes()))
    p1 = str(tmp_path / "scaled.gguf")
    write_gguf(p1, meta, tens + list(extra_tensors))
    return p1


def test_gguf_linear_scaling_and_rope_freqs_tensor(tmp_path):
    from helpers.device import dev
    cai = dev()
    spec = synthetic_spec(CFG, O.Q8_0, seed=78, std=0.08)
    seq = [int(t) for t in np.random.default_rng(6).integers(0, 300, 24)]
    # llama.rope.scaling.type = linear, factor 4 (neural/neuralpretrained.pas:17539-17557)
    p = gguf_with(tmp_path, spec, "llama", {"llama.rope.scaling.type": "linear", "llama.rope.scaling.factor": 4.0})
    dec = cai.Decoder.from_gguf(p)
    om = oracle_model(spec, acc64=1); om.set_thetas(scaled(1e4, 64, 1, 4.0))
    assert run_both(om, dec, seq) < TOL
    dec.close()
    # rope_freqs.weight: per-pair divisors (the llama3 table over the unscaled one)
    th = scaled(1e4, 64, 2, 8.0, 16, 1.0, 4.0)
    f = (scaled(1e4, 64, 0, 1.0).astype(np.float64) / th.astype(np.float64)).astype(np.float32)
    p = gguf_with(tmp_path, spec, "llama", None, [("rope_freqs.weight", [32], 0, f.tobytes())])
    dec = cai.Decoder.from_gguf(p)
    want = (scaled(1e4, 64, 0, 1.0).astype(np.float64) / f.astype(np.float64)).astype(np.float32)
    om = oracle_model(spec, acc64=1); om.set_thetas(want)
    assert run_both(om, dec, seq) < TOL
    dec.close()


def test_qwen2_file_without_an_epsilon_key_runs_with_1e_6(tmp_path):
    """The qwen2 branch of the reference's importer defaults the RMSNorm epsilon to 1e-6, the llama branch to 1e-5
    (neural/neuralpretrained.pas:17715, 17533); small activations make the difference visible."""
    from helpers.device import dev, rel_err
    from helpers.fixtures_io import GGUFFile
    cai = dev()
    spec = synthetic_spec(CFG, O.Q8_0, seed=79, std=0.004, qkv_bias=True)
    p0 = str(tmp_path / "q.gguf")
    spec_to_gguf(p0, spec, "qwen2")
    g = GGUFFile(p0)
    meta = {k: v for k, v in g.meta.items() if not k.endswith("layer_norm_rms_epsilon")}
    tens = [(n,) + (lambda r: (r[1], r[0], r[2].tobytes()))(g.raw(n)) for n in list(g.tensors)]
    p1 = str(tmp_path / "q_noeps.gguf")
    write_gguf(p1, meta, tens)
    dec = cai.Decoder.from_gguf(p1)
    assert abs(dec.cfg.eps - 1e-6) < 1e-12
    seq = [3, 299, 17, 17, 250, 9]
    om6 = oracle_model(spec, acc64=1, eps=1e-6)
    assert run_both(om6, dec, seq) < TOL
    dec.close()
