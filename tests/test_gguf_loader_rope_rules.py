"""What cai_decoder_load_gguf does with the rotary-scaling entries of a file, decided from the metadata alone (no device is
asked for before the file is accepted, so these run on a host without a GPU).

The reference's llama import accepts rope.scaling.type none / linear and refuses the rest
(neural/neuralpretrained.pas:17539-17557); its qwen2 import never reads the key and leaves the rotation unscaled
(neural/neuralpretrained.pas:17720): the library follows both.  One deliberate difference: a rope_freqs.weight tensor
(llama.cpp's per-frequency divisors of the Llama-3.1 rule), which the reference never reads, IS read and applied here; a
caller that wants the reference's rotation resets the divisors with cai_decoder_set_rope_freq_factors.  The tests pin these
three behaviours through the messages of files that are refused at a later stage for an unrelated reason (the library has
not been started on a device, or the block tensors are missing)."""
import importlib

import numpy as np
import pytest

from helpers.gguf_write import write_gguf

pkg = importlib.import_module("neural-api_amd")
cai = importlib.import_module("neural-api_amd.caihip")


def meta(arch):
    return {"general.architecture": arch, arch + ".block_count": 1, arch + ".embedding_length": 32, arch + ".feed_forward_length": 64,
            arch + ".attention.head_count": 2, arch + ".context_length": 16}


def tensors():
    z = lambda r, c: np.zeros((r, c), np.float32).tobytes()
    return [("token_embd.weight", [10, 32], 0, z(10, 32)), ("output_norm.weight", [32], 0, z(1, 32))]


def refusal(tmp_path, name, m, t):
    p = str(tmp_path / name)
    write_gguf(p, m, t)
    with pytest.raises(cai.CaiError) as e:
        cai.Decoder.from_gguf(p)
    return str(e.value)


def past_the_rope_stage(msg):
    return "rope" not in msg and ("cai_init has not been called" in msg or "missing tensor" in msg)


def test_llama_files_refuse_unknown_scaling_types_and_factors_below_one(tmp_path):
    m = meta("llama"); m["llama.rope.scaling.type"] = "yarn"; m["llama.rope.scaling.factor"] = 4.0
    msg = refusal(tmp_path, "a.gguf", m, tensors())
    assert "rope.scaling.type" in msg and "yarn" in msg and "supported: none, linear" in msg
    m = meta("llama"); m["llama.rope.scaling.type"] = "linear"; m["llama.rope.scaling.factor"] = 0.5
    assert "must be >= 1" in refusal(tmp_path, "b.gguf", m, tensors())
    # none / linear pass this stage
    for i, (ty, f) in enumerate([("none", 1.0), ("linear", 2.0)]):
        m = meta("llama"); m["llama.rope.scaling.type"] = ty; m["llama.rope.scaling.factor"] = f
        assert past_the_rope_stage(refusal(tmp_path, "c%d.gguf" % i, m, tensors()))


def test_qwen2_files_ignore_the_scaling_keys_as_the_reference_does(tmp_path):
    m = meta("qwen2"); m["qwen2.rope.scaling.type"] = "yarn"; m["qwen2.rope.scaling.factor"] = 4.0
    assert past_the_rope_stage(refusal(tmp_path, "q.gguf", m, tensors()))


def test_rope_freqs_tensor_is_read_not_ignored(tmp_path):
    # head_dim = 32 / 2 heads = 16 -> 8 rotary pairs; a tensor of another length is refused, which shows that it is looked at
    bad = tensors() + [("rope_freqs.weight", [5], 0, np.ones(5, np.float32).tobytes())]
    assert "rope_freqs.weight must be 8 F32 values" in refusal(tmp_path, "r.gguf", meta("llama"), bad)
    good = tensors() + [("rope_freqs.weight", [8], 0, np.ones(8, np.float32).tobytes())]
    assert past_the_rope_stage(refusal(tmp_path, "s.gguf", meta("llama"), good))
    # divisors together with linear scaling: refused rather than guessed at
    m = meta("llama"); m["llama.rope.scaling.type"] = "linear"; m["llama.rope.scaling.factor"] = 2.0
    assert "rope_freqs.weight together with linear scaling" in refusal(tmp_path, "t.gguf", m, good)
