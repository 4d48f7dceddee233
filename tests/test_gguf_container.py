"""The library's GGUF container reader against the reference's fixtures and its parse-error rules
(TNNetGGUFReader.ParseFile, neural/neuralgguf.pas:1072-1220; assertions of tests/TestNeuralPretrained.pas:5765-5817).
Runs without a GPU: the container entry points touch no device."""
import struct

import numpy as np
import pytest

from helpers.device import cai
from helpers.fixtures_io import GGUFFile, ref_path


def test_tiny_llama_f32_metadata_and_tensor_table():
    g = cai.GGUF(ref_path("tiny_llama_f32.gguf"))
    info = g.info()
    assert info["version"] == 3 and info["alignment"] == 32 and info["n_tensors"] == 21
    assert g.meta_str("general.architecture") == "llama"
    assert g.meta_int("llama.block_count") == 2
    assert g.meta_int("llama.embedding_length") == 8
    assert g.meta_int("llama.feed_forward_length") == 12
    assert g.meta_int("llama.attention.head_count") == 2
    assert g.meta_int("llama.attention.head_count_kv") == 1
    assert g.meta_int("llama.context_length") == 16
    assert g.meta_int("llama.vocab_size") == 11
    assert abs(g.meta_float("llama.rope.freq_base") - 10000.0) < 1e-3
    assert abs(g.meta_float("llama.attention.layer_norm_rms_epsilon") - 1e-5) < 1e-9
    assert g.meta_int("no.such.key", 77) == 77 and g.meta_str("no.such.key", "dflt") == "dflt"
    assert g.meta_str("tokenizer.ggml.model") == "llama"
    assert g.meta_array_count("tokenizer.ggml.tokens") == 11
    assert g.meta_array_str("tokenizer.ggml.tokens", 3) == "<tok_3>"
    assert g.has_tensor("token_embd.weight") and g.has_tensor("output.weight") and not g.has_tensor("nope")
    t = g.tensor("token_embd.weight")
    assert t["shape"] == [11, 8] and t["type"] == cai.F32          # ggml stores [8, 11]; served row-major
    assert g.tensor("blk.0.attn_k.weight")["shape"] == [4, 8]
    assert g.tensor("output_norm.weight")["shape"] == [8]
    with pytest.raises(cai.CaiError):
        g.tensor("nope")
    with pytest.raises(cai.CaiError):
        g.meta_array_str("tokenizer.ggml.tokens", 11)


@pytest.mark.parametrize("name", ["tiny_llama_f32.gguf", "tiny_llama_f16.gguf", "tiny_llama_q8.gguf", "tiny_kquant.gguf"])
def test_every_tensor_matches_the_python_reader_byte_for_byte(name):
    g = cai.GGUF(ref_path(name)); py = GGUFFile(ref_path(name))
    assert g.info()["n_tensors"] == len(py.tensors) and g.info()["data_start"] == py.data_start
    for i, (tname, t) in enumerate(py.tensors.items()):
        got = g.tensor(i)
        assert got["name"] == tname and got["type"] == t["type"] and got["shape"] == t["shape"] and got["offset"] == t["offset"]
        _, _, raw = py.raw(tname)
        assert np.array_equal(g.tensor_bytes(tname), raw)


def test_kquant_fixture_layout_facts():
    g = cai.GGUF(ref_path("tiny_kquant.gguf"))
    assert g.info()["version"] == 3 and g.info()["n_tensors"] == 5
    want = {"kq.Q4_K.weight": (12, 4096, 576), "kq.Q5_K.weight": (13, 4672, 704), "kq.Q6_K.weight": (14, 5376, 840), "kq.Q2_K.weight": (10, 6240, 336)}
    for n, (ty, off, nb) in want.items():
        t = g.tensor(n)
        assert (t["type"], t["offset"], t["nbytes"], t["shape"]) == (ty, off, nb, [1024])   # offsets are relative to the data section


def _gguf(version=3, meta=(), tensors=(), magic=b"GGUF", pad_to=None, data=b""):
    def s(x):
        return struct.pack("<Q", len(x)) + x
    b = magic + struct.pack("<IQQ", version, len(tensors), len(meta))
    for k, vt, payload in meta:
        b += s(k) + struct.pack("<I", vt) + payload
    for name, dims, ty, off in tensors:
        b += s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ty, off)
    if pad_to:
        b += b"\0" * (-len(b) % pad_to)
    return b + data


CASES = {
    "too small": (b"GGUF\3\0\0\0", "too small"),
    "bad magic": (_gguf(magic=b"GGML"), "bad magic"),
    "version 1": (_gguf(version=1), "unsupported version 1"),
    "implausible counts": (b"GGUF" + struct.pack("<IQQ", 3, 1 << 40, 0), "implausible header counts"),
    "empty key": (_gguf(meta=[(b"", 4, struct.pack("<I", 1))]), "empty metadata key"),
    "duplicate key": (_gguf(meta=[(b"a", 4, struct.pack("<I", 1)), (b"a", 4, struct.pack("<I", 2))]), "duplicate metadata key"),
    "truncated value": (_gguf(meta=[(b"a", 10, b"\1\2")]), "truncated"),
    "unknown value type": (_gguf(meta=[(b"a", 99, b"")]), "bad or truncated value"),
    "zero dims": (_gguf(tensors=[(b"t", [], 0, 0)]), "implausible n_dims 0"),
    "zero dimension": (_gguf(tensors=[(b"t", [0], 0, 0)]), "implausible dimension"),
    "duplicate tensor": (_gguf(tensors=[(b"t", [4], 0, 0), (b"t", [4], 0, 0)], pad_to=32, data=b"\0" * 64), "duplicate tensor name"),
    "q8_0 not block multiple": (_gguf(tensors=[(b"t", [33, 2], 8, 0)], pad_to=32, data=b"\0" * 128), "not a multiple of the block size 32"),
    "q4_k not block multiple": (_gguf(tensors=[(b"t", [128, 2], 12, 0)], pad_to=32, data=b"\0" * 512), "not a multiple of the block size 256"),
    "bad alignment": (_gguf(meta=[(b"general.alignment", 4, struct.pack("<I", 24))]), "not a positive power of two"),
    "byte size wraps": (_gguf(tensors=[(b"t", [0x7fffffff, 0x7fffffff, 2], 0, 0)], pad_to=32, data=b"\0" * 64), "byte size overflows"),
    "tensor outside data": (_gguf(tensors=[(b"t", [64], 0, 0)], pad_to=32, data=b"\0" * 64), "falls outside the data section"),
}


@pytest.mark.parametrize("case", list(CASES))
def test_malformed_files_are_refused_with_the_reference_reason(case, tmp_path):
    blob, needle = CASES[case]
    p = tmp_path / "bad.gguf"
    p.write_bytes(blob)
    with pytest.raises(cai.CaiError) as e:
        cai.GGUF(str(p))
    assert needle in str(e.value)


def test_minimal_valid_file_and_missing_file(tmp_path):
    p = tmp_path / "ok.gguf"
    p.write_bytes(_gguf(meta=[(b"general.alignment", 4, struct.pack("<I", 64)), (b"x.flag", 7, b"\1"), (b"x.neg", 5, struct.pack("<i", -7)),
                              (b"x.arr", 9, struct.pack("<IQ", 5, 3) + struct.pack("<3i", 1, 2, 3))],
                        tensors=[(b"t", [4, 2], 0, 0)], pad_to=64, data=np.arange(8, dtype=np.float32).tobytes()))
    g = cai.GGUF(str(p))
    assert g.info()["alignment"] == 64 and g.info()["data_start"] % 64 == 0
    assert g.meta_int("x.flag") == 1 and g.meta_int("x.neg") == -7 and g.meta_array_count("x.arr") == 3
    assert g.tensor("t")["shape"] == [2, 4]
    assert np.array_equal(g.tensor_bytes("t").view(np.float32), np.arange(8, dtype=np.float32))
    with pytest.raises(cai.CaiError):
        cai.GGUF(str(tmp_path / "absent.gguf"))


def test_string_array_reads_in_any_order_match_the_python_reader(tmp_path):
    """cai_gguf_meta_array_str remembers where the last read ended (a vocabulary walked in order costs one entry per call);
    forward, repeated, backward and scattered reads must all return the entry asked for."""
    words = [("tok%d" % i) * (1 + i % 5) for i in range(300)] + ["", "é✓"]
    payload = struct.pack("<IQ", 8, len(words)) + b"".join(struct.pack("<Q", len(w.encode())) + w.encode() for w in words)
    other = struct.pack("<IQ", 8, 2) + b"".join(struct.pack("<Q", 1) + c for c in (b"a", b"b"))
    p = tmp_path / "v.gguf"
    p.write_bytes(_gguf(meta=[(b"tokenizer.ggml.tokens", 9, payload), (b"other", 9, other)], pad_to=32))
    g = cai.GGUF(str(p))
    n = g.meta_array_count("tokenizer.ggml.tokens")
    assert n == len(words)
    order = list(range(n)) + [5, 5, 4, 301, 0, 150, 151, 149, 300] + list(range(n - 1, -1, -7))
    for i in order:
        assert g.meta_array_str("tokenizer.ggml.tokens", i) == words[i], i
        if i % 50 == 0:      # another array in between must not disturb the remembered position
            assert g.meta_array_str("other", 1) == "b"
    with pytest.raises(cai.CaiError):
        g.meta_array_str("tokenizer.ggml.tokens", n)


def _tiny_decoder_file(path, arch, extra_meta=(), drop=(), extra_tensors=()):
    """A one-block decoder file of zeros with the keys the loader requires (written with the tests' GGUF writer)."""
    from helpers.gguf_write import write_gguf
    meta = {"general.architecture": arch, arch + ".block_count": 1, arch + ".embedding_length": 32, arch + ".feed_forward_length": 64,
            arch + ".attention.head_count": 2, arch + ".context_length": 16}
    meta.update(dict(extra_meta))
    z = lambda r, c: np.zeros((r, c), np.float32).tobytes()
    tens = [("token_embd.weight", [10, 32], 0, z(10, 32)), ("output_norm.weight", [32], 0, z(1, 32))]
    for nm, r, c in [("attn_q", 32, 32), ("attn_k", 32, 32), ("attn_v", 32, 32), ("attn_output", 32, 32), ("ffn_up", 64, 32), ("ffn_gate", 64, 32), ("ffn_down", 32, 64)]:
        tens.append(("blk.0.%s.weight" % nm, [r, c], 0, z(r, c)))
    for nm in ("attn_norm", "ffn_norm"):
        tens.append(("blk.0.%s.weight" % nm, [32], 0, z(1, 32)))
    if arch == "qwen2":
        for nm in ("attn_q", "attn_k", "attn_v"):
            tens.append(("blk.0.%s.bias" % nm, [32], 0, z(1, 32)))
    tens = [t for t in tens if t[0] not in drop] + list(extra_tensors)
    write_gguf(path, meta, tens)


LOADER_REFUSALS = {
    # what the reference's importer refuses (neural/neuralpretrained.pas:17539-17557, 17755-17760) is refused here for the same reason
    "qwen2 sliding window": ("qwen2", {"qwen2.attention.sliding_window": 4096}, (), (), "sliding-window"),
    "qwen2 without a bias": ("qwen2", {}, ("blk.0.attn_k.bias",), (), "blk.0.attn_k.bias"),
    "yarn scaling": ("llama", {"llama.rope.scaling.type": "yarn", "llama.rope.scaling.factor": 4.0}, (), (), "supported: none, linear"),
    "linear factor below one": ("llama", {"llama.rope.scaling.type": "linear", "llama.rope.scaling.factor": 0.5}, (), (), "must be >= 1"),
    "block count beyond the tensor table": ("llama", {"llama.block_count": 100000}, (), (), "but the file lists"),
    "width the embedding does not have": ("llama", {"llama.embedding_length": 64}, (), (), "the metadata promises"),
    "implausible context": ("llama", {"llama.context_length": 1 << 30}, (), (), "implausible dimensions"),
    "heads that do not divide": ("llama", {"llama.attention.head_count_kv": 3}, (), (), "query heads over"),
    "rope_freqs of the wrong length": ("llama", {}, (), (("rope_freqs.weight", [4], 0, np.ones(4, np.float32).tobytes()),), "one per rotary pair"),
    "rope_freqs with linear scaling": ("llama", {"llama.rope.scaling.type": "linear", "llama.rope.scaling.factor": 2.0}, (),
                                       (("rope_freqs.weight", [8], 0, np.ones(8, np.float32).tobytes()),), "together with linear scaling"),
}


@pytest.mark.parametrize("case", list(LOADER_REFUSALS))
def test_decoder_loader_judges_the_metadata_before_it_needs_a_device(case, tmp_path):
    """cai_decoder_load_gguf refuses what it cannot run from the file's metadata alone, with the reason, GPU or not."""
    import ctypes as C
    arch, meta, drop, extra, needle = LOADER_REFUSALS[case]
    p = str(tmp_path / "m.gguf")
    _tiny_decoder_file(p, arch, meta, drop, extra)
    h = C.c_void_p()
    rc = cai.load().cai_decoder_load_gguf(p.encode(), 0, 1, 0, C.byref(h))
    assert rc != 0 and not h.value
    buf = C.create_string_buffer(2048); cai.load().cai_last_error(buf, 2048)
    assert needle in buf.value.decode(), buf.value.decode()


def test_pascal_binding_and_header_constants_agree():
    """CAI_* integer constants of the Pascal unit equal the header's."""
    import os
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    hdr = open(os.path.join(root, "include", "caihip.h")).read()
    pas = open(os.path.join(root, "neural-api_amd", "pascal", "caihip.pas")).read()
    h = {m.group(1): int(m.group(2)) for m in re.finditer(r"#define\s+(CAI_[A-Z0-9_]+)\s+\(?(-?\d+)\)?", hdr)}
    p = {m.group(1): int(m.group(2)) for m in re.finditer(r"\b(CAI_[A-Z0-9_]+)\s*=\s*(-?\d+)\s*;", pas)}
    assert len(p) >= 20
    for k, v in p.items():
        assert h.get(k) == v, (k, v, h.get(k))
    for k in ("CAI_Q5_K", "CAI_Q2_K", "CAI_Q3_K", "CAI_Q4_1", "CAI_Q5_0", "CAI_Q5_1", "CAI_ROPE_LINEAR", "CAI_ROPE_LLAMA3"):
        assert k in p, k


FUZZ_CHILD = r'''
import ctypes as C, importlib, os, sys
sys.path.insert(0, sys.argv[1])
cai = importlib.import_module("neural-api_amd.caihip")
L = cai.load()
d = sys.argv[2]
n_ok = 0
for name in sorted(os.listdir(d)):
    print(name, flush=True)                      # the last name printed names the file that took the process down
    path = os.path.join(d, name).encode()
    g = C.c_void_p()
    if L.cai_gguf_open(path, C.byref(g)) == 0:
        n_ok += 1
        ver, al = C.c_int(), C.c_int(); nt, nm, ds = C.c_int64(), C.c_int64(), C.c_int64()
        L.cai_gguf_info(g, C.byref(ver), C.byref(al), C.byref(nt), C.byref(nm), C.byref(ds))
        buf = C.create_string_buffer(256); ty, nd = C.c_int(), C.c_int(); dims = (C.c_int64 * 8)(); off, nb = C.c_int64(), C.c_int64()
        for i in range(min(nt.value, 64)):
            if L.cai_gguf_tensor_info(g, i, buf, 256, C.byref(ty), C.byref(nd), dims, C.byref(off), C.byref(nb)) == 0:
                p = C.c_void_p()
                if L.cai_gguf_tensor_data(g, i, C.byref(p)) == 0 and nb.value > 0:
                    C.string_at(p.value, 1); C.string_at(p.value + nb.value - 1, 1)      # first and last byte lie inside the mapping
        v = C.c_int64(); f = C.c_double()
        for key in (b"general.architecture", b"llama.block_count", b"llama.context_length", b"tokenizer.ggml.tokens", b"general.alignment"):
            L.cai_gguf_meta_int(g, key, C.byref(v)); L.cai_gguf_meta_float(g, key, C.byref(f)); L.cai_gguf_meta_str(g, key, buf, 256)
            if L.cai_gguf_meta_array_count(g, key, C.byref(v)) == 0:
                for i in (0, v.value - 1, v.value // 2): L.cai_gguf_meta_array_str(g, key, i, buf, 256)
        L.cai_gguf_close(g)
    h = C.c_void_p()
    if L.cai_decoder_load_gguf(path, 0, 1, 0, C.byref(h)) == 0 and h.value: L.cai_decoder_free(h)
print("done", n_ok, flush=True)
'''


def test_mutated_files_never_take_the_process_down(tmp_path):
    """Byte flips, overwritten length fields and truncations of a valid decoder file: every one is either refused or read,
    and every tensor the reader then hands out lies inside the mapping.  Runs in a child process so that a crash is a test
    failure that names the file; the files come from a fixed seed."""
    import os, subprocess, sys
    seed_file = tmp_path / "seed.gguf"
    _tiny_decoder_file(str(seed_file), "llama", {"tokenizer.ggml.tokens": ["a", "bc", "def"] * 5, "llama.rope.freq_base": 10000.0})
    blob = seed_file.read_bytes()
    g = cai.GGUF(str(seed_file)); head = g.info()["data_start"]; del g
    d = tmp_path / "cases"; d.mkdir()
    rng = np.random.default_rng(20240611)
    huge = [0xFFFFFFFFFFFFFFFF, 0xFFFFFFFFFFFFFFF0, 1 << 63, 1 << 40, (1 << 32) - 1, 1 << 31, 0]
    for i in range(360):
        b = bytearray(blob)
        kind = i % 4
        if kind == 0:                                  # a few flipped bytes in the header / metadata / tensor table
            for _ in range(int(rng.integers(1, 9))):
                b[int(rng.integers(0, head))] ^= int(rng.integers(1, 256))
        elif kind == 1:                                # a length, count, type or offset field replaced by an extreme value
            at = int(rng.integers(4, head - 8))
            b[at:at + 8] = struct.pack("<Q", huge[int(rng.integers(0, len(huge)))])
        elif kind == 2:                                # cut short
            b = b[:int(rng.integers(0, len(b)))]
        else:                                          # a run of the table overwritten with noise
            at = int(rng.integers(0, head - 16)); n = int(rng.integers(1, 16))
            b[at:at + n] = rng.integers(0, 256, n, dtype=np.uint8).tobytes()
        (d / ("case_%03d.gguf" % i)).write_bytes(bytes(b))
    (d / "case_seed.gguf").write_bytes(blob)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", FUZZ_CHILD, root, str(d)], capture_output=True, text=True, timeout=600)
    lines = r.stdout.strip().splitlines()
    assert r.returncode == 0, "child ended with %d after %s\n%s" % (r.returncode, lines[-1] if lines else "(nothing)", r.stderr[-2000:])
    assert lines[-1].startswith("done") and int(lines[-1].split()[1]) >= 1      # at least the unmodified file is read
