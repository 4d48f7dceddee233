"""Minimal GGUF v3 writer for tests: scalar/string metadata and raw tensors (data section aligned to 32)."""
import struct

import numpy as np


def _s(x):
    x = x.encode() if isinstance(x, str) else x
    return struct.pack("<Q", len(x)) + x


def write_gguf(path, meta, tensors, alignment=32):
    """meta: {key: int | float | str | list of str}; tensors: [(name, row_major_shape, ggml_type, raw_bytes)]."""
    b = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(meta))
    for k, v in meta.items():
        if isinstance(v, str):
            b += _s(k) + struct.pack("<I", 8) + _s(v)
        elif isinstance(v, float):
            b += _s(k) + struct.pack("<If", 6, v)
        elif isinstance(v, (list, tuple)):      # array of strings
            b += _s(k) + struct.pack("<IIQ", 9, 8, len(v)) + b"".join(_s(w) for w in v)
        else:
            b += _s(k) + struct.pack("<II", 4, v)
    off, blobs = 0, []
    for name, shape, ty, raw in tensors:
        raw = bytes(raw)
        b += _s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in reversed(shape)) + struct.pack("<IQ", ty, off)
        pad = -len(raw) % alignment
        blobs.append(raw + b"\0" * pad); off += len(raw) + pad
    b += b"\0" * (-len(b) % alignment)
    with open(path, "wb") as f:
        f.write(b + b"".join(blobs))


def spec_to_gguf(path, spec, arch):
    """Writes a dense llama/qwen2-style decoder spec (tests/helpers/model_build.py layout) as a GGUF file:
    gate|up is split back into ffn_up / ffn_gate; q/k rows are stored as they are (interleaved-rotary order)."""
    from . import oracle_lib as O
    c = spec["cfg"]
    meta = {"general.architecture": arch, arch + ".block_count": c["n_layers"], arch + ".embedding_length": c["d_model"],
            arch + ".feed_forward_length": c["ffn"], arch + ".attention.head_count": c["n_q_heads"],
            arch + ".attention.head_count_kv": c["n_kv_heads"], arch + ".context_length": c["max_ctx"],
            arch + ".attention.layer_norm_rms_epsilon": float(c["eps"]), arch + ".rope.freq_base": float(c["rope_theta"]),
            arch + ".attention.key_length": c["head_dim"]}
    out = []

    def mat(name, t, rows=None, row0=0):
        raw = np.asarray(t["raw"], np.uint8)
        rows = t["rows"] if rows is None else rows
        rb = raw.size // t["rows"]
        out.append((name, [rows, t["cols"]], t["type"], raw[row0 * rb:(row0 + rows) * rb].tobytes()))

    def vec(name, v):
        out.append((name, [len(v)], 0, np.asarray(v, np.float32).tobytes()))

    T, V = spec["tensors"], spec["vecs"]
    mat("token_embd.weight", T[(-1, O.W_EMBED)])
    if (-1, O.W_HEAD) in T:
        mat("output.weight", T[(-1, O.W_HEAD)])
    vec("output_norm.weight", V[(-1, O.V_FINAL_NORM)])
    for l in range(c["n_layers"]):
        p = "blk.%d." % l
        for slot, nm in ((O.W_Q, "attn_q"), (O.W_K, "attn_k"), (O.W_V, "attn_v")):
            mat(p + nm + ".weight", T[(l, slot)])
            if T[(l, slot)].get("bias") is not None:
                vec(p + nm + ".bias", T[(l, slot)]["bias"])
        mat(p + "attn_output.weight", T[(l, O.W_O)])
        gu = T[(l, O.W_GATEUP)]
        mat(p + "ffn_up.weight", gu, rows=c["ffn"], row0=0)
        mat(p + "ffn_gate.weight", gu, rows=c["ffn"], row0=c["ffn"])
        mat(p + "ffn_down.weight", T[(l, O.W_DOWN)])
        vec(p + "attn_norm.weight", V[(l, O.V_ATTN_NORM)])
        vec(p + "ffn_norm.weight", V[(l, O.V_MLP_NORM)])
    write_gguf(path, meta, out)
