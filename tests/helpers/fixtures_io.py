"""Readers for the data fixtures the tests use (GGUF, safetensors, logits JSON).

Test infrastructure only: plain numpy parsing of the container formats.  The GGUF layout follows
the reference reader (neural/neuralgguf.pas:1072-1220): header, typed metadata, tensor table with
ggml dims (ne[0] = contiguous axis) reversed to row-major, data section aligned to
general.alignment (default 32).
"""
import json
import os
import struct

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "golden")
REF_FIXTURES = os.path.join(GOLDEN, "ref_fixtures")

GGML_BLOCK = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34),
              10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210)}


class GGUFFile:
    def __init__(self, path):
        with open(path, "rb") as f:
            self.buf = f.read()
        b = self.buf
        assert b[:4] == b"GGUF"
        self.version, = struct.unpack_from("<I", b, 4)
        n_tensors, n_kv = struct.unpack_from("<QQ", b, 8)
        self.pos = 24
        self.meta = {}
        for _ in range(n_kv):
            key = self._str()
            vtype, = struct.unpack_from("<I", b, self.pos); self.pos += 4
            self.meta[key] = self._value(vtype)
        self.tensors = {}
        order = []
        for _ in range(n_tensors):
            name = self._str()
            nd, = struct.unpack_from("<I", b, self.pos); self.pos += 4
            ne = struct.unpack_from("<%dQ" % nd, b, self.pos); self.pos += 8 * nd
            ttype, off = struct.unpack_from("<IQ", b, self.pos); self.pos += 12
            self.tensors[name] = {"ne": list(ne), "shape": list(reversed(ne)), "type": ttype, "offset": off}
            order.append(name)
        align = int(self.meta.get("general.alignment", 32))
        self.data_start = (self.pos + align - 1) // align * align

    def _str(self):
        n, = struct.unpack_from("<Q", self.buf, self.pos); self.pos += 8
        s = self.buf[self.pos:self.pos + n].decode("utf-8", "replace"); self.pos += n
        return s

    def _value(self, t):
        b = self.buf
        simple = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
        if t in simple:
            v, = struct.unpack_from(simple[t], b, self.pos); self.pos += struct.calcsize(simple[t])
            return v
        if t == 8:
            return self._str()
        if t == 9:
            et, n = struct.unpack_from("<IQ", b, self.pos); self.pos += 12
            return [self._value(et) for _ in range(n)]
        raise ValueError("gguf value type %d" % t)

    def raw(self, name):
        """(type_id, row-major shape, raw bytes as uint8 array) of a tensor."""
        t = self.tensors[name]
        n = int(np.prod(t["ne"]))
        be, bb = GGML_BLOCK[t["type"]]
        nbytes = n // be * bb
        s = self.data_start + t["offset"]
        return t["type"], t["shape"], np.frombuffer(self.buf, dtype=np.uint8, count=nbytes, offset=s).copy()


def load_safetensors(path):
    """name -> float32 ndarray (F32, F16, BF16 supported)."""
    with open(path, "rb") as f:
        buf = f.read()
    hlen, = struct.unpack_from("<Q", buf, 0)
    header = json.loads(buf[8:8 + hlen])
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        s, e = info["data_offsets"]
        raw = np.frombuffer(buf, dtype=np.uint8, count=e - s, offset=8 + hlen + s)
        dt = info["dtype"]
        if dt == "F32":
            a = raw.view(np.float32).copy()
        elif dt == "F16":
            a = raw.view(np.float16).astype(np.float32)
        elif dt == "BF16":
            a = (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
        else:
            raise ValueError(dt)
        out[name] = a.reshape(info["shape"])
    return out


def load_json(name):
    with open(os.path.join(REF_FIXTURES, name)) as f:
        return json.load(f)


def ref_path(name):
    return os.path.join(REF_FIXTURES, name)
