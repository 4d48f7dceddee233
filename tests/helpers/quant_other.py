"""Test-side packers for the GGUF block types the oracle only decodes (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K).

Round-to-nearest with per-block min/max scales: simpler than ggml's error-minimising search, but a valid encoder of each
format (any bytes are), which is all the parity tests need; the decode side is what the reference defines
(neural/neuralgguf.pas:516-648, 718-944).  numpy only.
"""
import numpy as np


def _h(v):
    """float array -> the nearest halfs as bytes [..., 2] and as float32 values"""
    h = np.asarray(v, np.float32).astype(np.float16)
    return h[..., None].view(np.uint8), h.astype(np.float32)


def _safe_div(a, b):
    return np.divide(a, b, out=np.zeros_like(a), where=b != 0)


def _pack_nibbles(q):      # q [n, 32] in 0..15 -> [n, 16]: element e < 16 low nibble of byte e, else high nibble of byte e - 16
    return (q[:, :16] | (q[:, 16:] << 4)).astype(np.uint8)


def _pack_bits32(bit):     # bit [n, 32] in 0..1 -> little-endian 32-bit plane [n, 4]
    return np.packbits(bit.astype(np.uint8), axis=1, bitorder="little")


def _pack_k_scales(sc, mn):   # [n, 8] 6-bit each -> the 12 packed bytes of Q4_K / Q5_K
    p = np.zeros((sc.shape[0], 12), np.uint8)
    p[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
    p[:, 4:8] = (mn[:, 0:4] & 63) | ((mn[:, 4:8] >> 4) << 6)
    p[:, 8:12] = (sc[:, 4:8] & 15) | ((mn[:, 4:8] & 15) << 4)
    return p


def quantize_other(name, x):
    x = np.ascontiguousarray(x, np.float32)
    if name in ("Q4_1", "Q5_0", "Q5_1"):
        b = x.reshape(-1, 32)
        n = b.shape[0]
        if name == "Q5_0":
            i = np.argmax(np.abs(b), axis=1)
            db, d = _h(b[np.arange(n), i] / -16.0)
            q = np.clip(np.rint(_safe_div(b, d[:, None])) + 16, 0, 31).astype(np.int64)
            return np.concatenate([db, _pack_bits32(q >> 4), _pack_nibbles(q & 15)], 1).reshape(-1)
        levels = 15 if name == "Q4_1" else 31
        lo, hi = b.min(1), b.max(1)
        db, d = _h((hi - lo) / levels)
        mb, m = _h(lo)
        q = np.clip(np.rint(_safe_div(b - m[:, None], d[:, None])), 0, levels).astype(np.int64)
        if name == "Q4_1":
            return np.concatenate([db, mb, _pack_nibbles(q)], 1).reshape(-1)
        return np.concatenate([db, mb, _pack_bits32(q >> 4), _pack_nibbles(q & 15)], 1).reshape(-1)
    b = x.reshape(-1, 256)
    n = b.shape[0]
    if name == "Q5_K":
        s = b.reshape(n, 8, 32)
        lo = np.minimum(s.min(2), 0.0); hi = s.max(2)
        scale = (hi - lo) / 31.0; mins = -lo
        db, d = _h(scale.max(1) / 63.0); mb, dmin = _h(mins.max(1) / 63.0)
        sc = np.clip(np.rint(_safe_div(scale, d[:, None])), 0, 63).astype(np.int64)
        mn = np.clip(np.rint(_safe_div(mins, dmin[:, None])), 0, 63).astype(np.int64)
        dl = (d[:, None] * sc)[:, :, None]; ml = (dmin[:, None] * mn)[:, :, None]
        q = np.clip(np.rint(_safe_div(s + ml, np.broadcast_to(dl, s.shape).copy())), 0, 31).astype(np.int64)   # [n, 8, 32]
        qh = np.zeros((n, 32), np.int64)
        for j in range(8):
            qh |= (q[:, j, :] >> 4) << j
        ql = (q[:, 0::2, :] & 15) | ((q[:, 1::2, :] & 15) << 4)                                            # [n, 4, 32]
        return np.concatenate([db, mb, _pack_k_scales(sc, mn), qh.astype(np.uint8), ql.astype(np.uint8).reshape(n, 128)], 1).reshape(-1)
    s = b.reshape(n, 16, 16)
    if name == "Q2_K":
        lo = np.minimum(s.min(2), 0.0); hi = s.max(2)
        scale = (hi - lo) / 3.0; mins = -lo
        db, d = _h(scale.max(1) / 15.0); mb, dmin = _h(mins.max(1) / 15.0)
        sc = np.clip(np.rint(_safe_div(scale, d[:, None])), 0, 15).astype(np.int64)
        mn = np.clip(np.rint(_safe_div(mins, dmin[:, None])), 0, 15).astype(np.int64)
        dl = (d[:, None] * sc)[:, :, None]; ml = (dmin[:, None] * mn)[:, :, None]
        q = np.clip(np.rint(_safe_div(s + ml, np.broadcast_to(dl, s.shape).copy())), 0, 3).astype(np.int64).reshape(n, 2, 4, 32)
        qs = q[:, :, 0] | (q[:, :, 1] << 2) | (q[:, :, 2] << 4) | (q[:, :, 3] << 6)                          # [n, 2, 32]
        return np.concatenate([(sc | (mn << 4)).astype(np.uint8), qs.astype(np.uint8).reshape(n, 64), db, mb], 1).reshape(-1)
    if name == "Q3_K":
        i = np.argmax(np.abs(s), axis=2)
        scale = np.take_along_axis(s, i[:, :, None], 2)[:, :, 0] / -4.0
        j = np.argmax(np.abs(scale), axis=1)
        db, d = _h(scale[np.arange(n), j] / -32.0)
        sc = np.clip(np.rint(_safe_div(scale, d[:, None])), -32, 31).astype(np.int64)
        dl = (d[:, None] * sc)[:, :, None]
        q = (np.clip(np.rint(_safe_div(s, np.broadcast_to(dl, s.shape).copy())), -4, 3).astype(np.int64) + 4).reshape(n, 256)
        hm = np.zeros((n, 32), np.int64)
        for k in range(8):
            hm |= (q[:, 32 * k:32 * k + 32] >> 2) << k
        q2 = (q & 3).reshape(n, 2, 4, 32)
        qs = q2[:, :, 0] | (q2[:, :, 1] << 2) | (q2[:, :, 2] << 4) | (q2[:, :, 3] << 6)
        u = sc + 32
        sp = np.zeros((n, 12), np.int64)
        sp[:, 0:8] = (u[:, 0:8] & 15) | ((u[:, 8:16] & 15) << 4)
        for k in range(4):
            sp[:, 8 + k] = (u[:, k] >> 4) | ((u[:, k + 4] >> 4) << 2) | ((u[:, k + 8] >> 4) << 4) | ((u[:, k + 12] >> 4) << 6)
        return np.concatenate([hm.astype(np.uint8), qs.astype(np.uint8).reshape(n, 64), sp.astype(np.uint8), db], 1).reshape(-1)
    raise ValueError(name)
