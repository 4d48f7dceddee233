"""Synthetic block-quantized weights generated on the GPU (benchmark / full-size test plumbing).

torch is used only to make random bytes quickly: N(0, std) values are drawn on the device and packed into
GGUF blocks by vectorised torch ops; the resulting device pointer is handed to cai_qw_create, which copies.
The packers follow the same definitions as the CPU packers in oracle/oracle.c (Q8_0: reference writer,
neural/neuralgguf.pas:1966-1989; Q4_K: simple affine fit on the layout of neural/neuralgguf.pas:440-514);
they need not be bit-identical to them because parity is always judged on the bytes the device consumed.
"""
import torch

from . import caihip as cai


def _half_bytes(x):
    return x.to(torch.float16).view(torch.uint8)


def pack_q8_0(x):
    """x: [rows, cols] float32 -> uint8 [rows, cols/32, 34]"""
    rows, cols = x.shape
    xb = x.view(rows, cols // 32, 32)
    amax = xb.abs().amax(-1)
    scale = amax / 127.0
    inv = torch.where(scale > 0, 1.0 / scale, torch.zeros_like(scale))
    q = xb * inv[..., None]
    q = torch.where(q >= 0, torch.floor(q + 0.5), torch.ceil(q - 0.5)).clamp_(-127, 127).to(torch.int8)
    out = torch.empty(rows, cols // 32, 34, dtype=torch.uint8, device=x.device)
    out[..., 0:2] = _half_bytes(scale).view(rows, cols // 32, 2)
    out[..., 2:] = q.view(torch.uint8)
    return out


def pack_q4_0(x):
    rows, cols = x.shape
    xb = x.view(rows, cols // 32, 32)
    idx = xb.abs().argmax(-1, keepdim=True)
    mx = xb.gather(-1, idx).squeeze(-1)
    d = mx / -8.0
    inv = torch.where(d != 0, 1.0 / d, torch.zeros_like(d))
    q = (xb * inv[..., None] + 8.5).to(torch.int32).clamp_(0, 15).to(torch.uint8)
    out = torch.empty(rows, cols // 32, 18, dtype=torch.uint8, device=x.device)
    out[..., 0:2] = _half_bytes(d).view(rows, cols // 32, 2)
    out[..., 2:] = q[..., :16] | (q[..., 16:] << 4)
    return out


def pack_q4_k(x):
    """x: [rows, cols] float32 (cols % 256 == 0) -> uint8 [rows, cols/256, 144]"""
    rows, cols = x.shape
    nsb = cols // 256
    xb = x.view(rows, nsb, 8, 32)
    lo = xb.amin(-1).clamp(max=0.0)
    hi = torch.maximum(xb.amax(-1), lo)
    step = (hi - lo) / 15.0
    d16 = (step.amax(-1) / 63.0).to(torch.float16)
    m16 = ((-lo).amax(-1) / 63.0).to(torch.float16)
    d = d16.float()[..., None]; dm = m16.float()[..., None]
    sc = torch.where(d > 0, torch.round(step / d), torch.zeros_like(step)).clamp_(0, 63)
    mn = torch.where(dm > 0, torch.round(-lo / dm), torch.zeros_like(lo)).clamp_(0, 63)
    ds = (d * sc)[..., None]; off = (dm * mn)[..., None]
    q = torch.where(ds > 0, torch.round((xb + off) / ds), torch.zeros_like(xb)).clamp_(0, 15).to(torch.uint8)
    sc = sc.to(torch.uint8); mn = mn.to(torch.uint8)
    out = torch.empty(rows, nsb, 144, dtype=torch.uint8, device=x.device)
    out[..., 0:2] = d16.view(torch.uint8).view(rows, nsb, 2)
    out[..., 2:4] = m16.view(torch.uint8).view(rows, nsb, 2)
    out[..., 4:8] = (sc[..., :4] & 63) | ((sc[..., 4:] >> 4) << 6)
    out[..., 8:12] = (mn[..., :4] & 63) | ((mn[..., 4:] >> 4) << 6)
    out[..., 12:16] = (sc[..., 4:] & 15) | ((mn[..., 4:] & 15) << 4)
    qs = q.view(rows, nsb, 4, 2, 32)
    out[..., 16:] = (qs[..., 0, :] | (qs[..., 1, :] << 4)).reshape(rows, nsb, 128)
    return out


def pack_q5_k(x):
    """x: [rows, cols] float32 (cols % 256 == 0) -> uint8 [rows, cols/256, 176]: the affine fit of pack_q4_k with 32 levels; the
    fifth bit of weight i of sub-block j is bit j of plane byte i (layout of neural/neuralgguf.pas:516-587)"""
    rows, cols = x.shape
    nsb = cols // 256
    xb = x.view(rows, nsb, 8, 32)
    lo = xb.amin(-1).clamp(max=0.0)
    hi = torch.maximum(xb.amax(-1), lo)
    step = (hi - lo) / 31.0
    d16 = (step.amax(-1) / 63.0).to(torch.float16)
    m16 = ((-lo).amax(-1) / 63.0).to(torch.float16)
    d = d16.float()[..., None]; dm = m16.float()[..., None]
    sc = torch.where(d > 0, torch.round(step / d), torch.zeros_like(step)).clamp_(0, 63)
    mn = torch.where(dm > 0, torch.round(-lo / dm), torch.zeros_like(lo)).clamp_(0, 63)
    ds = (d * sc)[..., None]; off = (dm * mn)[..., None]
    q = torch.where(ds > 0, torch.round((xb + off) / ds), torch.zeros_like(xb)).clamp_(0, 31).to(torch.uint8)
    sc = sc.to(torch.uint8); mn = mn.to(torch.uint8)
    out = torch.empty(rows, nsb, 176, dtype=torch.uint8, device=x.device)
    out[..., 0:2] = d16.view(torch.uint8).view(rows, nsb, 2)
    out[..., 2:4] = m16.view(torch.uint8).view(rows, nsb, 2)
    out[..., 4:8] = (sc[..., :4] & 63) | ((sc[..., 4:] >> 4) << 6)
    out[..., 8:12] = (mn[..., :4] & 63) | ((mn[..., 4:] >> 4) << 6)
    out[..., 12:16] = (sc[..., 4:] & 15) | ((mn[..., 4:] & 15) << 4)
    plane = torch.zeros(rows, nsb, 32, dtype=torch.uint8, device=x.device)
    for j in range(8):
        plane |= (q[..., j, :] >> 4) << j
    out[..., 16:48] = plane
    qs = (q & 15).view(rows, nsb, 4, 2, 32)
    out[..., 48:] = (qs[..., 0, :] | (qs[..., 1, :] << 4)).reshape(rows, nsb, 128)
    return out


def pack_q6_k(x):
    """x: [rows, cols] float32 (cols % 256 == 0) -> uint8 [rows, cols/256, 210]: symmetric fit, one signed scale per 16
    weights, codes q in 0..63 standing for q - 32 (layout of neural/neuralgguf.pas:639-717)"""
    rows, cols = x.shape
    nsb = cols // 256
    xg = x.view(rows, nsb, 16, 16)
    step = xg.abs().amax(-1) / 31.0
    d16 = (step.amax(-1) / 127.0).to(torch.float16)
    d = d16.float()[..., None]
    sc = torch.where(d > 0, torch.round(step / d), torch.zeros_like(step)).clamp_(0, 127)
    ds = (d * sc)[..., None]
    q = (torch.where(ds > 0, torch.round(xg / ds), torch.zeros_like(xg)).clamp_(-32, 31) + 32).to(torch.uint8)
    q = q.view(rows, nsb, 2, 4, 32)                       # [half][j][l]: weight 128 half + 32 j + l
    out = torch.empty(rows, nsb, 210, dtype=torch.uint8, device=x.device)
    lo = q & 15; hi = q >> 4
    ql = torch.stack([lo[..., 0, :] | (lo[..., 2, :] << 4), lo[..., 1, :] | (lo[..., 3, :] << 4)], dim=-2)   # [half][2][32]
    out[..., 0:128] = ql.reshape(rows, nsb, 128)
    out[..., 128:192] = (hi[..., 0, :] | (hi[..., 1, :] << 2) | (hi[..., 2, :] << 4) | (hi[..., 3, :] << 6)).reshape(rows, nsb, 64)
    out[..., 192:208] = sc.to(torch.int8).view(torch.uint8)
    out[..., 208:210] = d16.view(torch.uint8).view(rows, nsb, 2)
    return out


PACKERS = {cai.Q8_0: pack_q8_0, cai.Q4_0: pack_q4_0, cai.Q4_K: pack_q4_k, cai.Q5_K: pack_q5_k, cai.Q6_K: pack_q6_k}


def random_qweight(qtype, rows, cols, gen, std=0.02, bias=False, chunk_rows=32768, keep_bytes=False):
    """Resident random matrix of the given block type.  Returns (QWeight, bytes tensor or None)."""
    parts = []
    for r0 in range(0, rows, chunk_rows):
        r = min(chunk_rows, rows - r0)
        x = torch.randn(r, cols, device="cuda", dtype=torch.float32, generator=gen) * std
        parts.append(PACKERS[qtype](x).reshape(-1))
        del x
    raw = parts[0] if len(parts) == 1 else torch.cat(parts)
    b = None
    if bias:
        b = (torch.randn(rows, device="cuda", dtype=torch.float32, generator=gen) * std).cpu().numpy()
    torch.cuda.synchronize()
    w = cai.QWeight(qtype, rows, cols, raw.data_ptr(), b)
    return w, (raw if keep_bytes else None), b


# the block types kept as the stored stream: (elements, bytes, offsets of the f16 fields) per block
RAW_BLOCKS = {cai.Q4_1: (32, 20, (0, 2)), cai.Q5_0: (32, 22, (0,)), cai.Q5_1: (32, 24, (0, 2)),
              cai.Q2_K: (256, 84, (80, 82)), cai.Q3_K: (256, 110, (108,)), cai.Q5_K: (256, 176, (0, 2))}


def random_raw_qweight(qtype, rows, cols, gen):
    """Resident matrix of a stored-stream block type for timing: random code / scale bytes (every pattern is a valid block),
    the f16 fields set to a small positive half so that the values stay finite."""
    be, bb, halfs = RAW_BLOCKS[qtype]
    raw = torch.randint(0, 256, (rows * (cols // be), bb), device="cuda", dtype=torch.uint8, generator=gen)
    for h in halfs:
        raw[:, h] = 0x66; raw[:, h + 1] = 0x10
    torch.cuda.synchronize()
    return cai.QWeight(qtype, rows, cols, raw.data_ptr())


def random_int8_rows(rows, cols, gen, scale=1e-3):
    """Resident random matrix in the reference's per-row int8 format (codes in [-127, 127], one float scale per row)."""
    codes = torch.randint(-127, 128, (rows, cols), device="cuda", dtype=torch.int8, generator=gen)
    scales = torch.full((rows,), scale, device="cuda", dtype=torch.float32)
    torch.cuda.synchronize()
    return cai.QWeight(cai.I8ROW, rows, cols, codes.data_ptr(), None, scales.data_ptr())


def more_bits_layer(i, n):
    """The blocks whose attn_v and ffn_down a Q4_K_M export keeps in Q6_K (the first and last eighth and every third between)."""
    return i < n // 8 or i >= 7 * n // 8 or (i - n // 8) % 3 == 2


def random_decoder_spec(cfg, qtype, head_qtype, seed=424242, qkv_bias=False, std=0.02, keep_bytes=False, embed_qtype=None, q6k_mix=False):
    """Backend-neutral spec whose tensors are already resident (entry "qw"); norm gains are 1.
    q6k_mix: attn_v and ffn_down of the more_bits_layer blocks in Q6_K (the Q4_K_M mix)."""
    import numpy as np
    gen = torch.Generator(device="cuda"); gen.manual_seed(seed)
    d, hq, hkv, hd, I, V, L = cfg["d_model"], cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"], cfg["vocab"], cfg["n_layers"]
    ne = cfg.get("n_experts", 0)
    T, Vv = {}, {}

    def put(key, qt, rows, cols, bias=False):
        w, raw, b = random_qweight(qt, rows, cols, gen, std, bias, keep_bytes=keep_bytes)
        T[key] = dict(qw=w, type=qt, rows=rows, cols=cols, raw_dev=raw, bias=b)

    put((-1, cai.W_EMBED), embed_qtype if embed_qtype is not None else head_qtype, V, d)
    if not cfg.get("tied", False):
        put((-1, cai.W_HEAD), head_qtype, V, d)
    Vv[(-1, cai.V_FINAL_NORM)] = np.ones(d, np.float32)
    for l in range(L):
        put((l, cai.W_Q), qtype, hq * hd, d, qkv_bias)
        put((l, cai.W_K), qtype, hkv * hd, d, qkv_bias)
        hi = q6k_mix and more_bits_layer(l, L)
        put((l, cai.W_V), cai.Q6_K if hi else qtype, hkv * hd, d, qkv_bias)
        put((l, cai.W_O), qtype, d, hq * hd)
        Vv[(l, cai.V_ATTN_NORM)] = np.ones(d, np.float32)
        Vv[(l, cai.V_MLP_NORM)] = np.ones(d, np.float32)
        if cfg.get("qk_norm_full", 0):
            Vv[(l, cai.V_Q_NORM)] = np.ones(hq * hd, np.float32)
            Vv[(l, cai.V_K_NORM)] = np.ones(hkv * hd, np.float32)
        if ne:
            put((l, cai.W_ROUTER), qtype, ne, d)
            put((l, cai.W_GATEUP), qtype, ne * 2 * I, d)
            put((l, cai.W_DOWN), qtype, ne * d, I)
        else:
            put((l, cai.W_GATEUP), qtype, 2 * I, d)
            put((l, cai.W_DOWN), cai.Q6_K if hi else qtype, d, I)
    c = {k: v for k, v in cfg.items() if k != "tied"}
    return dict(cfg=c, tensors=T, vecs=Vv)
