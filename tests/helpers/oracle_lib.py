"""ctypes binding of the CPU oracle (oracle/liboracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
ORACLE_DIR = os.path.join(ROOT, "oracle")
_LIB = None

F32, F16, Q4_0, Q8_0, Q4_K, Q6_K, I8ROW = 0, 1, 2, 8, 12, 14, 100
Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K = 3, 6, 7, 10, 11, 13   # decoded by the reference too (neural/neuralgguf.pas:1471-1523)
W_EMBED, W_HEAD, W_Q, W_K, W_V, W_O, W_GATEUP, W_DOWN, W_ROUTER = range(9)
V_ATTN_NORM, V_MLP_NORM, V_FINAL_NORM, V_Q_NORM, V_K_NORM = range(5)


class OrcConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d_model", "n_q_heads", "n_kv_heads", "head_dim", "ffn", "vocab", "max_ctx")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float)] + \
               [(n, C.c_int32) for n in ("window", "qk_norm_full", "n_experts", "top_k", "norm_topk", "kv_f16", "acc64", "evict_sinks", "evict_recent")]


def _p(a, t=C.c_void_p):
    return a.ctypes.data_as(t) if a is not None else None


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(so):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "-s"])
        L = C.CDLL(so)
        L.orc_f16_to_f32.restype = C.c_float; L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16; L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_row_bytes.restype = C.c_int64; L.orc_row_bytes.argtypes = [C.c_int, C.c_int64]
        L.orc_dequant.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]
        for n in ("orc_quant_q8_0", "orc_quant_q4_0", "orc_quant_q4_k", "orc_quant_q6_k"):
            getattr(L, n).argtypes = [C.c_void_p, C.c_int64, C.c_void_p]; getattr(L, n).restype = None
        L.orc_quant_int8_row.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]; L.orc_quant_int8_row.restype = None
        L.orc_gguf_deinterleaved_src_row.restype = C.c_int64; L.orc_gguf_deinterleaved_src_row.argtypes = [C.c_int64, C.c_int]
        L.orc_map_target_neuron.restype = C.c_int64; L.orc_map_target_neuron.argtypes = [C.c_int64, C.c_int]
        L.orc_gemv.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        L.orc_rmsnorm.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_void_p]; L.orc_rmsnorm.restype = None
        L.orc_rope_thetas.argtypes = [C.c_float, C.c_int, C.c_void_p]; L.orc_rope_thetas.restype = None
        L.orc_rope_thetas_scaled.argtypes = [C.c_float, C.c_int, C.c_int, C.c_float, C.c_int, C.c_float, C.c_float, C.c_void_p]
        L.orc_model_set_thetas.argtypes = [C.c_void_p, C.c_void_p, C.c_int]; L.orc_model_set_thetas.restype = None
        L.orc_model_set_rope_out_scale.argtypes = [C.c_void_p, C.c_float]; L.orc_model_set_rope_out_scale.restype = None
        L.orc_rope_out_scale.argtypes = [C.c_int, C.c_float]; L.orc_rope_out_scale.restype = C.c_float
        L.orc_rope_interleaved.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]; L.orc_rope_interleaved.restype = None
        L.orc_swiglu.argtypes = [C.c_void_p, C.c_int, C.c_void_p]; L.orc_swiglu.restype = None
        L.orc_softmax.argtypes = [C.c_void_p, C.c_int, C.c_void_p]; L.orc_softmax.restype = None
        L.orc_topk_gate.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]; L.orc_topk_gate.restype = None
        L.orc_argmax.argtypes = [C.c_void_p, C.c_int]
        L.orc_q4k_scale_min.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]; L.orc_q4k_scale_min.restype = None
        L.orc_attn_decode.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p]
        L.orc_attn_decode.restype = None
        L.orc_sample_candidates.restype = C.c_int
        L.orc_sample_candidates.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int, C.c_void_p, C.c_void_p]
        L.orc_attn_decode_evict.restype = None
        L.orc_attn_decode_evict.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p]
        L.orc_max_abs_finite.restype = C.c_float; L.orc_max_abs_finite.argtypes = [C.c_void_p, C.c_int]
        L.orc_kv_quant_row.restype = None; L.orc_kv_quant_row.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        L.orc_attn_decode_i8.restype = None
        L.orc_attn_decode_i8.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p]
        L.orc_model_new.restype = C.c_void_p; L.orc_model_new.argtypes = [C.POINTER(OrcConfig)]
        L.orc_model_free.argtypes = [C.c_void_p]; L.orc_model_free.restype = None
        L.orc_model_set_tensor.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_model_set_vec.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int]
        L.orc_model_reset.argtypes = [C.c_void_p]; L.orc_model_reset.restype = None
        L.orc_model_truncate.argtypes = [C.c_void_p, C.c_int]; L.orc_model_truncate.restype = None
        L.orc_model_len.argtypes = [C.c_void_p]
        L.orc_model_step.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        L.orc_model_hidden.argtypes = [C.c_void_p]; L.orc_model_hidden.restype = C.POINTER(C.c_float)
        L.orc_model_swap_selection.argtypes = [C.c_void_p, C.c_int, C.c_int]; L.orc_model_swap_selection.restype = None
        L.orc_model_router_probs.argtypes = [C.c_void_p, C.c_int]; L.orc_model_router_probs.restype = C.POINTER(C.c_float)
        L.orc_prompt_lookup_draft.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.cpu_avx_dot_f32.restype = C.c_float; L.cpu_avx_dot_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.cpu_avx_dot_int8.restype = C.c_float; L.cpu_avx_dot_int8.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.cpu_linear_f32.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int]; L.cpu_linear_f32.restype = None
        L.cpu_linear_int8.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int]; L.cpu_linear_int8.restype = None
        _LIB = L
    return _LIB


def row_bytes(t, cols):
    return lib().orc_row_bytes(t, cols)


def dequant(t, raw, n):
    raw = np.ascontiguousarray(raw)
    out = np.empty(n, np.float32)
    assert lib().orc_dequant(t, _p(raw), n, _p(out)) == 0
    return out


def quantize(t, x):
    """x: float32 array whose last axis is the contiguous (column) axis -> uint8 bytes, row-major."""
    x = np.ascontiguousarray(x, np.float32)
    n = x.size
    if t == F32:
        return x.view(np.uint8).reshape(-1).copy()
    if t == F16:
        return x.astype(np.float16).view(np.uint8).reshape(-1).copy()
    rb = row_bytes(t, x.shape[-1])
    assert rb > 0
    other = {Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q2_K: "Q2_K", Q3_K: "Q3_K", Q5_K: "Q5_K"}
    if t in other:     # the oracle only decodes these: numpy packers on the test side
        from helpers.quant_other import quantize_other
        out = quantize_other(other[t], x)
        assert out.size == n // x.shape[-1] * rb
        return out
    out = np.empty(n // x.shape[-1] * rb, np.uint8)
    fn = {Q8_0: lib().orc_quant_q8_0, Q4_0: lib().orc_quant_q4_0, Q4_K: lib().orc_quant_q4_k, Q6_K: lib().orc_quant_q6_k}[t]
    fn(_p(x), n, _p(out))
    return out


def quant_int8_rows(x):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    codes = np.empty((rows, cols), np.int8); scales = np.empty(rows, np.float32)
    for r in range(rows):
        lib().orc_quant_int8_row(_p(x[r]), cols, C.c_void_p(codes[r].ctypes.data), C.c_void_p(scales[r:r + 1].ctypes.data))
    return codes, scales


def gemv(t, raw, rows, cols, x, bias=None, act=0, acc64=0, scales=None):
    x = np.ascontiguousarray(x, np.float32).reshape(-1, cols)
    nb = x.shape[0]
    y = np.empty((nb, rows), np.float32)
    raw = np.ascontiguousarray(raw)
    if bias is not None:
        bias = np.ascontiguousarray(bias, np.float32)
    if scales is not None:
        scales = np.ascontiguousarray(scales, np.float32)
    assert lib().orc_gemv(t, _p(raw), _p(scales), rows, cols, _p(x), nb, _p(bias), act, acc64, _p(y)) == 0
    return y


class OracleModel:
    """Builds an orc_model from a dict of arrays; keeps them alive."""

    def __init__(self, cfg: OrcConfig):
        self.cfg = cfg
        self.h = lib().orc_model_new(C.byref(cfg))
        self.keep = []

    def set_tensor(self, layer, slot, t, rows, cols, raw, scales=None, bias=None):
        raw = np.ascontiguousarray(raw)
        scales = None if scales is None else np.ascontiguousarray(scales, np.float32)
        bias = None if bias is None else np.ascontiguousarray(bias, np.float32)
        self.keep += [raw, scales, bias]
        assert lib().orc_model_set_tensor(self.h, layer, slot, t, rows, cols, _p(raw), _p(scales), _p(bias)) == 0

    def set_vec(self, layer, slot, v):
        v = np.ascontiguousarray(v, np.float32)
        self.keep.append(v)
        assert lib().orc_model_set_vec(self.h, layer, slot, _p(v), v.size) == 0

    def set_thetas(self, th):
        th = np.ascontiguousarray(th, np.float32)
        lib().orc_model_set_thetas(self.h, _p(th), th.size)

    def set_rope_out_scale(self, s):
        lib().orc_model_set_rope_out_scale(self.h, s)

    def reset(self):
        lib().orc_model_reset(self.h)

    def truncate(self, n):
        lib().orc_model_truncate(self.h, n)

    def step(self, token, pos, want_logits=True):
        lg = np.empty(self.cfg.vocab, np.float32) if want_logits else None
        r = lib().orc_model_step(self.h, int(token), int(pos), _p(lg))
        assert r >= 0, "oracle step failed"
        return r, lg

    def hidden(self):
        """the input of the vocabulary projection at the last step (a copy)"""
        return np.ctypeslib.as_array(lib().orc_model_hidden(self.h), shape=(self.cfg.d_model,)).copy()

    def swap_selection(self, layer, pos):
        """the step at `pos` takes, in block `layer`, the (k+1)-th most probable expert instead of the k-th (-1: off)"""
        lib().orc_model_swap_selection(self.h, layer, pos)

    def router_probs(self, layer):
        """router soft-max of block `layer` at the last step (a copy)"""
        return np.ctypeslib.as_array(lib().orc_model_router_probs(self.h, layer), shape=(self.cfg.n_experts,)).copy()

    def __del__(self):
        try:
            lib().orc_model_free(self.h)
        except Exception:
            pass


def sample_candidates(logits, m, temperature=1.0, history=None, repetition=1.0, frequency=0.0, presence=0.0):
    """history: iterable of token ids (the context); returns (tokens, probs) of the m most probable, descending."""
    logits = np.ascontiguousarray(logits, np.float32)
    ids, counts = (np.unique(np.asarray(history, np.int32), return_counts=True) if history is not None and len(history) else (np.zeros(0, np.int32), np.zeros(0, np.int64)))
    ids = np.ascontiguousarray(ids, np.int32); counts = np.ascontiguousarray(counts, np.int32)
    tok = np.zeros(m, np.int32); p = np.zeros(m, np.float32)
    k = lib().orc_sample_candidates(_p(logits), logits.size, _p(ids), _p(counts), ids.size, repetition, frequency, presence, temperature, m, _p(tok), _p(p))
    return tok[:k], p[:k]


def prompt_lookup_draft(context, match_len, num_draft):
    context = np.ascontiguousarray(context, np.int32)
    out = np.empty(max(num_draft, 1), np.int32)
    n = lib().orc_prompt_lookup_draft(context.ctypes.data, context.size, match_len, num_draft, out.ctypes.data)
    return out[:n].tolist()
