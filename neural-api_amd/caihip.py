"""ctypes view of include/caihip.h (tests and bench plumbing; no compute here)."""
import ctypes as C
import os

import numpy as np

from . import lib_path

F32, F16, Q4_0, Q8_0, Q4_K, Q6_K, I8ROW = 0, 1, 2, 8, 12, 14, 100
Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K = 3, 6, 7, 10, 11, 13
ACT_NONE, ACT_RELU, ACT_SIGMOID, ACT_TANH = 0, 1, 2, 3
ROPE_NONE, ROPE_LINEAR, ROPE_LLAMA3, ROPE_NTK, ROPE_YARN = 0, 1, 2, 3, 4
X_DEVICE, Y_DEVICE, MATRIX_CORES = 1, 2, 4
KV_F32, KV_F16, KV_I8 = 0, 1, 2
W_EMBED, W_HEAD, W_Q, W_K, W_V, W_O, W_GATEUP, W_DOWN, W_ROUTER = range(9)
V_ATTN_NORM, V_MLP_NORM, V_FINAL_NORM, V_Q_NORM, V_K_NORM = range(5)

# every symbol include/caihip.h declares
SYMBOLS = """cai_init cai_shutdown cai_last_error cai_device_name cai_sync cai_get_stream cai_timer_start cai_timer_stop
cai_dev_alloc cai_dev_free cai_dev_upload cai_dev_download cai_dev_copy
cai_qw_create cai_qw_create_int8row cai_qw_destroy cai_qw_info cai_qw_dequant_rows cai_qgemv cai_ffn_gateup cai_qgemm
cai_rmsnorm cai_rope cai_swiglu cai_argmax cai_argmax_noalloc cai_router_topk
cai_kv_create cai_kv_destroy cai_kv_reset cai_kv_truncate cai_kv_len cai_kv_snapshot cai_kv_restore cai_kv_snap_destroy cai_kv_export_layer cai_kv_import_layer cai_kv_set_eviction cai_kv_rows cai_attn_decode
cai_decoder_create cai_decoder_destroy cai_decoder_set_weight cai_decoder_set_vector cai_decoder_step cai_decoder_hidden_state cai_decoder_step_window cai_prompt_lookup_draft cai_decoder_generate_lookup cai_decoder_generate cai_decoder_profile cai_decoder_timeline
cai_decoder_prefill cai_decoder_reset cai_decoder_truncate cai_decoder_len cai_decoder_set_eviction cai_decoder_cache_rows cai_decoder_set_kv_dtype cai_decoder_set_rope_scaling cai_decoder_set_rope_freq_factors cai_decoder_set_rope_out_scale cai_sample_candidates cai_decoder_candidates cai_decoder_snapshot cai_decoder_restore cai_decoder_fork
cai_decoder_weight_bytes cai_decoder_get_config cai_decoder_load_gguf
cai_gguf_open cai_gguf_close cai_gguf_info cai_gguf_meta_int cai_gguf_meta_float cai_gguf_meta_str cai_gguf_meta_array_count
cai_gguf_meta_array_str cai_gguf_find_tensor cai_gguf_tensor_info cai_gguf_tensor_data cai_gguf_load_qw""".split()


class DecoderConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d_model", "n_q_heads", "n_kv_heads", "head_dim", "ffn", "vocab", "max_ctx")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float)] + \
               [(n, C.c_int32) for n in ("window", "qk_norm_full", "n_experts", "top_k", "norm_topk", "kv_dtype", "max_batch")]


def prompt_lookup_draft(context, match_len, num_draft):
    """PromptLookupDraft on token ids (host only; the library need not be initialised)"""
    context = np.ascontiguousarray(context, np.int32)
    out = np.empty(max(num_draft, 1), np.int32); n = C.c_int32()
    check(load().cai_prompt_lookup_draft(_ptr(context), context.size, match_len, num_draft, _ptr(out), C.byref(n)))
    return out[:n.value].tolist()


class CaiError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("caihip error %d: %s" % (code, msg))
        self.code = code


_LIB = None


def load():
    """Loads libcaihip.so.  Fails loudly when it is missing: there is no other compute path."""
    global _LIB
    if _LIB is None:
        _LIB = C.CDLL(lib_path())
        for s in SYMBOLS:
            getattr(_LIB, s).restype = C.c_int
        vp, i64, i32, f32 = C.c_void_p, C.c_int64, C.c_int, C.c_float
        L = _LIB
        L.cai_init.argtypes = [i32]
        L.cai_last_error.argtypes = [C.c_char_p, i32]
        L.cai_device_name.argtypes = [C.c_char_p, i32]
        L.cai_get_stream.argtypes = [C.POINTER(vp)]
        L.cai_timer_stop.argtypes = [C.POINTER(f32)]
        L.cai_dev_alloc.argtypes = [i64, C.POINTER(vp)]
        L.cai_dev_free.argtypes = [vp]
        L.cai_dev_upload.argtypes = [vp, vp, i64]
        L.cai_dev_download.argtypes = [vp, vp, i64]
        L.cai_dev_copy.argtypes = [vp, vp, i64]
        L.cai_qw_create.argtypes = [i32, i64, i64, vp, vp, C.POINTER(vp)]
        L.cai_qw_create_int8row.argtypes = [i64, i64, vp, vp, vp, C.POINTER(vp)]
        L.cai_qw_destroy.argtypes = [vp]
        L.cai_qw_info.argtypes = [vp, C.POINTER(i32), C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)]
        L.cai_qw_dequant_rows.argtypes = [vp, i64, i64, vp, i32]
        L.cai_qgemv.argtypes = [vp, vp, i32, vp, i32, i32]
        L.cai_qgemm.argtypes = [vp, vp, i32, vp, i32]
        L.cai_ffn_gateup.argtypes = [vp, vp, vp, f32, i32, vp, i32]
        L.cai_rmsnorm.argtypes = [vp, vp, i32, i32, f32, vp, i32]
        L.cai_rope.argtypes = [vp, i32, i32, i32, f32, i32]
        L.cai_swiglu.argtypes = [vp, i32, i32, vp, i32]
        L.cai_argmax.argtypes = [vp, i32, vp, i32]
        L.cai_argmax_noalloc.argtypes = [vp, i32, vp]
        L.cai_router_topk.argtypes = [vp, i32, i32, i32, vp, vp, i32]
        L.cai_kv_create.argtypes = [i32, i32, i32, i32, i32, C.POINTER(vp)]
        L.cai_kv_destroy.argtypes = [vp]
        L.cai_kv_reset.argtypes = [vp]
        L.cai_kv_truncate.argtypes = [vp, i32]
        L.cai_kv_len.argtypes = [vp, i32, C.POINTER(i32)]
        L.cai_kv_snapshot.argtypes = [vp, C.POINTER(vp)]
        L.cai_kv_restore.argtypes = [vp, vp]
        L.cai_kv_snap_destroy.argtypes = [vp]
        L.cai_kv_set_eviction.argtypes = [vp, C.c_int, C.c_int]
        L.cai_kv_rows.argtypes = [vp, C.c_int, C.POINTER(C.c_int)]
        L.cai_kv_export_layer.argtypes = [vp, C.c_int, vp, vp, vp, vp]
        L.cai_kv_import_layer.argtypes = [vp, C.c_int, C.c_int, vp, vp, vp, vp]
        L.cai_attn_decode.argtypes = [vp, i32, vp, i32, i32, f32, vp, i32]
        L.cai_decoder_create.argtypes = [C.POINTER(DecoderConfig), C.POINTER(vp)]
        L.cai_decoder_destroy.argtypes = [vp]
        L.cai_decoder_set_weight.argtypes = [vp, i32, i32, vp]
        L.cai_decoder_set_vector.argtypes = [vp, i32, i32, vp, i32]
        L.cai_decoder_step.argtypes = [vp, vp, vp, i32, vp, vp]
        L.cai_decoder_generate.argtypes = [vp, i32, i32, i32, vp]
        L.cai_decoder_step_window.argtypes = [vp, i32, vp, i32, i32, vp, vp]
        L.cai_decoder_hidden_state.argtypes = [vp, i32, vp]
        L.cai_prompt_lookup_draft.argtypes = [vp, i32, i32, i32, vp, vp]
        L.cai_decoder_generate_lookup.argtypes = [vp, vp, i32, i32, i32, i32, vp, vp]
        L.cai_decoder_profile.argtypes = [vp, i32, i32, vp, i32]
        L.cai_decoder_timeline.argtypes = [vp, i32, vp, C.c_int64, vp, i32, vp, vp, vp]
        L.cai_decoder_prefill.argtypes = [vp, i32, vp, i32, i32, vp, vp]
        L.cai_decoder_reset.argtypes = [vp, i32]
        L.cai_decoder_truncate.argtypes = [vp, i32, i32]
        L.cai_decoder_len.argtypes = [vp, i32, C.POINTER(i32)]
        L.cai_decoder_set_eviction.argtypes = [vp, i32, i32]
        L.cai_decoder_set_kv_dtype.argtypes = [vp, i32]
        L.cai_decoder_set_rope_scaling.argtypes = [vp, i32, C.c_float, i32, C.c_float, C.c_float]
        L.cai_decoder_set_rope_freq_factors.argtypes = [vp, vp, i32]
        L.cai_decoder_set_rope_out_scale.argtypes = [vp, C.c_float]
        L.cai_sample_candidates.argtypes = [vp, i32, vp, vp, i32, C.c_float, C.c_float, C.c_float, C.c_float, i32, vp, vp, C.POINTER(i32), i32]
        L.cai_decoder_candidates.argtypes = [vp, i32, vp, vp, i32, C.c_float, C.c_float, C.c_float, C.c_float, i32, vp, vp, C.POINTER(i32)]
        L.cai_decoder_cache_rows.argtypes = [vp, i32, i32, C.POINTER(i32)]
        L.cai_decoder_snapshot.argtypes = [vp, i32, C.POINTER(vp)]
        L.cai_decoder_restore.argtypes = [vp, i32, vp]
        L.cai_decoder_fork.argtypes = [vp, i32, i32]
        L.cai_decoder_weight_bytes.argtypes = [vp, C.POINTER(i64)]
        L.cai_decoder_get_config.argtypes = [vp, C.POINTER(DecoderConfig)]
        L.cai_decoder_load_gguf.argtypes = [C.c_char_p, i32, i32, i32, C.POINTER(vp)]
        L.cai_gguf_open.argtypes = [C.c_char_p, C.POINTER(vp)]
        L.cai_gguf_close.argtypes = [vp]
        L.cai_gguf_info.argtypes = [vp, C.POINTER(i32), C.POINTER(i32), C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)]
        L.cai_gguf_meta_int.argtypes = [vp, C.c_char_p, C.POINTER(i64)]
        L.cai_gguf_meta_float.argtypes = [vp, C.c_char_p, C.POINTER(C.c_double)]
        L.cai_gguf_meta_str.argtypes = [vp, C.c_char_p, C.c_char_p, i32]
        L.cai_gguf_meta_array_count.argtypes = [vp, C.c_char_p, C.POINTER(i64)]
        L.cai_gguf_meta_array_str.argtypes = [vp, C.c_char_p, i64, C.c_char_p, i32]
        L.cai_gguf_find_tensor.argtypes = [vp, C.c_char_p, C.POINTER(i64)]
        L.cai_gguf_tensor_info.argtypes = [vp, i64, C.c_char_p, i32, C.POINTER(i32), C.POINTER(i32), C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)]
        L.cai_gguf_tensor_data.argtypes = [vp, i64, C.POINTER(vp)]
        L.cai_gguf_load_qw.argtypes = [vp, C.c_char_p, C.c_char_p, C.POINTER(vp)]
    return _LIB


def last_error():
    buf = C.create_string_buffer(1024)
    load().cai_last_error(buf, 1024)
    return buf.value.decode("utf-8", "replace")


def check(rc):
    if rc != 0:
        raise CaiError(rc, last_error())


def init(device=0):
    check(load().cai_init(device))


def device_name():
    buf = C.create_string_buffer(256)
    check(load().cai_device_name(buf, 256))
    return buf.value.decode()


def _ptr(a):
    if a is None:
        return None
    if isinstance(a, int):
        return C.c_void_p(a)
    return C.c_void_p(a.ctypes.data)


class QWeight:
    """Resident quantized matrix (cai_qw_t)."""

    def __init__(self, qtype, rows, cols, blocks, bias=None, scales=None):
        self.qtype, self.rows, self.cols = qtype, rows, cols
        h = C.c_void_p()
        if bias is not None:
            bias = np.ascontiguousarray(bias, np.float32)
        if qtype == I8ROW:
            if not isinstance(blocks, int):            # (an int is a pointer, host or device: taken as it is)
                blocks = np.ascontiguousarray(blocks).view(np.int8)
            if not isinstance(scales, int):
                scales = np.ascontiguousarray(scales, np.float32)
            check(load().cai_qw_create_int8row(rows, cols, _ptr(blocks), _ptr(scales), _ptr(bias), C.byref(h)))
        else:
            if not isinstance(blocks, int):
                blocks = np.ascontiguousarray(blocks)
            check(load().cai_qw_create(qtype, rows, cols, _ptr(blocks), _ptr(bias), C.byref(h)))
        self.h = h

    def dequant_rows(self, row0=0, n_rows=None):
        n_rows = self.rows - row0 if n_rows is None else n_rows
        out = np.empty((n_rows, self.cols), np.float32)
        check(load().cai_qw_dequant_rows(self.h, row0, n_rows, _ptr(out), 0))
        return out

    def gemv(self, x, act=0):
        x = np.ascontiguousarray(x, np.float32).reshape(-1, self.cols)
        y = np.empty((x.shape[0], self.rows), np.float32)
        check(load().cai_qgemv(self.h, _ptr(x), x.shape[0], _ptr(y), act, 0))
        return y

    def ffn_gateup(self, x, gain=None, eps=1e-6):
        x = np.ascontiguousarray(x, np.float32).reshape(-1, self.cols)
        y = np.empty((x.shape[0], self.rows // 2), np.float32)
        g = None if gain is None else np.ascontiguousarray(gain, np.float32)
        check(load().cai_ffn_gateup(self.h, _ptr(x), _ptr(g), eps, x.shape[0], _ptr(y), 0))
        return y

    def gemm(self, x, matrix_cores=False):
        x = np.ascontiguousarray(x, np.float32).reshape(-1, self.cols)
        y = np.empty((x.shape[0], self.rows), np.float32)
        check(load().cai_qgemm(self.h, _ptr(x), x.shape[0], _ptr(y), MATRIX_CORES if matrix_cores else 0))
        return y

    def device_bytes(self):
        b = C.c_int64()
        check(load().cai_qw_info(self.h, None, None, None, C.byref(b)))
        return b.value

    def close(self):
        if self.h:
            load().cai_qw_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _history(history):
    if history is None or len(history) == 0:
        return np.zeros(0, np.int32), np.zeros(0, np.int32)
    ids, counts = np.unique(np.asarray(history, np.int32), return_counts=True)
    return np.ascontiguousarray(ids, np.int32), np.ascontiguousarray(counts, np.int32)


def sample_candidates(logits, m, temperature=1.0, history=None, repetition=1.0, frequency=0.0, presence=0.0):
    logits = np.ascontiguousarray(logits, np.float32)
    ids, counts = _history(history)
    tok = np.zeros(m, np.int32); p = np.zeros(m, np.float32); k = C.c_int()
    check(load().cai_sample_candidates(_ptr(logits), logits.size, _ptr(ids), _ptr(counts), ids.size, repetition, frequency, presence, temperature, m, _ptr(tok), _ptr(p), C.byref(k), 0))
    return tok[:k.value], p[:k.value]


class KVCache:
    def __init__(self, n_layers, kv_heads, head_dim, max_ctx, dtype=KV_F32):
        self.h = C.c_void_p()
        self.kv_heads, self.head_dim, self.dtype = kv_heads, head_dim, dtype
        check(load().cai_kv_create(n_layers, kv_heads, head_dim, max_ctx, dtype, C.byref(self.h)))

    def attn_decode(self, layer, qkv, q_heads, window=0, softcap=0.0):
        qkv = np.ascontiguousarray(qkv, np.float32)
        out = np.empty(q_heads * self.head_dim, np.float32)
        check(load().cai_attn_decode(self.h, layer, _ptr(qkv), q_heads, window, softcap, _ptr(out), 0))
        return out

    def len(self, layer=0):
        n = C.c_int()
        check(load().cai_kv_len(self.h, layer, C.byref(n)))
        return n.value

    def reset(self):
        check(load().cai_kv_reset(self.h))

    def truncate(self, n):
        check(load().cai_kv_truncate(self.h, n))

    def snapshot(self):
        s = C.c_void_p()
        check(load().cai_kv_snapshot(self.h, C.byref(s)))
        return s

    def restore(self, s):
        check(load().cai_kv_restore(self.h, s))

    def set_eviction(self, sinks, recent):
        check(load().cai_kv_set_eviction(self.h, sinks, recent))

    def rows(self, layer=0):
        n = C.c_int()
        check(load().cai_kv_rows(self.h, layer, C.byref(n)))
        return n.value

    def export_layer(self, layer):
        """(k, v, k_scales, v_scales): the live rows in the cache's element type; scales are None unless int8."""
        n = self.rows(layer)
        et = {KV_F32: np.float32, KV_F16: np.float16, KV_I8: np.int8}[self.dtype]
        k = np.zeros((self.kv_heads, n, self.head_dim), et); v = np.zeros_like(k)
        ks = np.zeros((self.kv_heads, n), np.float32) if self.dtype == KV_I8 else None
        vs = np.zeros_like(ks) if ks is not None else None
        check(load().cai_kv_export_layer(self.h, layer, _ptr(k), _ptr(v), _ptr(ks) if ks is not None else None, _ptr(vs) if vs is not None else None))
        return k, v, ks, vs

    def import_layer(self, layer, k, v, ks=None, vs=None):
        k = np.ascontiguousarray(k); v = np.ascontiguousarray(v)
        if ks is not None:
            ks = np.ascontiguousarray(ks, np.float32); vs = np.ascontiguousarray(vs, np.float32)
        check(load().cai_kv_import_layer(self.h, layer, k.shape[1], _ptr(k), _ptr(v), _ptr(ks) if ks is not None else None, _ptr(vs) if vs is not None else None))

    def close(self):
        if self.h:
            load().cai_kv_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class GGUF:
    """cai_gguf_t: the container reader (no GPU needed)."""

    def __init__(self, path):
        self.h = C.c_void_p()
        check(load().cai_gguf_open(os.fsencode(path), C.byref(self.h)))

    def info(self):
        v, a = C.c_int(), C.c_int(); nt, nm, ds = C.c_int64(), C.c_int64(), C.c_int64()
        check(load().cai_gguf_info(self.h, C.byref(v), C.byref(a), C.byref(nt), C.byref(nm), C.byref(ds)))
        return dict(version=v.value, alignment=a.value, n_tensors=nt.value, n_meta=nm.value, data_start=ds.value)

    def meta_int(self, key, default=None):
        v = C.c_int64()
        rc = load().cai_gguf_meta_int(self.h, key.encode(), C.byref(v))
        if rc != 0 and default is not None:
            return default
        check(rc)
        return v.value

    def meta_float(self, key, default=None):
        v = C.c_double()
        rc = load().cai_gguf_meta_float(self.h, key.encode(), C.byref(v))
        if rc != 0 and default is not None:
            return default
        check(rc)
        return v.value

    def meta_str(self, key, default=None):
        buf = C.create_string_buffer(4096)
        rc = load().cai_gguf_meta_str(self.h, key.encode(), buf, 4096)
        if rc != 0 and default is not None:
            return default
        check(rc)
        return buf.value.decode("utf-8", "replace")

    def meta_array_count(self, key):
        v = C.c_int64()
        check(load().cai_gguf_meta_array_count(self.h, key.encode(), C.byref(v)))
        return v.value

    def meta_array_str(self, key, index):
        buf = C.create_string_buffer(4096)
        check(load().cai_gguf_meta_array_str(self.h, key.encode(), index, buf, 4096))
        return buf.value.decode("utf-8", "replace")

    def has_tensor(self, name):
        i = C.c_int64()
        return load().cai_gguf_find_tensor(self.h, name.encode(), C.byref(i)) == 0

    def tensor(self, name_or_index):
        i = C.c_int64(name_or_index) if isinstance(name_or_index, int) else C.c_int64()
        if not isinstance(name_or_index, int):
            check(load().cai_gguf_find_tensor(self.h, name_or_index.encode(), C.byref(i)))
        nb = C.create_string_buffer(512); t, nd = C.c_int(), C.c_int(); sh = (C.c_int64 * 8)(); off, nbytes = C.c_int64(), C.c_int64()
        check(load().cai_gguf_tensor_info(self.h, i.value, nb, 512, C.byref(t), C.byref(nd), sh, C.byref(off), C.byref(nbytes)))
        return dict(index=i.value, name=nb.value.decode(), type=t.value, shape=list(sh[:nd.value]), offset=off.value, nbytes=nbytes.value)

    def tensor_bytes(self, name):
        t = self.tensor(name)
        p = C.c_void_p()
        check(load().cai_gguf_tensor_data(self.h, t["index"], C.byref(p)))
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(t["nbytes"],)).copy()

    def close(self):
        if self.h:
            load().cai_gguf_close(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Decoder:
    """cai_decoder_t built from a backend-neutral spec: {"cfg", "tensors", "vecs"}."""

    @classmethod
    def from_gguf(cls, path, max_ctx=0, max_batch=1, kv_dtype=KV_F32):
        """llama / qwen2 file loaded by the library itself (cai_decoder_load_gguf)."""
        self = cls.__new__(cls)
        self.h = C.c_void_p(); self.weights = []
        check(load().cai_decoder_load_gguf(os.fsencode(path), max_ctx, max_batch, kv_dtype, C.byref(self.h)))
        self.cfg = DecoderConfig()
        check(load().cai_decoder_get_config(self.h, C.byref(self.cfg)))
        return self

    def __init__(self, spec, max_batch=1, kv_dtype=KV_F32, max_ctx=None):
        c = spec["cfg"]
        self.cfg = DecoderConfig(n_layers=c["n_layers"], d_model=c["d_model"], n_q_heads=c["n_q_heads"], n_kv_heads=c["n_kv_heads"],
                                 head_dim=c["head_dim"], ffn=c["ffn"], vocab=c["vocab"], max_ctx=max_ctx or c["max_ctx"], eps=c["eps"],
                                 rope_theta=c["rope_theta"], window=c.get("window", 0), qk_norm_full=c.get("qk_norm_full", 0),
                                 n_experts=c.get("n_experts", 0), top_k=c.get("top_k", 0), norm_topk=c.get("norm_topk", 0),
                                 kv_dtype=kv_dtype, max_batch=max_batch)
        self.h = C.c_void_p()
        check(load().cai_decoder_create(C.byref(self.cfg), C.byref(self.h)))
        self.weights = []
        for (layer, slot), t in spec["tensors"].items():
            w = t.get("qw") or QWeight(t["type"], t["rows"], t["cols"], t["raw"], t.get("bias"), t.get("scales"))
            self.weights.append(w)
            check(load().cai_decoder_set_weight(self.h, layer, slot, w.h))
        for (layer, slot), v in spec["vecs"].items():
            v = np.ascontiguousarray(v, np.float32)
            check(load().cai_decoder_set_vector(self.h, layer, slot, _ptr(v), v.size))

    def step(self, tokens, pos, want_logits=True):
        tokens = np.ascontiguousarray(np.atleast_1d(tokens), np.int32); pos = np.ascontiguousarray(np.atleast_1d(pos), np.int32)
        nb = tokens.size
        lg = np.empty((nb, self.cfg.vocab), np.float32) if want_logits else None
        am = np.empty(nb, np.int32)
        check(load().cai_decoder_step(self.h, _ptr(tokens), _ptr(pos), nb, _ptr(lg), _ptr(am)))
        return am, lg

    def generate(self, first_token, pos, n):
        out = np.empty(n, np.int32)
        check(load().cai_decoder_generate(self.h, int(first_token), int(pos), n, _ptr(out)))
        return out

    def hidden_state(self, row=0):
        """input of the vocabulary projection for a row of the last step or window (HiddenState of the reference session)"""
        out = np.empty(self.cfg.d_model, np.float32)
        check(load().cai_decoder_hidden_state(self.h, row, _ptr(out)))
        return out

    def step_window(self, tokens, pos0, seq=0, want_logits=True):
        """width-n window of ONE sequence: row r is the output at position pos0 + r (StepForward on a width-K twin)"""
        tokens = np.ascontiguousarray(np.atleast_1d(tokens), np.int32)
        n = tokens.size
        lg = np.empty((n, self.cfg.vocab), np.float32) if want_logits else None
        am = np.empty(n, np.int32)
        check(load().cai_decoder_step_window(self.h, seq, _ptr(tokens), n, int(pos0), _ptr(lg), _ptr(am)))
        return am, lg

    def generate_lookup(self, context, n, match_len=2, num_draft=4):
        """greedy continuation with prompt-lookup drafts; returns (tokens, passes).  context[:-1] must be in the cache"""
        context = np.ascontiguousarray(context, np.int32)
        out = np.empty(n, np.int32); passes = C.c_int32()
        check(load().cai_decoder_generate_lookup(self.h, _ptr(context), context.size, match_len, num_draft, n, _ptr(out), C.byref(passes)))
        return out, passes.value

    def profile(self, token, reps=8):
        """microseconds per step in each of the 8 kernel classes of the batch-1 step (see cai_decoder_profile)"""
        us = np.zeros(8, np.float32)
        check(load().cai_decoder_profile(self.h, int(token), reps, _ptr(us), 8))
        return us

    def timeline(self, token, stamps_cap=1 << 20, launches_cap=4096):
        """device-side stamps of one captured batch-1 step (see cai_decoder_timeline): a list of (class, stamps[work-groups][8]
        in microseconds from the earliest stamp; NaN where a work-group never took the stamp)"""
        st = np.zeros(stamps_cap, np.uint64); la = np.zeros(3 * launches_cap, np.int32)
        n_l = C.c_int32(); n_s = C.c_int64(); tpu = C.c_float()
        check(load().cai_decoder_timeline(self.h, int(token), _ptr(st), stamps_cap, _ptr(la), launches_cap, C.byref(n_l), C.byref(n_s), C.byref(tpu)))
        st = st[:n_s.value]
        t0 = st[st > 0].min() if (st > 0).any() else 0
        us = np.where(st > 0, (st.astype(np.int64) - np.int64(t0)).astype(np.float64) / tpu.value, np.nan)
        out = []
        for i in range(n_l.value):
            cls, wgs, first = (int(v) for v in la[3 * i: 3 * i + 3])
            out.append((cls, us[first: first + 8 * wgs].reshape(wgs, 8)))
        return out

    def prefill(self, tokens, pos0=0, seq=0, want_logits=True):
        tokens = np.ascontiguousarray(tokens, np.int32)
        lg = np.empty(self.cfg.vocab, np.float32) if want_logits else None
        am = C.c_int32()
        check(load().cai_decoder_prefill(self.h, seq, _ptr(tokens), tokens.size, pos0, _ptr(lg), C.byref(am)))
        return am.value, lg

    def reset(self, seq=0):
        check(load().cai_decoder_reset(self.h, seq))

    def truncate(self, n, seq=0):
        check(load().cai_decoder_truncate(self.h, seq, n))

    def len(self, seq=0):
        n = C.c_int()
        check(load().cai_decoder_len(self.h, seq, C.byref(n)))
        return n.value

    def set_eviction(self, sinks, recent):
        check(load().cai_decoder_set_eviction(self.h, sinks, recent))

    def candidates(self, m, row=0, temperature=1.0, history=None, repetition=1.0, frequency=0.0, presence=0.0):
        ids, counts = _history(history)
        tok = np.zeros(m, np.int32); p = np.zeros(m, np.float32); k = C.c_int()
        check(load().cai_decoder_candidates(self.h, row, _ptr(ids), _ptr(counts), ids.size, repetition, frequency, presence, temperature, m, _ptr(tok), _ptr(p), C.byref(k)))
        return tok[:k.value], p[:k.value]

    def set_kv_dtype(self, dtype):
        check(load().cai_decoder_set_kv_dtype(self.h, dtype))

    def set_rope_scaling(self, mode, factor, original_ctx=0, low_freq_factor=1.0, high_freq_factor=4.0):
        """mode: ROPE_NONE / ROPE_LINEAR / ROPE_LLAMA3 (rope_scaling of the importers, neural/neuralpretrained.pas:633-668); empty session only."""
        check(load().cai_decoder_set_rope_scaling(self.h, mode, factor, original_ctx, low_freq_factor, high_freq_factor))

    def set_rope_out_scale(self, scale):
        check(load().cai_decoder_set_rope_out_scale(self.h, scale))

    def set_rope_freq_factors(self, factors):
        f = np.ascontiguousarray(factors, np.float32)
        check(load().cai_decoder_set_rope_freq_factors(self.h, f.ctypes.data, f.size))

    def cache_rows(self, seq=0, layer=0):
        n = C.c_int()
        check(load().cai_decoder_cache_rows(self.h, seq, layer, C.byref(n)))
        return n.value

    def snapshot(self, seq=0):
        s = C.c_void_p()
        check(load().cai_decoder_snapshot(self.h, seq, C.byref(s)))
        return s

    def restore(self, s, seq=0):
        check(load().cai_decoder_restore(self.h, seq, s))

    def fork(self, src, dst):
        check(load().cai_decoder_fork(self.h, src, dst))

    def weight_bytes(self):
        b = C.c_int64()
        check(load().cai_decoder_weight_bytes(self.h, C.byref(b)))
        return b.value

    def close(self):
        if self.h:
            load().cai_decoder_destroy(self.h)
            self.h = None
            for w in self.weights:
                w.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
