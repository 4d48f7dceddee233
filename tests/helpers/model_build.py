"""Builds decoder model specs (config + per-slot tensors) for the oracle and the device decoder.

A spec is backend-neutral: {"cfg": dict, "tensors": {(layer, slot): dict(type, rows, cols, raw, scales, bias)},
"vecs": {(layer, slot): float32 array}}.  Row placement follows the reference importer
(neural/neuralpretrained.pas:14770-14989): neuron j <- HF row j, except q/k rows which are permuted per
head so that interleaved-pair RoPE equals HF rotate_half (MapTargetNeuron 14792-14812); up -> rows
0..I-1 and gate -> rows I..2I-1 of the fused gate|up layer (240-243, 17412-17421); MoE banks hold
expert e's up rows at e*2I, gate rows at e*2I+I, down rows at e*H (15372-15374).
"""
import json

import numpy as np

from . import oracle_lib as O
from .fixtures_io import GGUFFile, load_safetensors, ref_path


def _perm_rows_interleave(w, head_dim):
    """HF (rotate_half) row order -> interleaved order: target[map(r)] = w[r]."""
    rows = w.shape[0]
    out = np.empty_like(w)
    for r in range(rows):
        out[O.lib().orc_map_target_neuron(r, head_dim)] = w[r]
    return out


def _t(arr, qtype, bias=None):
    arr = np.ascontiguousarray(arr, np.float32)
    rows, cols = arr.shape
    if qtype == O.I8ROW:
        codes, scales = O.quant_int8_rows(arr)
        return dict(type=qtype, rows=rows, cols=cols, raw=codes.view(np.uint8).reshape(-1), scales=scales, bias=bias)
    return dict(type=qtype, rows=rows, cols=cols, raw=O.quantize(qtype, arr), scales=None, bias=bias)


def spec_from_hf(st, cfg_json, qtype=O.F32, max_ctx=None, head_qtype=None, embed_qtype=None):
    """st: name->float32 arrays in HF naming; cfg_json: HF config dict."""
    c = cfg_json
    d = c["hidden_size"]; hq = c["num_attention_heads"]; hkv = c.get("num_key_value_heads", hq)
    hd = c.get("head_dim") or d // hq
    L = c["num_hidden_layers"]; I = c["intermediate_size"]; V = c["vocab_size"]
    ne = c.get("num_experts", 0) or 0
    cfg = dict(n_layers=L, d_model=d, n_q_heads=hq, n_kv_heads=hkv, head_dim=hd, ffn=I, vocab=V,
               max_ctx=max_ctx or c.get("max_position_embeddings", 64), eps=float(c.get("rms_norm_eps", 1e-5)),
               rope_theta=float(c.get("rope_theta", 10000.0)), window=int(c.get("sliding_window") or 0) if c.get("model_type") == "mistral" else 0,
               qk_norm_full=1 if c.get("model_type") == "olmoe" else 0, n_experts=ne, top_k=c.get("num_experts_per_tok", 0) or 0,
               norm_topk=1 if c.get("norm_topk_prob", False) else 0, kv_f16=0, acc64=0)
    T, Vv = {}, {}
    emb = st["model.embed_tokens.weight"]
    T[(-1, O.W_EMBED)] = _t(emb, embed_qtype if embed_qtype is not None else qtype)
    if not c.get("tie_word_embeddings", False) and "lm_head.weight" in st:
        T[(-1, O.W_HEAD)] = _t(st["lm_head.weight"], head_qtype if head_qtype is not None else qtype)
    Vv[(-1, O.V_FINAL_NORM)] = st["model.norm.weight"]
    for l in range(L):
        p = "model.layers.%d." % l
        def bias(n):
            return st.get(p + "self_attn.%s_proj.bias" % n)
        qb, kb, vb = bias("q"), bias("k"), bias("v")
        T[(l, O.W_Q)] = _t(_perm_rows_interleave(st[p + "self_attn.q_proj.weight"], hd), qtype,
                           None if qb is None else _perm_rows_interleave(qb, hd))
        T[(l, O.W_K)] = _t(_perm_rows_interleave(st[p + "self_attn.k_proj.weight"], hd), qtype,
                           None if kb is None else _perm_rows_interleave(kb, hd))
        T[(l, O.W_V)] = _t(st[p + "self_attn.v_proj.weight"], qtype, vb)
        T[(l, O.W_O)] = _t(st[p + "self_attn.o_proj.weight"], qtype)
        Vv[(l, O.V_ATTN_NORM)] = st[p + "input_layernorm.weight"]
        Vv[(l, O.V_MLP_NORM)] = st[p + "post_attention_layernorm.weight"]
        if cfg["qk_norm_full"]:
            Vv[(l, O.V_Q_NORM)] = _perm_rows_interleave(st[p + "self_attn.q_norm.weight"], hd)
            Vv[(l, O.V_K_NORM)] = _perm_rows_interleave(st[p + "self_attn.k_norm.weight"], hd)
        if ne:
            T[(l, O.W_ROUTER)] = _t(st[p + "mlp.gate.weight"], qtype)
            gu = np.concatenate([np.concatenate([st[p + "mlp.experts.%d.up_proj.weight" % e],
                                                 st[p + "mlp.experts.%d.gate_proj.weight" % e]], 0) for e in range(ne)], 0)
            dn = np.concatenate([st[p + "mlp.experts.%d.down_proj.weight" % e] for e in range(ne)], 0)
            T[(l, O.W_GATEUP)] = _t(gu, qtype)
            T[(l, O.W_DOWN)] = _t(dn, qtype)
        else:
            T[(l, O.W_GATEUP)] = _t(np.concatenate([st[p + "mlp.up_proj.weight"], st[p + "mlp.gate_proj.weight"]], 0), qtype)
            T[(l, O.W_DOWN)] = _t(st[p + "mlp.down_proj.weight"], qtype)
    return dict(cfg=cfg, tensors=T, vecs={k: np.ascontiguousarray(v, np.float32) for k, v in Vv.items()})


def spec_from_ref_fixture(name, qtype=O.F32, **kw):
    st = load_safetensors(ref_path(name + ".safetensors"))
    with open(ref_path(name + "_config.json")) as f:
        cfg = json.load(f)
    return spec_from_hf(st, cfg, qtype, **kw)


def spec_from_gguf_llama(path, max_ctx=None):
    """llama/qwen2 GGUF: tensors are uploaded in STORED order and stored type.  llama.cpp's q/k row order
    is already the interleaved order (composition of GGUFDeinterleavedSrcRow, neuralgguf.pas:428-438, with
    MapTargetNeuron, neuralpretrained.pas:14792-14812, is the identity)."""
    g = GGUFFile(path)
    a = g.meta["general.architecture"]
    m = lambda k, dflt=None: g.meta.get("%s.%s" % (a, k), dflt)
    d = m("embedding_length"); hq = m("attention.head_count"); hkv = m("attention.head_count_kv", hq)
    L = m("block_count"); I = m("feed_forward_length"); hd = d // hq
    V = m("vocab_size") or g.tensors["token_embd.weight"]["shape"][0]
    cfg = dict(n_layers=L, d_model=d, n_q_heads=hq, n_kv_heads=hkv, head_dim=hd, ffn=I, vocab=V,
               max_ctx=max_ctx or m("context_length", 64), eps=float(m("attention.layer_norm_rms_epsilon", 1e-5)),
               rope_theta=float(m("rope.freq_base", 10000.0)), window=0, qk_norm_full=0, n_experts=0, top_k=0, norm_topk=0,
               kv_f16=0, acc64=0)

    def raw(name, bias_name=None):
        t, shape, b = g.raw(name)
        bias = None
        if bias_name and bias_name in g.tensors:
            bt, _, bb = g.raw(bias_name)
            bias = O.dequant(bt, bb, shape[0])
        return dict(type=t, rows=shape[0], cols=shape[1], raw=b, scales=None, bias=bias)

    def vec(name):
        t, shape, b = g.raw(name)
        return O.dequant(t, b, shape[0])

    T, Vv = {}, {}
    T[(-1, O.W_EMBED)] = raw("token_embd.weight")
    if "output.weight" in g.tensors:
        T[(-1, O.W_HEAD)] = raw("output.weight")
    Vv[(-1, O.V_FINAL_NORM)] = vec("output_norm.weight")
    for l in range(L):
        p = "blk.%d." % l
        T[(l, O.W_Q)] = raw(p + "attn_q.weight", p + "attn_q.bias")
        T[(l, O.W_K)] = raw(p + "attn_k.weight", p + "attn_k.bias")
        T[(l, O.W_V)] = raw(p + "attn_v.weight", p + "attn_v.bias")
        T[(l, O.W_O)] = raw(p + "attn_output.weight")
        Vv[(l, O.V_ATTN_NORM)] = vec(p + "attn_norm.weight")
        Vv[(l, O.V_MLP_NORM)] = vec(p + "ffn_norm.weight")
        up, gate = raw(p + "ffn_up.weight"), raw(p + "ffn_gate.weight")
        assert up["type"] == gate["type"]
        T[(l, O.W_GATEUP)] = dict(type=up["type"], rows=up["rows"] * 2, cols=up["cols"],
                                  raw=np.concatenate([up["raw"], gate["raw"]]), scales=None, bias=None)
        T[(l, O.W_DOWN)] = raw(p + "ffn_down.weight")
    return dict(cfg=cfg, tensors=T, vecs=Vv)


def synthetic_spec(cfg, qtype, head_qtype=None, seed=424242, qkv_bias=False, std=0.02):
    """Random-init N(0, std) decoder of the given shape, quantised with the oracle's packers.
    Norm gains are 1 (BASELINE config convention)."""
    rng = np.random.default_rng(seed)
    c = dict(cfg)
    d, hq, hkv, hd, I, V, L = c["d_model"], c["n_q_heads"], c["n_kv_heads"], c["head_dim"], c["ffn"], c["vocab"], c["n_layers"]
    ne = c.get("n_experts", 0)
    for k, v in dict(window=0, qk_norm_full=0, n_experts=0, top_k=0, norm_topk=0, kv_f16=0, acc64=0).items():
        c.setdefault(k, v)
    rn = lambda r, k: rng.standard_normal((r, k), dtype=np.float32) * np.float32(std)
    T, Vv = {}, {}
    T[(-1, O.W_EMBED)] = _t(rn(V, d), head_qtype if head_qtype is not None else qtype)
    if not c.get("tied", False):
        T[(-1, O.W_HEAD)] = _t(rn(V, d), head_qtype if head_qtype is not None else qtype)
    c.pop("tied", None)
    Vv[(-1, O.V_FINAL_NORM)] = np.ones(d, np.float32)
    for l in range(L):
        b = (lambda n: rng.standard_normal(n, dtype=np.float32) * np.float32(std)) if qkv_bias else (lambda n: None)
        T[(l, O.W_Q)] = _t(rn(hq * hd, d), qtype, b(hq * hd))
        T[(l, O.W_K)] = _t(rn(hkv * hd, d), qtype, b(hkv * hd))
        T[(l, O.W_V)] = _t(rn(hkv * hd, d), qtype, b(hkv * hd))
        T[(l, O.W_O)] = _t(rn(d, hq * hd), qtype)
        Vv[(l, O.V_ATTN_NORM)] = np.ones(d, np.float32)
        Vv[(l, O.V_MLP_NORM)] = np.ones(d, np.float32)
        if c["qk_norm_full"]:
            Vv[(l, O.V_Q_NORM)] = np.ones(hq * hd, np.float32)
            Vv[(l, O.V_K_NORM)] = np.ones(hkv * hd, np.float32)
        if ne:
            T[(l, O.W_ROUTER)] = _t(rn(ne, d), qtype)
            T[(l, O.W_GATEUP)] = _t(rn(ne * 2 * I, d), qtype)
            T[(l, O.W_DOWN)] = _t(rn(ne * d, I), qtype)
        else:
            T[(l, O.W_GATEUP)] = _t(rn(2 * I, d), qtype)
            T[(l, O.W_DOWN)] = _t(rn(d, I), qtype)
    return dict(cfg=c, tensors=T, vecs=Vv)


def oracle_model(spec, **override):
    cfgd = dict(spec["cfg"]); cfgd.update(override)
    cfg = O.OrcConfig(**cfgd)
    m = O.OracleModel(cfg)
    for (layer, slot), t in spec["tensors"].items():
        m.set_tensor(layer, slot, t["type"], t["rows"], t["cols"], t["raw"], t["scales"], t["bias"])
    for (layer, slot), v in spec["vecs"].items():
        m.set_vec(layer, slot, v)
    return m
