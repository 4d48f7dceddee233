#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode tok/s on the Qwen2.5-7B shape (Q4_K body, Q8_0 head) on one MI355X.

One "step" is one decoded token: the whole per-token pass of the quantized decode path (28 blocks + head + arg-max)
with weights, KV cache and activations resident in HBM.  Prints ONE JSON line (see the keys below).
"""
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E bandwidth

CONFIGS = {
    # BASELINE.json configs[2]: Qwen2.5-7B shape, Q4_K body, Q8_0 untied head, QKV bias
    "qwen2.5-7b-q4k": dict(cfg=dict(n_layers=28, d_model=3584, n_q_heads=28, n_kv_heads=4, head_dim=128, ffn=18944, vocab=152064,
                                    max_ctx=768, eps=1e-6, rope_theta=1e6), qtype="Q4_K", head="Q8_0", bias=True, prompt=512),
    # the same shape as llama.cpp's Q4_K_M preset writes it: output.weight and attn_v / ffn_down of about half the blocks in Q6_K
    "qwen2.5-7b-q4_k_m": dict(cfg=dict(n_layers=28, d_model=3584, n_q_heads=28, n_kv_heads=4, head_dim=128, ffn=18944, vocab=152064,
                                       max_ctx=768, eps=1e-6, rope_theta=1e6), qtype="Q4_K", head="Q6_K", embed="Q4_K", q6k_mix=True, bias=True, prompt=512),
    # BASELINE.json configs[0] (the reference's own CPU-runnable case): SmolLM2-135M shape, Q8_0, tied head
    "smollm2-135m-q8_0": dict(cfg=dict(n_layers=30, d_model=576, n_q_heads=9, n_kv_heads=3, head_dim=64, ffn=1536, vocab=49152,
                                       max_ctx=256, eps=1e-5, rope_theta=1e5, tied=True), qtype="Q8_0", head="Q8_0", bias=False, prompt=16),
    # configs[3]: OLMoE-1B-7B shape, Q8_0, 64 experts top-8, full-width QK norm
    "olmoe-1b-7b-q8_0": dict(cfg=dict(n_layers=16, d_model=2048, n_q_heads=16, n_kv_heads=16, head_dim=128, ffn=1024, vocab=50304,
                                      max_ctx=768, eps=1e-5, rope_theta=1e4, qk_norm_full=1, n_experts=64, top_k=8, norm_topk=0),
                             qtype="Q8_0", head="Q8_0", bias=False, prompt=256),
    # configs[4]: Qwen2.5-32B shape, Q4_K body and head, fp16 KV cache, 8192-token context (batch via --batch)
    "qwen2.5-32b-q4k": dict(cfg=dict(n_layers=64, d_model=5120, n_q_heads=40, n_kv_heads=8, head_dim=128, ffn=27648, vocab=152064,
                                     max_ctx=8448, eps=1e-6, rope_theta=1e6), qtype="Q4_K", head="Q4_K", bias=True, prompt=8192, kv="f16"),
    # reduced shapes for quick local runs of this script
    "tiny-q4k": dict(cfg=dict(n_layers=2, d_model=512, n_q_heads=4, n_kv_heads=2, head_dim=128, ffn=1024, vocab=4096,
                              max_ctx=256, eps=1e-6, rope_theta=1e6), qtype="Q4_K", head="Q8_0", bias=True, prompt=16),
}


def cpu_baseline(cfg, seconds_budget=20.0):
    """Restated reference AVX2 int8-per-row path (oracle/cpu_baseline.c) on a bounded sample of the same workload:
    ONE decoder block's linear layers + the LM head, timed on this host's cores; extrapolated to a full token."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from helpers import oracle_lib as O
    L = O.lib()
    threads = min(L.cpu_max_threads(), 16)
    d, I, V = cfg["d_model"], cfg["ffn"], cfg["vocab"]
    qw, kw = cfg["n_q_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    shapes = [(qw, d), (kw, d), (kw, d), (d, qw), (2 * I, d), (d, I)]
    rng = np.random.default_rng(0)
    mats = []
    for r, c in shapes + [(V, d)]:
        codes = rng.integers(-127, 128, (r, c), dtype=np.int8)
        scales = np.full(r, 1e-3, np.float32)
        mats.append((codes, scales, np.empty(r, np.float32), rng.standard_normal(c).astype(np.float32)))

    def run(ms):
        for codes, scales, y, x in ms:
            L.cpu_linear_int8(codes.ctypes.data, scales.ctypes.data, codes.shape[0], codes.shape[1], x.ctypes.data, 1, None, y.ctypes.data, threads)

    run(mats)  # warm-up
    reps, t_layer, t_head = 0, [], []
    t_end = time.perf_counter() + seconds_budget
    while time.perf_counter() < t_end and reps < 8:
        t0 = time.perf_counter(); run(mats[:-1]); t1 = time.perf_counter(); run(mats[-1:]); t2 = time.perf_counter()
        t_layer.append(t1 - t0); t_head.append(t2 - t1); reps += 1
    tl, th = sorted(t_layer)[len(t_layer) // 2], sorted(t_head)[len(t_head) // 2]
    tok_s = 1.0 / (cfg["n_layers"] * tl + th)
    return {"value": round(tok_s, 3), "unit": "tok/s", "cores": threads, "kind": "port",
            "sample": "restated AVX2 int8-per-row kernels (reference's default ChatTerminal path): 1 of %d blocks' linear layers + LM head, "
                      "median of %d runs, extrapolated to a full token; attention/norms excluded" % (cfg["n_layers"], reps)}


def gemv_sweep(cai, synth, torch, with_cpu):
    """One JSON line per (type, shape, batch): resident blocks, x and y on the device, HIP-event time per launch while
    rotating over enough copies of the matrix to exceed the 256 MB infinity cache (at most 24 copies: the small shapes stay
    cache-resident and are labelled so)."""
    lib = cai.load()
    QT = {"Q8_0": (cai.Q8_0, 34 / 32), "Q4_0": (cai.Q4_0, 18 / 32), "Q4_K": (cai.Q4_K, 144 / 256), "Q6_K": (cai.Q6_K, 210 / 256),
          "I8ROW": (cai.I8ROW, 1.0)}   # I8ROW: the reference's own per-row int8 format
    shapes = [(2048, 2048), (5632, 2048), (2048, 5632), (18944, 3584), (152064, 3584)]
    gen = torch.Generator(device="cuda"); gen.manual_seed(424242)
    cpu = None
    if with_cpu:
        import numpy as np
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        from helpers import oracle_lib as O
        cpu = O.lib()
    for name, (qt, bpw) in QT.items():
        for rows, cols in shapes:
            mat_bytes = rows * cols * bpw
            copies = int(max(1, min(24, -(-320e6 // mat_bytes))))
            ws = [synth.random_int8_rows(rows, cols, gen) if name == "I8ROW" else synth.random_qweight(qt, rows, cols, gen)[0] for _ in range(copies)]
            for nb in (1, 4):
                x = torch.randn(nb, cols, device="cuda"); y = torch.empty(nb, rows, device="cuda")
                torch.cuda.synchronize()
                for w in ws:
                    cai.check(lib.cai_qgemv(w.h, x.data_ptr(), nb, y.data_ptr(), 0, cai.X_DEVICE | cai.Y_DEVICE))
                reps = max(2, int(200 // copies))
                cai.check(lib.cai_sync()); cai.check(lib.cai_timer_start())
                for _ in range(reps):
                    for w in ws:
                        cai.check(lib.cai_qgemv(w.h, x.data_ptr(), nb, y.data_ptr(), 0, cai.X_DEVICE | cai.Y_DEVICE))
                ms = C.c_float(); cai.check(lib.cai_timer_stop(C.byref(ms)))
                us = ms.value * 1e3 / (reps * copies)
                algo = mat_bytes + 4 * cols * nb + 4 * rows * nb
                line = {"gemv": name, "rows": rows, "cols": cols, "batch": nb, "us_per_launch": round(us, 2),
                        "algorithmic_bytes": int(algo), "GB_per_s": round(algo / us / 1e3, 1), "frac_of_8TBps": round(algo / us / 1e3 / HBM_PEAK_GBS, 4),
                        "working_set": "hbm" if copies * mat_bytes > 300e6 else "cache-resident (%d x %.1f MB)" % (copies, mat_bytes / 1e6)}
                if cpu is not None and nb == 1 and name == "I8ROW":
                    # restated reference AVX2 int8-per-row kernel on the same shape (1 B/weight), all host threads
                    import numpy as np
                    thr = min(cpu.cpu_max_threads(), 16)
                    rng = np.random.default_rng(0)
                    codes = rng.integers(-127, 128, (rows, cols), dtype=np.int8); sc = np.full(rows, 1e-3, np.float32)
                    xv = rng.standard_normal(cols).astype(np.float32); yv = np.empty(rows, np.float32)
                    ts = []
                    for _ in range(5):
                        t0 = time.perf_counter()
                        cpu.cpu_linear_int8(codes.ctypes.data, sc.ctypes.data, rows, cols, xv.ctypes.data, 1, None, yv.ctypes.data, thr)
                        ts.append(time.perf_counter() - t0)
                    t = sorted(ts)[2]
                    line["cpu_int8row_port"] = {"us": round(t * 1e6, 1), "GB_per_s": round(rows * cols / t / 1e9, 2), "cores": thr}
                print(json.dumps(line), flush=True)
            for w in ws:
                w.close()
            del ws
            torch.cuda.empty_cache()


# HBM bytes per launch of the 7B-shape gate|up kernel from hardware counters (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000
# KiB, factors from a 1 GiB copy kernel): profiles/gemv_q4k_gateup_qwen7b_hbm_traffic.txt.  Not measurable from
# inside this process; re-collect when the kernel changes.
GATEUP_TRAFFIC_BYTES = int((37522.5 * 2.000 + 74.2 * 1.000) * 1024)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=192)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="qwen2.5-7b-q4k", choices=list(CONFIGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--kernel-reps", type=int, default=5)
    ap.add_argument("--kv", choices=["f32", "f16", "i8"], default=None, help="KV cache element type (default: the configuration's own)")
    ap.add_argument("--batch", type=int, default=1, help="independent sequences decoded together (1..8)")
    ap.add_argument("--gemv-sweep", action="store_true", help="isolated matrix-vector sweep (BASELINE configs[1]): Q8_0 / Q4_0 / Q4_K and per-row int8, five shapes, batch 1 and 4")
    ap.add_argument("--copy-calibration", action="store_true", help="only run the 1 GiB device copy kernel 5 times (reference for traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives are part of it)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    importlib.import_module("neural-api_amd")
    cai = importlib.import_module("neural-api_amd.caihip")
    synth = importlib.import_module("neural-api_amd.synth")
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr); sys.exit(3)
    cai.init(0)
    if args.copy_calibration:
        a = torch.ones(1 << 28, dtype=torch.float32, device="cuda"); b = torch.empty_like(a)
        torch.cuda.synchronize()
        for _ in range(5):
            cai.check(cai.load().cai_dev_copy(b.data_ptr(), a.data_ptr(), a.numel() * 4))
        cai.check(cai.load().cai_sync())
        print(json.dumps({"copy_calibration": {"bytes_read": a.numel() * 4, "bytes_written": a.numel() * 4, "launches": 5}}))
        return
    if args.gemv_sweep:
        gemv_sweep(cai, synth, torch, not args.no_cpu_baseline)
        return
    conf = CONFIGS[args.config]
    cfg = dict(conf["cfg"])
    prompt_len = conf["prompt"]
    K, W = args.steps, args.warmup
    if prompt_len + W + K > cfg["max_ctx"]:
        cfg["max_ctx"] = prompt_len + W + K
    QT = {"Q4_K": cai.Q4_K, "Q8_0": cai.Q8_0, "Q4_0": cai.Q4_0, "Q6_K": cai.Q6_K}
    t0 = time.time()
    spec = synth.random_decoder_spec(cfg, QT[conf["qtype"]], QT[conf["head"]], seed=424242, qkv_bias=conf["bias"],
                                     embed_qtype=QT[conf["embed"]] if "embed" in conf else None, q6k_mix=conf.get("q6k_mix", False))
    B = args.batch
    kv_kind = args.kv or conf.get("kv", "f32")
    dec = cai.Decoder(spec, max_batch=B, kv_dtype={"f32": cai.KV_F32, "f16": cai.KV_F16, "i8": cai.KV_I8}[kv_kind])
    torch.cuda.empty_cache()
    t_build = time.time() - t0
    wbytes = dec.weight_bytes()
    n_lin_weights = cfg["n_layers"] * (cfg["d_model"] * (cfg["n_q_heads"] + 2 * cfg["n_kv_heads"]) * cfg["head_dim"] + cfg["n_q_heads"] * cfg["head_dim"] * cfg["d_model"] + 3 * cfg["ffn"] * cfg["d_model"])

    rng = np.random.default_rng(424242)
    prompt = rng.integers(0, cfg["vocab"], prompt_len).astype(np.int32)
    lib = cai.load()
    pf_ms = C.c_float(0)
    if prompt_len > 1:
        dec.prefill(prompt[:min(8, prompt_len - 1)], 0, want_logits=False)   # warm the prefill kernels and buffers
        dec.reset()
        cai.check(lib.cai_sync()); cai.check(lib.cai_timer_start())
        dec.prefill(prompt[:-1], 0, want_logits=False)
        cai.check(lib.cai_timer_stop(C.byref(pf_ms)))
        for b in range(1, B):
            dec.prefill(prompt[:-1], 0, seq=b, want_logits=False)
    tok = int(prompt[-1]); pos = prompt_len - 1

    def decode(tok, pos, n):
        """n greedy steps of all B sequences; batch 1 chains the steps on the device, a batch steps from the host"""
        if B == 1:
            out = dec.generate(tok, pos, n)
            return int(out[-1])
        toks = np.full(B, tok, np.int32) if np.isscalar(tok) else tok
        for i in range(n):
            toks, _ = dec.step(toks, np.full(B, pos + i, np.int32), want_logits=False)
        return toks

    if W > 0:
        tok = decode(tok, pos, W); pos += W
    cai.check(lib.cai_sync()); torch.cuda.synchronize()
    ms = C.c_float()
    t1 = time.perf_counter()
    cai.check(lib.cai_timer_start())
    decode(tok, pos, K)
    cai.check(lib.cai_timer_stop(C.byref(ms)))
    cai.check(lib.cai_sync()); torch.cuda.synchronize()
    wall = time.perf_counter() - t1
    ms_per_step = wall * 1e3 / K
    tok_s = K * B / wall
    ctx_mid = pos + K // 2
    kv_bytes = B * cfg["n_layers"] * 2 * cfg["n_kv_heads"] * cfg["head_dim"] * {"f32": 4, "f16": 2, "i8": 1}[kv_kind] * ctx_mid
    ne = cfg.get("n_experts", 0)
    algo_bytes = wbytes + kv_bytes

    # ---- dominant kernel: fused RMSNorm + gate|up GEMV + SwiGLU (76.4 MB of blocks per launch at the 7B shape) ----
    L = cfg["n_layers"]
    if ne:
        print(json.dumps({"metric": "decode tok/s (%s)" % args.config, "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
                          "ms_per_step": round(ms_per_step, 4), "batch": B, "algorithmic_bytes_per_step": int(algo_bytes),
                          "whole_step_hbm_frac": round(algo_bytes / (wall / K) / 1e9 / HBM_PEAK_GBS, 4),
                          "prefill": {"tokens": prompt_len - 1, "ms": round(pf_ms.value, 2)}}))
        return
    gu = [spec["tensors"][(l, cai.W_GATEUP)]["qw"] for l in range(L)]
    d, I = cfg["d_model"], cfg["ffn"]
    x = torch.randn(d, device="cuda"); g = torch.ones(d, device="cuda"); y = torch.empty(I, device="cuda")
    torch.cuda.synchronize()
    for w in gu:  # warm the code path; rotating over all layers keeps the 256 MB infinity cache cold like a real token
        cai.check(lib.cai_ffn_gateup(w.h, x.data_ptr(), g.data_ptr(), cfg["eps"], 1, y.data_ptr(), cai.X_DEVICE | cai.Y_DEVICE))
    cai.check(lib.cai_sync())
    cai.check(lib.cai_timer_start())
    for _ in range(args.kernel_reps):
        for w in gu:
            cai.check(lib.cai_ffn_gateup(w.h, x.data_ptr(), g.data_ptr(), cfg["eps"], 1, y.data_ptr(), cai.X_DEVICE | cai.Y_DEVICE))
    kms = C.c_float()
    cai.check(lib.cai_timer_stop(C.byref(kms)))
    k_avg_us = kms.value * 1e3 / (args.kernel_reps * L)
    qbytes = {"Q4_K": 144 / 256, "Q8_0": 34 / 32, "Q4_0": 18 / 32}[conf["qtype"]]
    k_bytes = 2 * I * d * qbytes + 4 * d * 2 + 4 * I     # blocks + x + gain + y
    k_gbs = k_bytes / (k_avg_us * 1e-6) / 1e9

    res = {
        "metric": "decode tok/s @bs1 (Qwen2.5-7B-shape Q4_K) + % of HBM-bandwidth roofline" if args.config == "qwen2.5-7b-q4k" and B == 1
                  else "decode tok/s (%s, batch %d)" % (args.config, B),
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "q4_k/q8_0 weights, f32 accumulate", "data": "synthetic",
        "config": {"workload": "%s: %d-token random prompt (seed 424242), then greedy decode at batch %d; timed %d decode steps at ctx %d..%d"
                               % (args.config, prompt_len, B, K, pos + 1, pos + K),
                   "weights": "random N(0,0.02), %s body + %s head, %s KV cache" % (conf["qtype"], conf["head"], kv_kind),
                   "algorithmic_bytes_per_step": int(algo_bytes), "hip_event_ms_per_step": round(ms.value / K, 4),
                   "whole_step_hbm_frac": round(algo_bytes / (wall / K) / 1e9 / HBM_PEAK_GBS, 4), "device": cai.device_name(),
                   "build_s": round(t_build, 1),
                   "prefill": {"tokens": prompt_len - 1, "ms": round(pf_ms.value, 2),
                               "tok_per_s": round((prompt_len - 1) / max(pf_ms.value, 1e-6) * 1e3, 1),
                               "linear_tflops": round(2.0 * n_lin_weights * (prompt_len - 1) / max(pf_ms.value, 1e-6) / 1e9, 1),
                               "note": "multi-token ingestion: f16 MFMA (exact scale*nibble weight operand, hi/lo-split activations = 2 MFMA passes per useful FLOP) + prompt attention; MFMA f16 dense peak 2500 TFLOP/s"}},
        "roofline": {"bound": "hbm", "kernel": "%s (RMSNorm+gate|up+SwiGLU, %dx%d)" % ("gemv_q4k_dot<1,1,false,2>" if conf["qtype"] == "Q4_K" else "gemv_fast<%s>" % conf["qtype"], 2 * I, d),
                     "achieved": round(k_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(k_gbs / HBM_PEAK_GBS, 4),
                     "avg_launch_us": round(k_avg_us, 2), "algorithmic_bytes_per_launch": int(k_bytes),
                     "traffic": GATEUP_TRAFFIC_BYTES if args.config == "qwen2.5-7b-q4k" else None, "traffic_unit": "bytes/launch"},
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
