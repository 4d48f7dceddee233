"""The environment switches the library reads select other code paths (no stream capture; token-by-token prompts;
prompt attention through the decode kernels and the bound of its partial-result buffer; the older form of the small-batch step).  Each is read once per process, so each case runs in a child process with the
variable set and is checked against the oracle there: a Q4_K decoder with QKV bias and 7 query heads per KV head, a 40-token
prompt through cai_decoder_prefill, then 8 greedy tokens through cai_decoder_generate, a window step and the lookup loop."""
import os
import subprocess
import sys

import pytest

from helpers.device import ROOT

pytestmark = pytest.mark.gpu

CHILD = r"""
import sys, importlib
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, %(tests)r)
from helpers import oracle_lib as O
from helpers.model_build import oracle_model, synthetic_spec
from helpers.device import dev, rel_err
cai = dev()
cfg = dict(n_layers=2, d_model=512, n_q_heads=14, n_kv_heads=2, head_dim=128, ffn=1024, vocab=2048, max_ctx=96, eps=1e-6, rope_theta=1e6)
spec = synthetic_spec(cfg, O.Q4_K, head_qtype=O.Q8_0, qkv_bias=True, std=0.05)
om, dec = oracle_model(spec, acc64=1), cai.Decoder(spec)
prompt = np.random.default_rng(7).integers(0, cfg["vocab"], 40).tolist()
for p, t in enumerate(prompt):
    tok_o, lo = om.step(t, p)
tok_d, ld = dec.prefill(prompt, 0)
assert rel_err(ld, lo) < 1e-3, rel_err(ld, lo)
assert tok_d == tok_o
gen = dec.generate(tok_d, len(prompt), 8).tolist()
ref = []
for i in range(8):
    tok_o, _ = om.step(tok_o, len(prompt) + i); ref.append(tok_o)
assert gen == ref, (gen, ref)
# a width-5 window of the same sequence (eager launches under CAIHIP_NO_GRAPH) and the lookup loop built on it
dec.truncate(len(prompt))
am, lg = dec.step_window([tok_d] + gen[:4], len(prompt))
assert am.tolist() == gen[:5], (am.tolist(), gen)
dec.truncate(len(prompt))
got, passes = dec.generate_lookup(prompt + [tok_d], 8, 1, 4)
assert got.tolist() == gen and passes <= 8
print("CHILD_OK")
"""


@pytest.mark.parametrize("switches", [{"CAIHIP_NO_GRAPH": "1"}, {"CAIHIP_PREFILL_TOKENWISE": "1"}, {"CAIHIP_PROMPT_FLASH": "0"},
                                      # prompt attention on the decode kernels with room for 4 rows' partial results per launch
                                      # (14 heads x 1 slice x 130 floats a row): the 40-token prompt attends in 10 groups
                                      {"CAIHIP_PROMPT_FLASH": "0", "CAIHIP_PROMPT_PART_KB": "32"},
                                      # batched / window steps of a Q4_K model through the form with activation planes and slice
                                      # partials (the one-launch form takes them otherwise)
                                      {"CAIHIP_SMALL_BATCH_PLANES": "1"}])
def test_switch_selected_path_matches_the_oracle(switches):
    env = dict(os.environ); env.update(switches)
    code = CHILD % dict(root=ROOT, tests=os.path.join(ROOT, "tests"))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "CHILD_OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]


MOE_CHILD = r"""
import sys
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, %(tests)r)
from helpers import oracle_lib as O
from helpers.model_build import oracle_model, synthetic_spec
from helpers.device import dev, rel_err
cai = dev()
# 16 KV heads x 16 slices of 64 rows = 256 work-groups: the decode attention of this cache is the one-work-group-per-KV-head kernel
cfg = dict(n_layers=2, d_model=256, n_q_heads=32, n_kv_heads=16, head_dim=128, ffn=96, vocab=512, max_ctx=1024, eps=1e-5, rope_theta=1e4,
           n_experts=8, top_k=3, norm_topk=1)
spec = synthetic_spec(cfg, O.Q8_0, std=0.05)
om, dec = oracle_model(spec, kv_f16=1), cai.Decoder(spec, kv_dtype=cai.KV_F16)
prompt = np.random.default_rng(11).integers(0, cfg["vocab"], 70).tolist()      # crosses a slice boundary
for p, t in enumerate(prompt):
    tok_o, lo = om.step(t, p)
    tok_d, ld = dec.step(np.array([t]), np.array([p]))
    assert rel_err(ld[0], lo) < 1e-3, (p, rel_err(ld[0], lo))
    assert int(tok_d[0]) == tok_o, p
print("CHILD_OK")
"""


@pytest.mark.parametrize("switches", [{}, {"CAIHIP_ATTN_GROUP_MFMA": "0"}, {"CAIHIP_ROUTER_LAUNCHES": "1"}, {"CAIHIP_MOE_DOWN_LAUNCHES": "1"}])
def test_moe_fp16_cache_paths_match_the_oracle(switches):
    """A Q8_0 mixture-of-experts decoder over a half-precision cache, token by token against the oracle: by default the grouped
    decode attention runs on the matrix cores, the router is one launch (products, soft-max and top-k; the last work-group to
    arrive selects) and the gathered down projection adds the gate-weighted mixture itself; each switch puts one of the three back
    on its separate launches."""
    env = dict(os.environ); env.update(switches)
    code = MOE_CHILD % dict(root=ROOT, tests=os.path.join(ROOT, "tests"))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "CHILD_OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]


ATTN_CHILD = r"""
import sys
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, %(tests)r)
from helpers.device import dev
from test_gpu_attention import oracle_run, oracle_run_i8
cai = dev()
hq, hkv, dk, ctx, n = 40, 8, 128, 8192, 90          # 8 KV heads x 33 slices: the one-work-group-per-KV-head kernel
rows = np.random.default_rng(5).standard_normal((n, (hq + 2 * hkv) * dk)).astype(np.float32)
for kv, window, softcap in (("f16", 0, 0.0), ("i8", 70, 25.0)):
    if kv == "i8":
        want, (kq, vq, ks, vs) = oracle_run_i8(rows, hq, hkv, dk, n, window, softcap)
    else:
        want = oracle_run(rows, hq, hkv, dk, n, window, 1, softcap)
    cache = cai.KVCache(1, hkv, dk, ctx, cai.KV_I8 if kv == "i8" else cai.KV_F16)
    for pos in range(n):
        got = cache.attn_decode(0, rows[pos], hq, window, softcap)
        assert np.max(np.abs(got - want[pos])) < 1e-5 * max(1.0, np.max(np.abs(want[pos]))), (kv, pos)
    if kv == "i8":
        k, v, s_k, s_v = cache.export_layer(0)
        np.testing.assert_array_equal(k, kq); np.testing.assert_array_equal(v, vq)
        np.testing.assert_array_equal(s_k, ks); np.testing.assert_array_equal(s_v, vs)
print("CHILD_OK")
"""


def test_grouped_attention_valu_form_under_its_switch():
    """CAIHIP_ATTN_GROUP_MFMA=0: half-precision and int8 caches of 128-wide heads go back to the VALU form of the per-KV-head
    decode kernel (the default takes them to the matrix-core form, tests/test_gpu_attention.py): same bar, int8 codes and scales exact."""
    env = dict(os.environ); env["CAIHIP_ATTN_GROUP_MFMA"] = "0"
    code = ATTN_CHILD % dict(root=ROOT, tests=os.path.join(ROOT, "tests"))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "CHILD_OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]


SHUTDOWN_CHILD = r"""
import sys, importlib
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, %(tests)r)
from helpers import oracle_lib as O
from helpers.model_build import synthetic_spec
from helpers.device import dev, rel_err
cai = dev()
cfg = dict(n_layers=2, d_model=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=1024, vocab=600, max_ctx=96, eps=1e-5, rope_theta=1e4)
spec = synthetic_spec(cfg, O.Q4_K, head_qtype=O.Q8_0, std=0.05)
prompt = np.random.default_rng(3).integers(0, cfg["vocab"], 40).tolist()

def session():
    dec = cai.Decoder(spec, max_batch=3)
    out = [dec.prefill(prompt, 0, seq=b)[1].copy() for b in range(3)]          # prompt workspace
    tok = np.full(3, 5)
    for i in range(4):                                                          # small-batch workspace, captured graph
        tok, lg = dec.step(tok, np.full(3, len(prompt) + i)); out.append(lg.copy())
    dec.close()
    return out

a = session()
cai.check(cai.load().cai_shutdown())          # frees the stream, the staging buffers and both activation workspaces
cai.init(0)
b = session()
for x, y in zip(a, b):
    assert np.array_equal(np.asarray(x), np.asarray(y))
cai.check(cai.load().cai_shutdown())
print("CHILD_OK")
"""


def test_shutdown_frees_the_workspaces_and_a_second_init_runs_the_same():
    """cai_shutdown followed by cai_init in one process: the matrix-core paths allocate their activation workspaces afresh and
    every result is bit-identical to the first session's."""
    code = SHUTDOWN_CHILD % dict(root=ROOT, tests=os.path.join(ROOT, "tests"))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "CHILD_OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]


LATE_PROMPT_CHILD = r"""
import sys, importlib
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, %(tests)r)
from helpers import oracle_lib as O
from helpers.model_build import synthetic_spec
from helpers.device import dev, rel_err
cai = dev()
cfg = dict(n_layers=1, d_model=128, n_q_heads=2, n_kv_heads=1, head_dim=64, ffn=256, vocab=512, max_ctx=36864, eps=1e-5, rope_theta=1e4)
spec = synthetic_spec(cfg, O.Q8_0, head_qtype=O.Q8_0, std=0.08)
dec = cai.Decoder(spec)
toks = np.random.default_rng(11).integers(0, cfg["vocab"], 33000).tolist()
head, tail = toks[:-96], toks[-96:]
dec.prefill(head, 0)
tok_a, la = dec.prefill(tail, len(head))          # 288 slices x 2 heads x 66 floats = 152 KB a row: groups of 13 rows under the 2 MB bound
dec.truncate(len(head))
for i, t in enumerate(tail):
    am, lb = dec.step(t, len(head) + i)
assert rel_err(la, lb[0]) < 1e-4, rel_err(la, lb[0])
assert tok_a == int(am[0])
print("CHILD_OK")
"""


def test_prompt_late_in_a_long_cache_on_the_decode_kernels_attends_in_bounded_groups():
    """A head_dim-64 model (its prompts attend through the decode kernels) with a 36864-row cache: 96 prompt tokens at position
    32904 need 288 slices of partial results per row and head; with the buffer bounded to 2 MB they attend in groups of 13 rows.
    The result equals stepping the same 96 tokens one at a time (the reference's own prompt order,
    neural/neuralchatengine.pas:1466-1470; that path is compared with the oracle elsewhere - the oracle itself would need
    minutes for 33000 positions)."""
    env = dict(os.environ); env["CAIHIP_PROMPT_PART_KB"] = "2048"
    code = LATE_PROMPT_CHILD % dict(root=ROOT, tests=os.path.join(ROOT, "tests"))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "CHILD_OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
