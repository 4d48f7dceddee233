"""The three environment switches the library reads select other code paths (no stream capture; token-by-token prompts;
prompt attention through the decode kernels).  Each is read once per process, so each case runs in a child process with the
variable set and is checked against the oracle there: a Q4_K decoder with QKV bias and 7 query heads per KV head, a 40-token
prompt through cai_decoder_prefill, then 8 greedy tokens through cai_decoder_generate."""
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
print("CHILD_OK")
"""


@pytest.mark.parametrize("var,val", [("CAIHIP_NO_GRAPH", "1"), ("CAIHIP_PREFILL_TOKENWISE", "1"), ("CAIHIP_PROMPT_FLASH", "0")])
def test_switch_selected_path_matches_the_oracle(var, val):
    env = dict(os.environ); env[var] = val
    code = CHILD % dict(root=ROOT, tests=os.path.join(ROOT, "tests"))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "CHILD_OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
