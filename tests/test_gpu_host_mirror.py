"""The C++ host mirror (neural-api_amd/host): its self-checking program and the command-line greedy decoder."""
import os
import subprocess

import numpy as np
import pytest

from helpers.fixtures_io import ref_path

pytestmark = pytest.mark.gpu
HOST = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "neural-api_amd", "host")


def _built(name):
    p = os.path.join(HOST, name)
    assert os.path.exists(p), "%s is not built: run make in neural-api_amd/csrc" % p
    return p


def test_host_mirror_self_check():
    r = subprocess.run([_built("caihip_host_test"), ref_path("tiny_llama_f32.gguf")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "host mirror ok" in r.stdout, r.stdout + r.stderr


@pytest.mark.parametrize("stepwise", [False, True])
def test_command_line_greedy_decode_matches_the_binding(stepwise):
    from helpers.device import dev
    cai = dev()
    prompt, n_new = [1, 5, 2, 7], 6
    dec = cai.Decoder.from_gguf(ref_path("tiny_llama_f32.gguf"), max_ctx=32)
    want = []
    for p, t in enumerate(prompt):
        am, _ = dec.step(t, p)
    want.append(int(am[0]))
    for k in range(1, n_new):
        am, _ = dec.step(want[-1], len(prompt) + k - 1)
        want.append(int(am[0]))
    cmd = [_built("caihip_run"), ref_path("tiny_llama_f32.gguf"), str(n_new), "--max-ctx", "32"] + (["--stepwise"] if stepwise else []) + [str(t) for t in prompt]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert [int(t) for t in lines[0].split()] == want
    assert lines[1].startswith("stats: prompt 4 tok") and lines[1].endswith("cache %d" % (len(prompt) + n_new - 1))


def test_command_line_reports_loader_errors():
    r = subprocess.run([_built("caihip_run"), ref_path("tiny_kquant.gguf"), "2", "1"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and "general.architecture" in r.stderr
