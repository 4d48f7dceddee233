"""bench.py's command-line contract that needs no GPU: one GPU only (a larger --gpus exits with a message, before anything touches
a device), and the flags the profiles' commands use exist."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_flags_used_by_the_committed_profile_commands_exist():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0
    for flag in ("--steps", "--warmup", "--config", "--no-cpu-baseline", "--reps", "--kernel-reps", "--kv", "--batch", "--prompt", "--max-ctx",
                 "--gemv-sweep", "--gemm-sweep", "--copy-calibration"):
        assert flag in r.stdout, flag
