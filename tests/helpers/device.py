"""Loads the product library for the GPU tests (through its C ABI only)."""
import importlib
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# torch first: it brings its own copy of the HIP runtime, and a process that has started the system's copy through the
# product library before torch's is loaded finds no device from torch afterwards (tests that make weights with torch on
# the device would then depend on which test file ran first)
import torch  # noqa: E402,F401

pkg = importlib.import_module("neural-api_amd")
cai = importlib.import_module("neural-api_amd.caihip")
_inited = False


def dev():
    """Returns the ctypes view after cai_init(0); raises if the HIP library is missing or no GPU is present."""
    global _inited
    if not _inited:
        cai.init(0)
        _inited = True
    return cai


def rel_err(got, want, floor=0.0):
    """max |got - want| / max(max |want|, floor): the logit tolerance metric (bar: <= 1e-3).
    `floor` is the typical magnitude of a result (for a lone output that happens to cancel to ~0)."""
    import numpy as np
    denom = max(float(np.max(np.abs(want))), floor, 1e-30)
    return float(np.max(np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)))) / denom
