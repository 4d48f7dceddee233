"""caihip: MI355X (gfx950) quantized LLM decode path for CAI Neural API.

The product is the C-ABI shared library ``libcaihip.so`` (HIP kernels + C entry points declared in
``include/caihip.h``).  This package only locates/builds it and offers a thin ctypes view used by
the tests and the benchmark; it holds no compute of its own and has no CPU fallback.
"""
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("CAIHIP_LIB") or os.path.join(PKG_DIR, "libcaihip.so")   # (CAIHIP_LIB: another build of the library)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")


def build(force=True, jobs=8):
    """Compiles every HIP source for gfx950 into libcaihip.so (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", CSRC_DIR, "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return LIB_PATH


def lib_path():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libcaihip.so is not built; run `make -C neural-api_amd/csrc` (or __graft_entry__.build())")
    return LIB_PATH
