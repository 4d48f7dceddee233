"""CPU-side checks of the C-ABI boundary: the library loads and exports every symbol the header declares."""
import ctypes
import os
import re

from helpers.device import ROOT, cai, pkg


def header_symbols():
    with open(os.path.join(ROOT, "include", "caihip.h")) as f:
        text = f.read()
    return sorted(set(re.findall(r"^\s*int\s+(cai_[a-z0-9_]+)\s*\(", text, re.M)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(pkg.lib_path())
    syms = header_symbols()
    assert len(syms) >= 40
    for s in syms:
        assert hasattr(lib, s), "libcaihip.so does not export %s" % s


def test_binding_lists_exactly_the_header_symbols():
    assert sorted(cai.SYMBOLS) == header_symbols()


def test_calls_before_init_fail_with_state_error():
    lib = cai.load()
    # no GPU work: the library must refuse, not crash, and explain itself
    if lib.cai_sync() != 0:
        assert "cai_init" in cai.last_error()


def test_header_is_plain_c():
    import subprocess, tempfile
    with tempfile.NamedTemporaryFile("w", suffix=".c", delete=False) as f:
        f.write('#include "caihip.h"\nint main(void){ cai_decoder_config c; (void)c; return 0; }\n')
        path = f.name
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), path])
    os.unlink(path)
