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


def header_arities():
    with open(os.path.join(ROOT, "include", "caihip.h")) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    out = {}
    for name, args in re.findall(r"^\s*int\s+(cai_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text, re.M | re.S):
        args = args.strip()
        out[name] = 0 if args in ("", "void") else len(args.split(","))
    return out


def pascal_arities():
    with open(os.path.join(ROOT, "neural-api_amd", "pascal", "caihip.pas")) as f:
        text = f.read()
    out = {}
    for name, args in re.findall(r"^function\s+(cai_[a-z0-9_]+)\s*\(([^)]*)\)\s*:\s*LongInt\s*;\s*cdecl\s*;\s*external\s+CAIHIP_LIB\s*;", text, re.M | re.S):
        n = 0
        for group in args.split(";"):
            if group.strip():
                n += len(group.split(":")[0].split(","))
        out[name] = n
    return out


def test_pascal_unit_declares_the_header_symbols_with_the_same_arities():
    """The Free Pascal binding cannot be compiled here (no fpc): at least its externals must name exactly the header's
    entry points, each with the header's number of parameters, every one cdecl and returning a 32-bit integer."""
    h, p = header_arities(), pascal_arities()
    assert sorted(h) == header_symbols()
    assert sorted(p) == sorted(h), "only in header: %s; only in caihip.pas: %s" % (sorted(set(h) - set(p)), sorted(set(p) - set(h)))
    for name in h:
        assert p[name] == h[name], "%s: %d parameters in caihip.h, %d in caihip.pas" % (name, h[name], p[name])


def test_decoder_config_record_matches_the_struct():
    """Field order and count of TCaiDecoderConfig against cai_decoder_config (both packed 4-byte fields)."""
    with open(os.path.join(ROOT, "include", "caihip.h")) as f:
        body = re.search(r"typedef struct cai_decoder_config \{(.*?)\} cai_decoder_config;", f.read(), re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    c_fields = [n.strip() for decl in body.split(";") if decl.strip() for n in re.sub(r"^\s*(int32_t|float)\s+", "", decl.strip()).split(",")]
    with open(os.path.join(ROOT, "neural-api_amd", "pascal", "caihip.pas")) as f:
        rec = re.search(r"TCaiDecoderConfig = packed record(.*?)end;", f.read(), re.S).group(1)
    p_fields = [n.strip() for decl in rec.split(";") if decl.strip() for n in decl.split(":")[0].split(",")]
    assert p_fields == c_fields == [n for n, _ in cai.DecoderConfig._fields_]


def test_more_experts_than_the_router_ranks_are_refused_without_a_device():
    """512 experts is what the router kernel ranks; a larger bank is refused when the decoder is created (before any device
    work, so the answer is the same on a machine without a GPU) instead of leaving expert ids unwritten."""
    import ctypes as C
    lib = cai.load()
    cfg = cai.DecoderConfig(n_layers=1, d_model=256, n_q_heads=2, n_kv_heads=2, head_dim=64, ffn=256, vocab=100, max_ctx=16, eps=1e-5,
                            rope_theta=1e4, n_experts=1024, top_k=8, max_batch=1)
    h = C.c_void_p()
    assert lib.cai_decoder_create(C.byref(cfg), C.byref(h)) == -1
    assert "1024 experts" in cai.last_error()
    cfg.n_experts, cfg.top_k = 8, 9
    assert lib.cai_decoder_create(C.byref(cfg), C.byref(h)) == -1


def pascal_call_sites(path):
    """(name, number of arguments) of every cai_* call in a Pascal source (comments stripped, parentheses balanced)."""
    with open(path) as f:
        text = f.read()
    text = re.sub(r"\{.*?\}", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    calls = []
    for m in re.finditer(r"\b(cai_[a-z0-9_]+)\s*\(", text):
        depth, i, n_args, seen = 1, m.end(), 0, False
        while depth and i < len(text):
            ch = text[i]
            if ch in "([":
                depth += 1; seen = True
            elif ch in ")]":
                depth -= 1
            elif ch == "," and depth == 1:
                n_args += 1
            elif not ch.isspace():
                seen = True
            i += 1
        calls.append((m.group(1), n_args + 1 if seen else 0))
    return calls


def test_pascal_session_unit_calls_only_declared_externals_with_their_arities():
    """caihipsession.pas (the TNNetStreamingDecoder-shaped session over the decoder entry points) cannot be compiled here:
    every library call it makes must at least name an external of caihip.pas and pass the declared number of arguments,
    and it must cover the session surface the chat engine uses."""
    decl = pascal_arities()
    calls = pascal_call_sites(os.path.join(ROOT, "neural-api_amd", "pascal", "caihipsession.pas"))
    assert len(calls) >= 15
    for name, n in calls:
        assert name in decl, "%s is not declared in caihip.pas" % name
        assert n == decl[name], "%s called with %d arguments, declared with %d" % (name, n, decl[name])
    used = {name for name, _ in calls}
    for need in ("cai_init", "cai_decoder_load_gguf", "cai_decoder_step", "cai_decoder_prefill", "cai_decoder_generate", "cai_decoder_candidates",
                 "cai_decoder_truncate", "cai_decoder_reset", "cai_decoder_snapshot", "cai_decoder_restore", "cai_decoder_set_kv_dtype",
                 "cai_decoder_set_eviction", "cai_decoder_cache_rows", "cai_decoder_destroy", "cai_last_error"):
        assert need in used, need
