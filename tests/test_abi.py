"""The C-ABI library loads on a machine without a GPU and exports every function that
include/paged_attn.h declares; the ctypes prototypes cover the same set."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "paged_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pa_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("pa_kv_store", "pa_kv_store_fp8", "pa_decode", "pa_decode_partials", "pa_merge",
                 "pa_prefill", "pa_workspace_bytes", "pa_last_error", "pa_version"):
        assert must in names


def test_library_exports_every_declared_symbol(pa):
    assert pa._native.is_built(), "libpaged_attn.so missing: run __graft_entry__.build()"
    lib = ctypes.CDLL(pa._native.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name


def test_ctypes_prototypes_match_the_header(pa):
    assert sorted(pa._native.SIGNATURES) == declared_functions()
    text = open(os.path.join(ROOT, "include", "paged_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for name, (_res, argtypes) in pa._native.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^)]*)\)" % name, text)
        args = m.group(1).strip()
        n = 0 if args in ("", "void") else len(args.split(","))
        assert n == len(argtypes), (name, n, len(argtypes))


def test_host_only_calls(lib):
    assert lib.pa_version() >= 2
    assert lib.pa_workspace_bytes(64, 16, 128, 8) >= 64 * 16 * 8 * (128 + 2) * 4
    # argument errors are reported before any launch, so these run without a GPU
    assert lib.pa_kv_store(None, None, 0, 0, None, None, None, 4, 1024, 2, 64, None) == -1
    assert lib.pa_decode(None, 0, 0, None, None, None, None, 0, None, 0, 0, None, None, 0, 1, 16, 8,
                         128, 16, 4, 1.0, 0, 1, None, 0, 0, 0, 0, None) == -1
    assert lib.pa_decode_noalloc(None, 0, 0, None, None, None, None, 0, None, 0, 0, None, None, 0, 1, 16, 8,
                                 128, 16, 4, 1.0, 0, 1, 0, 0, 0, None) == -1
    # partials beyond the built-in scratch are refused before anything touches a GPU
    assert lib.pa_workspace_bytes(4096, 16, 128, 64) > 16 * 1024 * 1024
    assert lib.pa_decode_noalloc(None, 0, 0, None, None, None, None, 0, None, 0, 0, None, None, 0, 4096, 16, 8,
                                 128, 16, 4, 1.0, 512, 64, 0, 0, 0, None) == -4
    assert b"scratch" in lib.pa_last_error()
