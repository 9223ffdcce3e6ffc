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


def test_fastcall_bindings_agree_with_ctypes(pa, lib):
    """The hottest entry points are bound through pa_fastcall when it is built (always, after
    __graft_entry__.build()): same addresses, same arguments, same return values and error texts as the
    ctypes functions, and a TypeError / OverflowError where ctypes would have raised one."""
    native = pa._native
    assert os.path.exists(os.path.join(ROOT, "ai-infra-train-infer_amd", "pa_fastcall.so")), "run __graft_entry__.build()"
    assert set(lib.fast_entries) == set(native.FAST_ENTRIES)
    for name in native.FAST_ENTRIES:
        assert getattr(lib, name) is not getattr(lib._cdll, name)
    for name in set(native.SIGNATURES) - set(native.FAST_ENTRIES):
        assert getattr(lib, name) is getattr(lib._cdll, name)
    empty = (1234, 0, 2048, 1234, 1234, None, None, 0, 1234, 128, 128, 1234, 1234, 2048, 0, 16, 8, 128, 16, 100, 0.088,
             0, 1, None, 0, 0, 0, 0, None)                                   # batch 0: returns before touching anything
    cases = [("pa_decode", empty, 0)]
    bad = list(empty)
    bad[14] = -1
    cases.append(("pa_decode", tuple(bad), -1))
    cases.append(("pa_kv_store", (None, None, 0, 0, None, None, None, 4, 1024, 2, 64, None), -1))
    cases.append(("pa_silu_mul", (None, 8, None, 8, None, 8, 0, 0, 8, None), 0))             # no rows
    cases.append(("pa_silu_mul", (None, 8, None, 8, None, 8, 0, 3, 8, None), -1))            # null pointers
    cases.append(("pa_add_rms_norm", (None, 8, None, 0, None, 0, 1e-6, None, 0, None, 8, 0, 3, 8, None), -1))
    cases.append(("pa_sample", (None, 0, 0, 5, 7, 0.7, 0.9, None, None, None), -1))           # two floats in a row
    for name, args, want in cases:
        fast, slow = getattr(lib, name)(*args), getattr(lib._cdll, name)(*args)
        assert fast == slow == want, (name, fast, slow)
        if want:
            getattr(lib, name)(*args)
            text = lib.pa_last_error()
            getattr(lib._cdll, name)(*args)
            assert text == lib.pa_last_error() and name.encode() in text
    with pytest.raises(TypeError):
        lib.pa_decode(*empty[:-1])
    with pytest.raises(TypeError):
        lib.pa_decode(1.5, *empty[1:])
    with pytest.raises(TypeError):
        lib.pa_decode(*empty[:2], "2048", *empty[3:])
    with pytest.raises(OverflowError):
        lib.pa_decode(empty[0], 1 << 40, *empty[2:])
    with pytest.raises(OverflowError):
        lib.pa_decode(-5, *empty[1:])
    # an int where a float goes is taken, as ctypes takes it
    assert lib.pa_decode(*empty[:20], 1, *empty[21:]) == 0
