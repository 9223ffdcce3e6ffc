"""ctypes binding of libpaged_attn.so (the C ABI declared in include/paged_attn.h).

The library is the only compute path of this package: there is no CPU or PyTorch fallback.
If it has not been built, every call raises RuntimeError.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpaged_attn.so")

PA_OK = 0
PA_ERR_BAD_ARG = -1
PA_ERR_UNSUPPORTED = -2
PA_ERR_LAUNCH = -3
PA_ERR_WORKSPACE = -4

DTYPE_F16 = 0
DTYPE_BF16 = 1
DTYPE_F32 = 2
DTYPE_FP8_E4M3 = 3

_i64 = ctypes.c_int64
_int = ctypes.c_int
_ptr = ctypes.c_void_p
_f32 = ctypes.c_float

# name -> (restype, argtypes); mirrors include/paged_attn.h one to one
SIGNATURES = {
    "pa_version": (_int, []),
    "pa_last_error": (ctypes.c_char_p, []),
    "pa_kv_store": (_int, [_ptr, _ptr, _i64, _i64, _ptr, _ptr, _ptr, _i64, _i64, _int, _i64, _ptr]),
    "pa_kv_store_fp8": (_int, [_ptr, _ptr, _int, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _i64,
                               _i64, _i64, _ptr]),
    "pa_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "pa_decode": (_int, [_ptr, _int, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64, _i64, _ptr, _ptr,
                         _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _i64, _ptr, _i64,
                         _int, _int, _int, _ptr]),
    "pa_decode_shared_prefix": (_int, [_ptr, _int, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64, _i64, _ptr, _ptr,
                                       _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _i64, _ptr, _i64,
                                       _int, _ptr, _i64, _ptr, _i64, _i64, _i64, _ptr, _i64, _ptr]),
    "pa_check_shared_prefix": (_int, [_ptr, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr]),
    "pa_decode_noalloc": (_int, [_ptr, _int, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64, _i64, _ptr,
                                 _ptr, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _i64,
                                 _int, _int, _int, _ptr]),
    "pa_decode_partials": (_int, [_ptr, _int, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64, _i64, _ptr,
                                  _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _i64, _ptr, _i64,
                                  _int, _int, _int, _ptr]),
    "pa_merge": (_int, [_ptr, _i64, _ptr, _ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64, _ptr]),
    "pa_prefill": (_int, [_ptr, _int, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64, _ptr, _ptr,
                          _ptr, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _int, _ptr]),
    "pa_fp8_e4m3_to_f32": (_int, [_ptr, _ptr, _i64, _ptr]),
    "pa_f32_to_fp8_e4m3": (_int, [_ptr, _ptr, _i64, _ptr]),
    "pa_qk_norm_rope_store": (_int, [_ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _int, _f32, _ptr,
                                     _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64,
                                     _i64, _i64, _i64, _i64, _ptr]),
    "pa_sample": (_int, [_ptr, _int, _i64, _i64, _i64, _f32, _f32, _ptr, _ptr, _ptr]),
    "pa_copy_blocks": (_int, [_ptr, _i64, _i64, _i64, _i64, _ptr, _i64, _ptr]),
    "pa_add_rms_norm": (_int, [_ptr, _i64, _ptr, _i64, _ptr, _int, _f32, _ptr, _i64, _ptr, _i64, _int, _i64, _i64, _ptr]),
    "pa_silu_mul": (_int, [_ptr, _i64, _ptr, _i64, _ptr, _i64, _int, _i64, _i64, _ptr]),
    "pa_gather_kv": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _ptr, _i64, _ptr, _ptr, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _ptr]),
    "pa_decode_advance": (_int, [_ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _ptr]),
    "pa_prefill_metadata": (_int, [_ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _i64, _i64, _ptr]),
    "pa_slot_mapping": (_int, [_ptr, _ptr, _ptr, _i64, _ptr, _i64, _i64, _i64, _i64, _i64, _ptr]),
    "pa_check_tables": (_int, [_ptr, _i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _ptr]),
}

# Entry points a decode step calls once or more per layer: bound through pa_fastcall (a small CPython
# module, csrc/fastcall) when it has been built, because ctypes spends 3-5 us converting their 10-35
# arguments and the module 0.3 us.  Their callers pass addresses and sizes as plain ints, None for a
# null pointer and floats for floats, which is all the module accepts; every other entry, and every
# entry when the module is missing, goes through ctypes.
FAST_ENTRIES = ("pa_decode", "pa_decode_shared_prefix", "pa_qk_norm_rope_store", "pa_add_rms_norm", "pa_silu_mul",
                "pa_kv_store", "pa_kv_store_fp8", "pa_prefill", "pa_sample")
_KIND = {_ptr: "p", _i64: "q", _int: "i", _f32: "f"}


class _Library:
    """The loaded library.  Attributes are its entry points: ctypes functions, or pa_fastcall bindings of
    the same addresses with the same arguments and return values."""

    def __init__(self, cdll, fast):
        self._cdll = cdll
        self.fast_entries = tuple(sorted(fast))
        for name in SIGNATURES:
            setattr(self, name, fast.get(name) or getattr(cdll, name))

    def __getattr__(self, name):          # entry points outside SIGNATURES (none today) and dunder lookups
        return getattr(self._cdll, name)


def _fast_bindings(cdll):
    try:
        from . import pa_fastcall
    except ImportError:
        return {}
    import functools
    fast = {}
    for name in FAST_ENTRIES:
        restype, argtypes = SIGNATURES[name]
        addr = ctypes.cast(getattr(cdll, name), ctypes.c_void_p).value
        index = pa_fastcall.bind(addr, "".join(_KIND[t] for t in argtypes), restype is _i64)
        fast[name] = functools.partial(pa_fastcall.call, index)
    return fast


_lock = threading.Lock()
_lib = None


def is_built():
    return os.path.exists(LIB_PATH)


def load():
    """Load the library once and attach the prototypes. Raises RuntimeError if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libpaged_attn.so is not built (%s). Build it with "
                "`python ai-infra-train-infer_amd/build.py`; this package has no fallback path."
                % LIB_PATH)
        # torch ships its own HIP runtime with the same soname; importing it first makes the
        # library bind to the runtime that owns torch's streams and allocations.
        import torch  # noqa: F401
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = _Library(lib, _fast_bindings(lib))
    return _lib


def last_error():
    msg = load().pa_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(rc, what):
    """Turn a non-zero C return code into RuntimeError carrying pa_last_error()."""
    if rc != PA_OK:
        raise RuntimeError("%s failed (code %d): %s" % (what, rc, last_error()))
