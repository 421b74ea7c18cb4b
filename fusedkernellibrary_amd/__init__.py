"""MI355X (gfx950) backend of the fused data-parallel execution path.

The product is native: `libfklhip.so` (C ABI declared in include/fklhip.h, hand-written HIP kernels) and the
C++20 host headers under include/fused_kernel/.  This Python package only locates and loads the library for
tests and benchmarks (their case drivers and synthetic workloads live under tests/).  There is no CPU fallback: if the library is missing
or cannot be loaded, importing `lib()` raises.
"""
from __future__ import annotations

import ctypes as _C
import os as _os

PKG_DIR = _os.path.dirname(_os.path.abspath(__file__))
ROOT_DIR = _os.path.dirname(PKG_DIR)
LIB_PATH = _os.path.join(PKG_DIR, "libfklhip.so")

_lib = None

# Every symbol include/fklhip.h declares.
ABI_SYMBOLS = (
    "fklhip_abi_version", "fklhip_error_string", "fklhip_get_device", "fklhip_set_device", "fklhip_device_count",
    "fklhip_stream_create", "fklhip_stream_destroy", "fklhip_stream_sync", "fklhip_malloc", "fklhip_malloc_pitch",
    "fklhip_free", "fklhip_host_alloc", "fklhip_host_free", "fklhip_memcpy_async", "fklhip_memcpy2d_async",
    "fklhip_memset_async", "fklhip_event_create", "fklhip_event_destroy", "fklhip_event_record", "fklhip_event_sync",
    "fklhip_event_elapsed_ms", "fklhip_lookup", "fklhip_launch_handle", "fklhip_launch", "fklhip_last_launch",
    "fklhip_signature_count", "fklhip_signature_at", "fklhip_jit_log", "fklhip_strip_form",
)


def lib() -> _C.CDLL:
    """Loads libfklhip.so (built in-tree by `python -m fusedkernellibrary_amd.build`)."""
    global _lib
    if _lib is None:
        if not _os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m fusedkernellibrary_amd.build` "
                "(hipcc --offload-arch=gfx950). There is no fallback path.")
        l = _C.CDLL(LIB_PATH, mode=_C.RTLD_GLOBAL)
        l.fklhip_error_string.restype = _C.c_char_p
        l.fklhip_error_string.argtypes = [_C.c_int]
        l.fklhip_launch.argtypes = [_C.c_char_p, _C.c_void_p, _C.c_size_t, _C.c_void_p]
        l.fklhip_lookup.argtypes = [_C.c_char_p, _C.POINTER(_C.c_void_p)]
        l.fklhip_launch_handle.argtypes = [_C.c_void_p, _C.c_void_p, _C.c_size_t, _C.c_void_p]
        l.fklhip_event_create.argtypes = [_C.POINTER(_C.c_void_p)]
        l.fklhip_event_destroy.argtypes = [_C.c_void_p]
        l.fklhip_event_record.argtypes = [_C.c_void_p, _C.c_void_p]
        l.fklhip_event_sync.argtypes = [_C.c_void_p]
        l.fklhip_event_elapsed_ms.argtypes = [_C.POINTER(_C.c_float), _C.c_void_p, _C.c_void_p]
        l.fklhip_stream_create.argtypes = [_C.POINTER(_C.c_void_p)]
        l.fklhip_stream_destroy.argtypes = [_C.c_void_p]
        l.fklhip_stream_sync.argtypes = [_C.c_void_p]
        l.fklhip_last_launch.argtypes = [_C.POINTER(_C.c_char_p), _C.POINTER(_C.c_uint), _C.POINTER(_C.c_uint), _C.POINTER(_C.c_uint)]
        _lib = l
    return _lib


def check(code: int, what: str = "") -> None:
    if code != 0:
        raise RuntimeError(f"GPU Error: {lib().fklhip_error_string(code).decode()} ({what}, code {code})")


def signatures() -> list[tuple[str, int]]:
    l = lib()
    n = _C.c_int()
    check(l.fklhip_signature_count(_C.byref(n)), "signature_count")
    out = []
    for i in range(n.value):
        s = _C.c_char_p()
        b = _C.c_size_t()
        check(l.fklhip_signature_at(i, _C.byref(s), _C.byref(b)), "signature_at")
        out.append((s.value.decode(), b.value))
    return out


def last_launch() -> dict:
    k = _C.c_char_p()
    g = (_C.c_uint * 3)()
    b = (_C.c_uint * 3)()
    lds = _C.c_uint()
    lib().fklhip_last_launch(_C.byref(k), g, b, _C.byref(lds))
    return {"kernel": (k.value or b"").decode(), "grid": list(g), "block": list(b), "lds_bytes": lds.value}
