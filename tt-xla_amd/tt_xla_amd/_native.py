"""ctypes binding of libttpa.so (the C ABI declared in include/ttpa.h)."""

from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libttpa.so")
CSRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "csrc"))

OK = 0
ERR_INVALID_ARGUMENT = -1
ERR_UNSUPPORTED = -2
ERR_WORKSPACE = -3
ERR_LAUNCH = -4

KV_BF16 = 0
KV_BFP8 = 1

_p, _i64, _i32, _int, _f32, _sz = C.c_void_p, C.c_int64, C.c_int32, C.c_int, C.c_float, C.c_size_t

# name -> (restype, argtypes); must list every symbol include/ttpa.h declares
SIGNATURES = {
    "ttpa_abi_version": (_int, []),
    "ttpa_last_error": (C.c_char_p, []),
    "ttpa_device_compute_units": (_int, []),
    "ttpa_profile_next_attention": (_int, [_p, _p]),
    "ttpa_paged_update_cache": (
        _int,
        [_p, _p, _i64, _i64, _p, _int, _p, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _p],
    ),
    "ttpa_paged_update_cache_kv": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _p, _int, _p, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _p],
    ),
    "ttpa_paged_fill_cache": (
        _int,
        [_p, _p, _i64, _i64, _i64, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _i32, _i32, _i32,
         _i32, _i32, _p],
    ),
    "ttpa_paged_fill_cache_kv": (
        _int,
        [_p, _p, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _i32, _i32,
         _i32, _i32, _i32, _p],
    ),
    "ttpa_paged_decode_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32]),
    "ttpa_paged_sdpa_decode": (
        _int,
        [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _i32,
         _i32, _i32, _f32, _i32, _p, _sz, _p],
    ),
    "ttpa_paged_sdpa_decode_windowed": (
        _int,
        [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _i32,
         _i32, _i32, _f32, _i32, _i32, _p, _p, _sz, _p],
    ),
    "ttpa_paged_sdpa_decode_masked": (
        _int,
        [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _i32,
         _i32, _i32, _f32, _i32, _p, _i64, _i64, _p, _sz, _p],
    ),
    "ttpa_paged_update_decode": (
        _int,
        [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _p, _i64, _p, _int, _i32, _i32,
         _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _p, _p, _sz, _p],
    ),
    "ttpa_static_scratch_bytes": (_sz, []),
    "ttpa_static_scratch_init": (_int, []),
    "ttpa_paged_update_decode_static": (
        _int,
        [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _p, _i64, _p, _int, _i32, _i32,
         _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _p, _p],
    ),
    "ttpa_paged_mla_decode_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32]),
    "ttpa_paged_mla_decode": (
        _int,
        [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _i32,
         _i32, _i32, _i32, _f32, _p, _p, _sz, _p],
    ),
    "ttpa_paged_mla_decode_masked": (
        _int,
        [_p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _i32,
         _i32, _i32, _i32, _f32, _p, _i64, _i64, _p, _sz, _p],
    ),
    "ttpa_sdpa_prefill": (
        _int,
        [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _p,
         _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _p],
    ),
    "ttpa_sdpa_prefill_windowed": (
        _int,
        [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _p,
         _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _p],
    ),
    "ttpa_sdpa_prefill_format": (
        _int,
        [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _p,
         _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _p],
    ),
    "ttpa_sdpa_prefill_expanded": (
        _int,
        [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _p,
         _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _p, _i64, _p],
    ),
    "ttpa_sdpa_prefill_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32, _i32, _i32]),
    "ttpa_latent_prefill": (
        _int,
        [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i64, _i64,
         _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _p],
    ),
    "ttpa_sdpa_prefill_fill": (
        _int,
        [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64,
         _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32,
         _p, _p, _p, _i64, _p, _int, _i32, _i32, _i32, _i32, _p],
    ),
    "ttpa_bfp8_quantize": (_int, [_p, _p, _p, _i64, _p]),
    "ttpa_bfp8_dequantize": (_int, [_p, _p, _p, _i64, _p]),
}


class TtpaError(RuntimeError):
    """A libttpa call returned a negative status."""

    def __init__(self, fn: str, code: int, message: str):
        super().__init__(f"{fn} failed ({code}): {message}")
        self.code = code


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    """Loads the library once.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing; build it with `make -C {CSRC_DIR}` "
                "(hipcc, --offload-arch=gfx950)"
            )
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.ttpa_abi_version() != 1:
            raise RuntimeError("libttpa.so ABI version mismatch; rebuild it")
        _lib = handle
    return _lib


def call(name: str, *args) -> None:
    """Invokes a status-returning entry point and raises TtpaError on failure."""
    handle = lib()
    rc = getattr(handle, name)(*args)
    if rc != OK:
        raise TtpaError(name, rc, handle.ttpa_last_error().decode("utf-8", "replace"))
