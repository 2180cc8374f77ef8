"""ctypes binding of libuniql_amd.so (the C ABI declared in include/uniql_amd.h and, for the
test hooks and measurement aids, include/uniql_amd_diag.h).

There is no fallback: if the library is missing or cannot be loaded every
operator raises.  The library is built by `python -m uniql_amd.build`.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint, c_void_p

from .build import LIB_PATH

OK = 0
F_OUT_F32 = 1 << 0
F_FORCE_SKINNY = 1 << 1
F_FORCE_TILED = 1 << 2
F_TRANSPOSE_OUT = 1 << 3
F_SEPARATE_ROTATION = 1 << 4
DT_F16, DT_BF16, DT_F32 = 0, 1, 2
EPI_NONE, EPI_SILU_MUL, EPI_RELU2 = 0, 1, 2

# every exported symbol with (restype, argtypes); tests check the list against the header
SIGNATURES = {
    "uniql_abi_version": (c_int, []),
    "uniql_status_string": (c_char_p, [c_int]),
    "uniql_stream_capture_id": (c_int, [c_void_p, ctypes.POINTER(ctypes.c_ulonglong)]),
    "uniql_clear": (c_int, [c_void_p, c_size_t, c_void_p]),
    "uniql_diag_mfma_loop": (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    "uniql_w4a16_gemm_accum_bytes": (c_size_t, [c_int, c_int, c_int]),
    "uniql_w4a16_gemm_temp_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "uniql_w4a16_gemm": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_int64, c_void_p, c_size_t, c_void_p, c_size_t,
                                 c_int, c_int, c_int, c_int, c_int, c_float, c_uint, c_void_p]),
    "uniql_w4a16_gemm_static_limit": (c_size_t, [c_int]),
    "uniql_w4a16_gemm_static": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                        c_int, c_int, c_int, c_int, c_int, c_float, c_uint, c_void_p]),
    "uniql_w4a16_linear_temp_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "uniql_w4a16_linear_workspace": (c_int, [c_int, c_int, c_int, c_int, c_int, c_uint,
                                             ctypes.POINTER(c_size_t), ctypes.POINTER(c_size_t)]),
    "uniql_w4a16_linear": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_int64, c_void_p, c_int64, c_int, c_int,
                                   c_void_p, c_int64, c_void_p, c_size_t, c_void_p, c_size_t,
                                   c_int, c_int, c_int, c_int, c_int, c_float, c_uint, c_void_p]),
    "uniql_w4a16_read_floor_sink_bytes": (c_size_t, [c_int, c_int, c_int, c_uint]),
    "uniql_w4a16_read_floor": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_uint, c_void_p]),
    "uniql_w4a16_dequant": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "uniql_w4a16_quantize": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                     c_int, c_int, c_int, c_int, c_void_p]),
    "uniql_w4a16_pack": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "uniql_w4_embedding_lookup": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                          c_int64, c_int, c_void_p]),
    "uniql_w4_embedding_quantize": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "uniql_rope_indices": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                   c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "uniql_fwht": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_float, c_int, c_void_p]),
    "uniql_fwht_composite": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_float, c_int, c_void_p]),
}

_lib = None


class UniqlLibraryError(RuntimeError):
    pass


def library_path() -> str:
    return os.environ.get("UNIQL_AMD_LIB", LIB_PATH)


def load():
    """Loads the shared library once.  torch must already be imported so that the
    HIP runtime it ships is the one the kernels register with."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (brings libamdhip64 into the process first)
    path = library_path()
    if not os.path.exists(path):
        raise UniqlLibraryError(
            f"{path} not found: build it with `python -m uniql_amd.build` (there is no CPU fallback)")
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != OK:
        msg = load().uniql_status_string(code).decode()
        raise RuntimeError(f"{what}: {msg} (code {code})")
