"""ctypes binding of libflashsvd_hip.so (the C ABI declared in include/flashsvd_hip.h).

The library is the only compute path of this package: if it is missing or fails to load,
``load()`` raises — there is no PyTorch or CPU fallback behind it.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libflashsvd_hip.so"

_lib = None

_i32p = ctypes.POINTER(ctypes.c_int32)

# name -> (restype, argtypes); mirrors include/flashsvd_hip.h declaration by declaration
SIGNATURES = {
    "fsvd_version": (c_int, []),
    "fsvd_last_error": (c_char_p, []),
    "fsvd_linear": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_float, c_void_p, c_int64,
                            c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_swiglu_linear": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
                                   c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_qkv_rope_append": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                     c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int64, c_int64, c_int64,
                                     c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_attn_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "fsvd_attn_decode_densekv": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                         c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int,
                                         c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64,
                                         c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p]),
    "fsvd_rmsnorm": (c_int, [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "fsvd_attn_decode_rankkv": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64,
                                        c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                        c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                        c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p]),
    "fsvd_lowrank_expand_heads": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int,
                                          c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p]),
    "fsvd_attn_prefill": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                  c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64,
                                  c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p]),
    "fsvd_xw_linear_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "fsvd_xw_linear": (c_int, [c_void_p, c_int64, c_int64, c_int, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_int64, c_int,
                               c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "fsvd_reconstruct_qkv_workspace_bytes": (c_size_t, [c_int] * 8),
    "fsvd_reconstruct_qkv_token": (c_int, [c_void_p, c_int64, c_int64, c_int64] * 3 + [c_void_p, c_int64, c_int64] * 3
                                   + [c_void_p, c_int64] * 3 + [c_void_p, c_int64, c_int64] * 3 + [c_int] * 8
                                   + [c_void_p, c_size_t, c_void_p]),
    "fsvd_mlp_dual_split_workspace_bytes": (c_size_t, [c_int] * 6),
    "fsvd_mlp_dual_split": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                    c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
}


class FlashSVDHipError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, fn: str, code: int, message: str):
        super().__init__(f"{fn} failed with status {code}: {message}")
        self.code = code
        self.detail = message


def load():
    """Load the shared library once and attach argument types; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m flashsvd_amd._build` "
            "(hipcc --offload-arch=gfx950). flashsvd_amd has no fallback path.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(fn_name: str, code: int) -> None:
    if code != 0:
        msg = load().fsvd_last_error()
        raise FlashSVDHipError(fn_name, code, msg.decode() if msg else "")
