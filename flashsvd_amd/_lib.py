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


class ExpandDesc(ctypes.Structure):
    """fsvd_expand_desc: one head expansion of a batched call (fsvd_lowrank_expand_heads_multi)."""
    _fields_ = [("p", c_void_p), ("sp_b", c_int64), ("sp_m", c_int64), ("sp_h", c_int64),
                ("u", c_void_p), ("ldu", c_int64), ("bias", c_void_p),
                ("y", c_void_p), ("sy_b", c_int64), ("sy_m", c_int64), ("sy_h", c_int64),
                ("heads", ctypes.c_int32), ("R", ctypes.c_int32), ("rotate", ctypes.c_int32),
                ("dst_by_position", ctypes.c_int32), ("dst_rows", ctypes.c_int32), ("rsv0", ctypes.c_int32)]


class TagBuf(ctypes.Structure):
    """fsvd_tagbuf: a tagged hand-off vector and which of its per-step uses a phase touches."""
    _fields_ = [("ptr", c_void_p), ("uses_per_step", ctypes.c_int32), ("use", ctypes.c_int32)]


class _PhaseU1(ctypes.Union):
    _fields_ = [("nsplit", ctypes.c_int32), ("rows0", ctypes.c_int32)]


class _PhaseU2(ctypes.Union):
    _fields_ = [("rope_len", ctypes.c_int32), ("in_off", ctypes.c_int32)]


class _PhaseU3(ctypes.Union):
    _fields_ = [("S", ctypes.c_int32), ("in2_len", ctypes.c_int32)]


class _PhaseAttnPtrs(ctypes.Structure):
    _fields_ = [("cos", c_void_p), ("sin", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p)]


class _PhaseGemvBufs(ctypes.Structure):
    _fields_ = [("aux2", TagBuf), ("out1", TagBuf)]


class _PhaseU4(ctypes.Union):
    _anonymous_ = ("attn_ptrs", "gemv_bufs")
    _fields_ = [("attn_ptrs", _PhaseAttnPtrs), ("gemv_bufs", _PhaseGemvBufs)]


class _PhaseU5(ctypes.Union):
    _fields_ = [("sc_s", c_int64), ("in2_off", ctypes.c_int32)]


class Phase(ctypes.Structure):
    """fsvd_phase (include/flashsvd_hip.h), field for field; the unions overlay the fields of an attention phase with
    those of a GEMV phase."""
    _anonymous_ = ("u1", "u2", "u3", "u4", "u5")
    _fields_ = [("type", ctypes.c_int32), ("epilogue", ctypes.c_int32),
                ("N", ctypes.c_int32), ("K", ctypes.c_int32), ("nmat", ctypes.c_int32), ("mode", ctypes.c_int32),
                ("H", ctypes.c_int32), ("Hk", ctypes.c_int32), ("Dh", ctypes.c_int32), ("u1", _PhaseU1),
                ("u2", _PhaseU2), ("u3", _PhaseU3),
                ("fparam", c_float), ("flags", ctypes.c_int32),
                ("W", c_void_p * 3), ("norm_w", c_void_p), ("u4", _PhaseU4),
                ("u5", _PhaseU5), ("sc_h", c_int64),
                ("plain_out", c_void_p),
                ("inp", TagBuf), ("aux0", TagBuf), ("in2", TagBuf), ("out0", TagBuf),
                ("qsz", c_void_p * 2), ("ldg", ctypes.c_int32), ("gshift", ctypes.c_int32), ("wbits", ctypes.c_int32),
                ("shared_in", ctypes.c_int32),
                ("share_q", ctypes.c_int32), ("share_r", ctypes.c_int32), ("m_kp", ctypes.c_uint32), ("dk", ctypes.c_int32)]


assert ctypes.sizeof(Phase) == 256, "fsvd_phase is 64 words: the kernel carries a descriptor in one register per lane"


class StepState(ctypes.Structure):
    """fsvd_step_state."""
    _fields_ = [("epoch", ctypes.c_int32), ("err", ctypes.c_int32), ("pos", ctypes.c_int32), ("step", ctypes.c_int32),
                ("token", c_int64), ("err_wg", ctypes.c_int32), ("spin_limit", ctypes.c_int32)]


PH_EMBED, PH_GEMV, _PH_RESERVED, PH_ATTN, PH_MERGE, PH_ARGMAX = range(6)
EP_STORE, EP_RESID, EP_SWIGLU, EP_LOGITS, EP_F32 = range(5)
PF_NOWAIT, PF_STAGE2, PF_SPLIT, PF_LEAD = 1, 2, 4, 8
WBITS_FP16 = -16
WBITS_Q4_FP16 = -4

# name -> (restype, argtypes); mirrors include/flashsvd_hip.h declaration by declaration
SIGNATURES = {
    "fsvd_version": (c_int, []),
    "fsvd_last_error": (c_char_p, []),
    "fsvd_linear": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_float, c_void_p, c_int64,
                            c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_linear_rankkv_append": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_float, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int, c_int, c_void_p]),
    "fsvd_swiglu_linear": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
                                   c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_linear_q4": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p,
                               c_float, c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_dequant_q4": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "fsvd_swiglu_linear_q4": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int64, c_int64, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_qkv_rope_append": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                     c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int64, c_int64, c_int64,
                                     c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_attn_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "fsvd_attn_decode_densekv": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                         c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int,
                                         c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64,
                                         c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "fsvd_attn_decode_densekv_static_max_bytes": (c_size_t, []),
    "fsvd_attn_decode_densekv_static": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                                c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int,
                                                c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64,
                                                c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "fsvd_rmsnorm": (c_int, [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "fsvd_attn_decode_rankkv": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64,
                                        c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                        c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                        c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_int, c_void_p]),
    "fsvd_attn_decode_rankkv_scores_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "fsvd_rankkv_append": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p,
                                   c_int, c_int, c_int, c_int, c_void_p]),
    "fsvd_lowrank_expand_heads": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int,
                                          c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_int, c_void_p]),
    "fsvd_lowrank_expand_heads_multi": (c_int, [ctypes.POINTER(ExpandDesc), c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                                                c_int, c_void_p]),
    "fsvd_attn_prefill": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                  c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64,
                                  c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "fsvd_xw_linear_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "fsvd_xw_linear": (c_int, [c_void_p, c_int64, c_int64, c_int, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_int64, c_int,
                               c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "fsvd_reconstruct_qkv_workspace_bytes": (c_size_t, [c_int] * 8),
    "fsvd_reconstruct_qkv_token": (c_int, [c_void_p, c_int64, c_int64, c_int64] * 3 + [c_void_p, c_int64, c_int64] * 3
                                   + [c_void_p, c_int64] * 3 + [c_void_p, c_int64, c_int64] * 3 + [c_int] * 8
                                   + [c_void_p, c_size_t, c_void_p]),
    "fsvd_mlp_dual_split_workspace_bytes": (c_size_t, [c_int] * 6),
    "fsvd_decode_step_workgroups": (c_int, []),
    "fsvd_decode_step_prepare": (c_int, [c_void_p, c_int, c_int]),
    "fsvd_decode_step_validate": (c_int, [c_void_p, c_int, c_int]),
    "fsvd_set_workspace": (c_int, [c_void_p, c_size_t, c_void_p]),
    "fsvd_decode_step": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "fsvd_decode_step_trace": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
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
