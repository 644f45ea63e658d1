"""Dual-split low-rank SwiGLU MLP for decode, on the reference's operand layouts.

Function names, signatures, tile-override environment variables and error messages follow
kernels/mlp/decode/dual_split_triton.py (:10-129 config pickers, :535-983 wrappers) and
kernels/mlp/decode/dual_split_triton_pcat_s.py (:123-218).  Every variant runs the same three HIP
launches (gate/up product + SwiGLU, D-tiled product with DownV, product with DownU); the variants
differ only in where intermediate results are rounded, which the library reproduces.  Tile sizes
other than BD (the D-tile of the partial sums) do not change results and are ignored."""
from __future__ import annotations

import os
from typing import Optional

import torch

from .. import _lib
from ..torch_ops import ops as _OPS
from ._common import check, dtype_code, scratch, stream


def _env_overrides(cfg: dict, prefix: str, keys) -> dict:
    for key in keys:
        raw = os.getenv(f"{prefix}_{'WARPS' if key == 'warps' else 'STAGES' if key == 'stages' else key}", "").strip()
        if not raw:
            continue
        try:
            val = int(raw)
        except ValueError:
            continue
        if val > 0:
            cfg[key] = val
    return cfg


def _pick_dual_split_token_config(R: int, D: int) -> dict:
    if max(R, D) >= 8192 or R >= 1024:
        cfg = {"BR": 128, "BD": 128, "BR2": 256, "warps": 8, "stages": 2}
    elif R >= 512:
        cfg = {"BR": 64, "BD": 128, "BR2": 128, "warps": 4, "stages": 2}
    else:
        cfg = {"BR": 64, "BD": 128, "BR2": 256, "warps": 4, "stages": 2}
    return _env_overrides(cfg, "FLASH_SVD_DUAL_SPLIT", ("BR", "BD", "BR2", "warps", "stages"))


def _pick_dual_split_token_v2_config(R: int, D: int) -> dict:
    if max(R, D) >= 8192 or R >= 1024:
        cfg = {"BR": 128, "BD": 128, "BR2": 128, "warps": 8, "stages": 2}
    else:
        cfg = {"BR": 64, "BD": 128, "BR2": 128, "warps": 4, "stages": 2}
    return _env_overrides(cfg, "FLASH_SVD_DUAL_SPLIT_V2", ("BR", "BD", "BR2", "warps", "stages"))


def _pick_dual_split_token_v2_sm80_config(R: int, D: int, *, is_sm80: bool = False) -> dict:
    if max(R, D) >= 8192 or R >= 1024:
        cfg = {"BR": 128, "BD": 64, "BR2": 128, "GD": 2, "warps": 8, "stages": 2 if is_sm80 else 1}
    elif R >= 512:
        cfg = {"BR": 64, "BD": 64, "BR2": 128, "GD": 2, "warps": 8 if is_sm80 else 4, "stages": 2}
    else:
        cfg = {"BR": 64, "BD": 128, "BR2": 128, "GD": 1, "warps": 4, "stages": 2}
    return _env_overrides(cfg, "FLASH_SVD_DUAL_SPLIT_V2_SM80", ("BR", "BD", "BR2", "GD", "warps", "stages"))


def _pick_dual_split_token_v3_config(R: int, D: int, H: int) -> dict:
    if max(R, D, H) >= 8192 or max(R, H) >= 1024:
        cfg = {"BR": 128, "BD": 128, "BR2": 128, "BH": 128, "GH": 4, "warps": 8, "stages": 2}
    else:
        cfg = {"BR": 64, "BD": 128, "BR2": 128, "BH": 128, "GH": 2, "warps": 4, "stages": 2}
    return _env_overrides(cfg, "FLASH_SVD_DUAL_SPLIT_V3", ("BR", "BD", "BR2", "BH", "GH", "warps", "stages"))


def _pick_dual_split_pcat_s_config(R: int, D: int) -> dict:
    cfg = {"BT": 16, "BR": 64, "BD": 128, "BR2": 128, "warps": 4, "stages": 2}
    return _env_overrides(cfg, "FLASH_SVD_DUAL_SPLIT_PCAT_S", ("BT", "BR", "BD", "BR2", "warps", "stages"))


def _check_operands(R: int, GateU, UpU, DownV, DownU):
    if GateU.shape[0] != R:
        raise ValueError(f"GateU must be [R, D] with R={R}, got {tuple(GateU.shape)}")
    if UpU.shape != GateU.shape:
        raise ValueError(f"UpU shape {tuple(UpU.shape)} must match GateU shape {tuple(GateU.shape)}")
    D = int(GateU.shape[1])
    if tuple(DownV.shape) != (D, R):
        raise ValueError(f"DownV must be [D, R]=[{D}, {R}], got {tuple(DownV.shape)}")
    if DownU.ndim != 2 or DownU.shape[0] != R:
        raise ValueError(f"DownU must be [R, H] with R={R}, got {tuple(DownU.shape)}")
    return D, int(DownU.shape[1])


def _check_workspace(ws, shape, device, name):
    if ws is None:
        return
    if tuple(ws.shape) != tuple(shape):
        raise ValueError(f"{name} must be {tuple(shape)}, got {tuple(ws.shape)}")
    if ws.device != device:
        raise ValueError(f"{name} must be on the same device as inputs")
    if ws.dtype != torch.float32:
        raise ValueError(f"{name} must have dtype float32")


def _run(p_up_2d, p_gate_2d, GateU, UpU, DownV, DownU, b2, *, variant: int, BD: int, partials_fp32: bool = True,
         s_out: Optional[torch.Tensor] = None):
    """Custom operator flashsvd_hip::mlp_dual_split on [T, R] coefficient rows."""
    return _OPS.mlp_dual_split.default(p_up_2d, p_gate_2d, GateU, UpU, DownV, DownU, b2, int(variant), int(BD), bool(partials_fp32), s_out)


def _fast_path_ok(p_up_2d, p_gate_2d, GateU, UpU, DownV, DownU, variant, partials_fp32, s_out) -> bool:
    """bf16 or fp16, fp32 partial sums rounded once (v2 / v2_sm80 / pcat_s, and v1 with fp32 partials), no caller workspace:
    the arithmetic of three product-path launches on nn.Linear-layout twins of the operands."""
    if os.getenv("FLASHSVD_AMD_REFERENCE_LAYOUT_FAST", "1") == "0":
        return False
    if s_out is not None or not (variant == 2 or (variant == 1 and partials_fp32)):
        return False
    if p_up_2d.dtype not in (torch.bfloat16, torch.float16) or any(t.dtype != p_up_2d.dtype for t in (p_gate_2d, GateU, UpU, DownV, DownU)):
        return False
    R, D, Hd = p_up_2d.shape[1], GateU.shape[1], DownU.shape[1]
    return p_up_2d.stride(1) == 1 and p_gate_2d.stride(1) == 1 and R % 8 == 0 and D % 8 == 0 and Hd % 8 == 0


def _run_fast(p_up_2d, p_gate_2d, GateU, UpU, DownV, DownU, b2):
    from .. import hip_ops
    from ._common import linear_layout_of
    T, R = p_up_2d.shape
    # the coefficient rows as one [T, 2R] buffer [PGate | PUp]: adjacent views of such a packed tensor are used in place,
    # anything else (separate tensors, the [PUp | PGate] order of the pcat_s variant) is packed by one small copy
    if p_up_2d.data_ptr() == p_gate_2d.data_ptr() + R * 2 and p_up_2d.stride(0) == p_gate_2d.stride(0) >= 2 * R:
        p = p_gate_2d.as_strided((T, 2 * R), (p_gate_2d.stride(0), 1))
    else:
        p = torch.cat([p_gate_2d, p_up_2d], dim=1)
    gate_u, up_u = linear_layout_of(GateU), linear_layout_of(UpU)          # [D, R]
    h = hip_ops.swiglu_linear(p, gate_u, up_u, up_off=R, mode=1)           # h = round(silu(g32) * u32), dual_split_triton.py:207
    s = hip_ops.linear(h, linear_layout_of(DownV))                        # S: fp32 sum over D, one rounding (:719-720)
    return hip_ops.linear(s, linear_layout_of(DownU), None if b2 is None else b2.to(s.dtype).contiguous())


def _run_impl(p_up_2d, p_gate_2d, GateU, UpU, DownV, DownU, b2, variant, BD, partials_fp32, s_out):
    if _fast_path_ok(p_up_2d, p_gate_2d, GateU, UpU, DownV, DownU, variant, partials_fp32, s_out):
        return _run_fast(p_up_2d, p_gate_2d, GateU, UpU, DownV, DownU, b2)
    T, R = p_up_2d.shape
    D, Hd = int(GateU.shape[1]), int(DownU.shape[1])
    dt = dtype_code(p_up_2d)
    gate_u, up_u, down_v, down_u = GateU.contiguous(), UpU.contiguous(), DownV.contiguous(), DownU.contiguous()
    for t, nm in ((gate_u, "GateU"), (up_u, "UpU"), (down_v, "DownV"), (down_u, "DownU")):
        if t.dtype != p_up_2d.dtype:
            raise ValueError(f"{nm} has dtype {t.dtype}, expected {p_up_2d.dtype}")
    if b2 is not None:
        b2 = b2.to(p_up_2d.dtype).contiguous()
    y = torch.empty((T, Hd), device=p_up_2d.device, dtype=p_up_2d.dtype)
    lib = _lib.load()
    ws = scratch(p_up_2d.device, lib.fsvd_mlp_dual_split_workspace_bytes(T, R, D, Hd, dt, int(BD)), "dual_split")
    rc = lib.fsvd_mlp_dual_split(p_up_2d.data_ptr(), p_up_2d.stride(0), p_gate_2d.data_ptr(), p_gate_2d.stride(0),
                                 gate_u.data_ptr(), gate_u.stride(0), up_u.data_ptr(), up_u.stride(0),
                                 down_v.data_ptr(), down_v.stride(0), down_u.data_ptr(), down_u.stride(0),
                                 None if b2 is None else b2.data_ptr(), y.data_ptr(), y.stride(0),
                                 None if s_out is None else s_out.data_ptr(), T, R, D, Hd, dt, int(variant), int(BD),
                                 int(bool(partials_fp32)), ws.data_ptr(), ws.numel() * 4, stream())
    check("fsvd_mlp_dual_split", rc)
    return y


def _prep(PUp, PGate):
    if PUp.ndim != 3 or PGate.ndim != 3:
        raise ValueError(f"PUp/PGate must be [B, L, R], got {tuple(PUp.shape)} and {tuple(PGate.shape)}")
    if PUp.shape != PGate.shape:
        raise ValueError(f"PUp and PGate shapes must match, got {tuple(PUp.shape)} and {tuple(PGate.shape)}")
    B, L, R = PUp.shape
    T = int(B * L)
    return B, L, R, T, PUp.contiguous().reshape(T, R), PGate.contiguous().reshape(T, R)


def flashsvd_mlp_dual_split_triton_v1(PUp, PGate, GateU, UpU, DownV, DownU, b2=None, *, BR=None, BD=None, BR2=None,
                                      num_warps=None, num_stages=None, store_partials_fp32: bool = False):
    """Per-D-tile partials of h @ DownV pass through a workspace (input dtype unless
    store_partials_fp32) and are summed; Y = S @ DownU (+ b2)."""
    assert PUp.is_cuda and PGate.is_cuda and GateU.is_cuda and UpU.is_cuda and DownV.is_cuda and DownU.is_cuda
    B, L, R, T, pu, pg = _prep(PUp, PGate)
    _check_operands(R, GateU, UpU, DownV, DownU)
    cfg = _pick_dual_split_token_config(R, int(GateU.shape[1]))
    y = _run(pu, pg, GateU, UpU, DownV, DownU, b2, variant=1, BD=cfg["BD"] if BD is None else BD,
             partials_fp32=bool(store_partials_fp32))
    return y.reshape(B, L, DownU.shape[1])


def flashsvd_mlp_dual_split_triton_v2(PUp, PGate, GateU, UpU, DownV, DownU, b2=None, *, BR=None, BD=None, BR2=None,
                                      num_warps=None, num_stages=None, workspace_s2d: Optional[torch.Tensor] = None):
    """fp32 S accumulated over the D tiles (in tile order), rounded to the input dtype, then
    Y = S @ DownU (+ b2).  ``workspace_s2d`` (fp32 [T,R]) receives S."""
    assert PUp.is_cuda and PGate.is_cuda and GateU.is_cuda and UpU.is_cuda and DownV.is_cuda and DownU.is_cuda
    B, L, R, T, pu, pg = _prep(PUp, PGate)
    _check_operands(R, GateU, UpU, DownV, DownU)
    _check_workspace(workspace_s2d, (T, R), PUp.device, "workspace_s2d")
    cfg = _pick_dual_split_token_v2_config(R, int(GateU.shape[1]))
    y = _run(pu, pg, GateU, UpU, DownV, DownU, b2, variant=2, BD=cfg["BD"] if BD is None else BD, s_out=workspace_s2d)
    return y.reshape(B, L, DownU.shape[1])


def flashsvd_mlp_dual_split_triton_v2_sm80(PUp, PGate, GateU, UpU, DownV, DownU, b2=None, *, BR=None, BD=None, BR2=None,
                                           num_warps=None, num_stages=None, workspace_s2d: Optional[torch.Tensor] = None,
                                           GD=None):
    """Same arithmetic as v2 (the reference variant only regroups D tiles per program)."""
    assert PUp.is_cuda and PGate.is_cuda and GateU.is_cuda and UpU.is_cuda and DownV.is_cuda and DownU.is_cuda
    B, L, R, T, pu, pg = _prep(PUp, PGate)
    _check_operands(R, GateU, UpU, DownV, DownU)
    _check_workspace(workspace_s2d, (T, R), PUp.device, "workspace_s2d")
    cfg = _pick_dual_split_token_v2_sm80_config(R, int(GateU.shape[1]))
    y = _run(pu, pg, GateU, UpU, DownV, DownU, b2, variant=2, BD=cfg["BD"] if BD is None else BD, s_out=workspace_s2d)
    return y.reshape(B, L, DownU.shape[1])


def flashsvd_mlp_dual_split_triton_v3(PUp, PGate, GateU, UpU, DownV, DownU, b2=None, *, BR=None, BD=None, BR2=None,
                                      BH=None, GH=None, num_warps=None, num_stages=None,
                                      workspace_y: Optional[torch.Tensor] = None):
    """DownU fused: per-tile s = h @ DownV rounded to the input dtype, Y accumulated in fp32 from
    the rounded tiles and rounded once; b2 added afterwards.  ``workspace_y`` is validated only
    (the deterministic reduction needs no caller accumulator)."""
    assert PUp.is_cuda and PGate.is_cuda and GateU.is_cuda and UpU.is_cuda and DownV.is_cuda and DownU.is_cuda
    B, L, R, T, pu, pg = _prep(PUp, PGate)
    _, Hd = _check_operands(R, GateU, UpU, DownV, DownU)
    _check_workspace(workspace_y, (T, Hd), PUp.device, "workspace_y")
    cfg = _pick_dual_split_token_v3_config(R, int(GateU.shape[1]), Hd)
    y = _run(pu, pg, GateU, UpU, DownV, DownU, b2, variant=3, BD=cfg["BD"] if BD is None else BD)
    return y.reshape(B, L, Hd)


def flashsvd_mlp_dual_split_triton_pcat_s(PCat, GateU, UpU, DownV, DownU, b2=None, *, BT=None, BR=None, BD=None, BR2=None,
                                          num_warps=None, num_stages=None, workspace_s2d: Optional[torch.Tensor] = None):
    """Packed input PCat [B,L,2R] with PCat[..., :R] = PUp and PCat[..., R:] = PGate; v2 arithmetic."""
    assert PCat.is_cuda and GateU.is_cuda and UpU.is_cuda and DownV.is_cuda and DownU.is_cuda
    if PCat.ndim != 3:
        raise ValueError(f"PCat must be [B, L, 2R], got {tuple(PCat.shape)}")
    B, L, two_r = PCat.shape
    if two_r % 2 != 0:
        raise ValueError(f"PCat last dim must be even, got {two_r}")
    R = int(two_r // 2)
    _check_operands(R, GateU, UpU, DownV, DownU)
    T = int(B * L)
    _check_workspace(workspace_s2d, (T, R), PCat.device, "workspace_s2d")
    p2 = PCat.contiguous().reshape(T, 2 * R)
    cfg = _pick_dual_split_pcat_s_config(R, int(GateU.shape[1]))
    y = _run(p2[:, :R], p2[:, R:], GateU, UpU, DownV, DownU, b2, variant=2, BD=cfg["BD"] if BD is None else BD,
             s_out=workspace_s2d)
    return y.reshape(B, L, DownU.shape[1])


flashsvd_ffn_dual_split_token = flashsvd_mlp_dual_split_triton_v1
flashsvd_ffn_dual_split_token_v2 = flashsvd_mlp_dual_split_triton_v2
flashsvd_ffn_dual_split_token_v2_sm80 = flashsvd_mlp_dual_split_triton_v2_sm80
flashsvd_ffn_dual_split_token_v3 = flashsvd_mlp_dual_split_triton_v3

__all__ = [
    "flashsvd_mlp_dual_split_triton_v1", "flashsvd_mlp_dual_split_triton_v2", "flashsvd_mlp_dual_split_triton_v2_sm80",
    "flashsvd_mlp_dual_split_triton_v3", "flashsvd_mlp_dual_split_triton_pcat_s",
    "flashsvd_ffn_dual_split_token", "flashsvd_ffn_dual_split_token_v2", "flashsvd_ffn_dual_split_token_v2_sm80",
    "flashsvd_ffn_dual_split_token_v3",
]
