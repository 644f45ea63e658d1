"""Tensor-level wrappers over the C ABI: shape/dtype/device checks in Python, raw pointers and
the current torch stream handed to libflashsvd_hip.  PyTorch only provides device memory and
streams here; every arithmetic step runs in the HIP library."""
from __future__ import annotations

import math
import os
from typing import Optional

import torch

from . import _lib
from .torch_ops import ops as _OPS

_BF16 = torch.bfloat16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, name: str, *, dtype=_BF16) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor, got device {t.device}")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")


_ELEM_CODES = {torch.bfloat16: 0, torch.float16: 1}     # FSVD_BF16, FSVD_FP16


def _elem(t: torch.Tensor, name: str):
    """Element type of a call on the fused product path, named by its first operand: (torch dtype, C-ABI code).  Every
    other 16-bit tensor of the call must be of the same type."""
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor, got device {t.device}")
    code = _ELEM_CODES.get(t.dtype)
    if code is None:
        raise ValueError(f"{name} must be torch.bfloat16 or torch.float16, got {t.dtype}")
    return t.dtype, code


def _rows(t: torch.Tensor, name: str) -> torch.Tensor:
    """View as [rows, last] with unit stride on the last axis (copies only if it must)."""
    if t.stride(-1) != 1:
        t = t.contiguous()
    if t.dim() == 1:
        return t.unsqueeze(0)
    if t.dim() == 2:
        return t
    try:
        return t.view(-1, t.shape[-1])
    except RuntimeError:
        return t.reshape(-1, t.shape[-1])


_SPLIT_WS: dict = {}                      # device index -> scratch tensor registered with the library (kept alive here)
_SPLIT_WS_BYTES = (64 << 20) + (64 << 10)
_SPLIT_WS_OLD: dict = {}                  # device index -> replaced buffers: graphs captured earlier may hold their addresses
_SPLIT_WS_MAX = 1 << 30


def ensure_split_workspace(device: torch.device, min_bytes: int = 0) -> bool:
    """Register, once per device, the scratch the library's K-split projections (3..127 rows) work in.  The library
    allocates nothing itself; this hands it 64 MiB of torch memory, or ``min_bytes`` rounded up to a power of two (up to
    1 GiB) when a caller needs more: a larger buffer then replaces the registered one (a doubling each time at least, so
    a growing demand costs a logarithmic number of replacements), and the old one is kept alive until
    ``release_split_workspace`` because graphs captured earlier hold its address.  ``FLASHSVD_AMD_SPLITK=0`` keeps the
    library without scratch; so does a first call made under stream capture (an allocation there would belong to the
    graph's pool), and a registered buffer is never replaced under capture.  Launches that use the scratch must be
    ordered on one stream per device.  Returns whether a buffer of at least ``min_bytes`` is registered."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    need = max(int(min_bytes), _SPLIT_WS_BYTES)
    have = _SPLIT_WS.get(idx)
    if have is not None and have.numel() >= need:
        return True
    if os.environ.get("FLASHSVD_AMD_SPLITK", "1") == "0" or torch.cuda.is_current_stream_capturing() or need > _SPLIT_WS_MAX:
        return have is not None and min_bytes <= 0
    if need > _SPLIT_WS_BYTES:
        need = min(_SPLIT_WS_MAX, 1 << (need - 1).bit_length())
    with torch.cuda.device(idx):
        ws = torch.empty(need, dtype=torch.uint8, device=f"cuda:{idx}")
        rc = _lib.load().fsvd_set_workspace(ws.data_ptr(), ws.numel(), _stream())
        _lib.check("fsvd_set_workspace", rc)
        torch.cuda.current_stream().synchronize()      # cleared before any other stream can use it
    if have is not None:
        _SPLIT_WS_OLD.setdefault(idx, []).append(have)
    _SPLIT_WS[idx] = ws
    return True


def release_split_workspace(device: Optional[torch.device] = None) -> None:
    """Unregister (and free) the scratch of ``device`` and the buffers it replaced; the library runs without scratch
    until it is registered again.  Graphs captured while a buffer was registered must not be replayed afterwards."""
    idx = torch.cuda.current_device() if device is None or device.index is None else device.index
    _SPLIT_WS_OLD.pop(idx, None)
    if _SPLIT_WS.pop(idx, None) is not None:
        with torch.cuda.device(idx):
            torch.cuda.synchronize()
            _lib.check("fsvd_set_workspace", _lib.load().fsvd_set_workspace(None, 0, None))


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, *,
           norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
           residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None, cfg: int = 0) -> torch.Tensor:
    """out = (residual +) linear(rmsnorm?(x), weight, bias); weight is nn.Linear layout [N, K].
    Dispatches to the custom operator flashsvd_hip::linear (``.out`` when ``out`` is given)."""
    if out is None:
        return _OPS.linear.default(x, weight, bias, norm_weight, float(eps), residual, int(cfg))
    return _OPS.linear.out(x, weight, bias, norm_weight, float(eps), residual, int(cfg), out=out)


def _linear_impl(x, weight, bias, norm_weight, eps, residual, out, cfg):
    dt, code = _elem(x, "x")
    _need(weight, "weight", dtype=dt)
    if weight.dim() != 2 or weight.stride(1) != 1:
        raise ValueError(f"weight must be [N, K] with unit inner stride, got {tuple(weight.shape)} strides {weight.stride()}")
    N, K = weight.shape
    if x.shape[-1] != K:
        raise ValueError(f"x last dim {x.shape[-1]} != weight in_features {K}")
    x2 = _rows(x, "x")
    B = x2.shape[0]
    if out is None:
        out = torch.empty(*x.shape[:-1], N, device=x.device, dtype=dt)
    _need(out, "out", dtype=dt)
    o2 = _rows(out, "out")
    if o2.shape != (B, N) or o2.data_ptr() != out.data_ptr():
        raise ValueError("out must be a dense [..., N] tensor matching x")
    r2 = None
    if residual is not None:
        _need(residual, "residual", dtype=dt)
        r2 = _rows(residual, "residual")
        if r2.shape != (B, N):
            raise ValueError(f"residual shape {tuple(residual.shape)} does not match output [{B}, {N}]")
    for t, nm, n in ((bias, "bias", N), (norm_weight, "norm_weight", K)):
        if t is not None:
            _need(t, nm, dtype=dt)
            if t.shape != (n,) or not t.is_contiguous():
                raise ValueError(f"{nm} must be a contiguous [{n}] tensor")
    lib = _lib.load()
    if B >= 3:
        ensure_split_workspace(x.device)
    if norm_weight is not None and B >= 3 and cfg == 0 and K % 32 == 0:
        # three rows and more run on the matrix cores, which take the activations as they are: normalise once
        # up front (same rounding points as the fused prologue)
        x2 = _rmsnorm_impl(x2, norm_weight, eps, None)
        norm_weight = None
    rc = lib.fsvd_linear(x2.data_ptr(), x2.stride(0), weight.data_ptr(), weight.stride(0), _ptr(bias), _ptr(norm_weight),
                         float(eps), _ptr(r2), 0 if r2 is None else r2.stride(0), o2.data_ptr(), o2.stride(0),
                         B, N, K, int(cfg), code, _stream())
    _lib.check("fsvd_linear", rc)
    return out


def linear_rankkv_append(x: torch.Tensor, weight: torch.Tensor, pk_cache: torch.Tensor, pv_cache: torch.Tensor, positions: torch.Tensor, *,
                         ranks, norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6) -> torch.Tensor:
    """The packed rank projection of one or two decoded tokens, ``p = norm(x) @ weight.T`` with ``weight = [q_v; k_v; v_v]``
    and ``ranks = (rq, rk, rv)``, which also stores the Pk | Pv parts of every row at ``pk_cache[b, positions[b]]`` /
    ``pv_cache[b, positions[b]]`` (caches [>=B, S, R]): ``linear`` followed by ``rankkv_append`` in one launch, same bits.
    Custom operator flashsvd_hip::linear_rankkv_append (the caches are mutated arguments)."""
    rq, rk, rv = (int(r) for r in ranks)
    return _OPS.linear_rankkv_append.default(x, weight, pk_cache, pv_cache, positions, rq, rk, rv, norm_weight, float(eps))


def _linear_rankkv_append_impl(x, weight, pk_cache, pv_cache, positions, rq, rk, rv, norm_weight, eps):
    dt, code = _elem(x, "x")
    _need(weight, "weight", dtype=dt); _need(pk_cache, "pk_cache", dtype=dt); _need(pv_cache, "pv_cache", dtype=dt)
    _need(positions, "positions", dtype=torch.int32)
    if weight.dim() != 2 or weight.stride(1) != 1 or weight.shape[0] != rq + rk + rv:
        raise ValueError(f"weight must be [rq + rk + rv, K] = [{rq + rk + rv}, K] with unit inner stride, got {tuple(weight.shape)}")
    K = weight.shape[1]
    x2 = _rows(x, "x")
    B = x2.shape[0]
    if x2.shape[1] != K or B > 2:
        raise ValueError(f"x must be one or two rows of {K} values, got {tuple(x.shape)}")
    for c, r, nm in ((pk_cache, rk, "pk_cache"), (pv_cache, rv, "pv_cache")):
        if c.dim() != 3 or c.shape[0] < B or c.shape[2] != r or c.stride(2) != 1 or c.shape[1] != pk_cache.shape[1]:
            raise ValueError(f"{nm} must be [>={B}, S, {r}] with unit inner stride, got {tuple(c.shape)}")
    if positions.numel() != B or not positions.is_contiguous():
        raise ValueError(f"positions must be a contiguous int32 [{B}] tensor")
    if norm_weight is not None:
        _need(norm_weight, "norm_weight", dtype=dt)
        if norm_weight.shape != (K,) or not norm_weight.is_contiguous():
            raise ValueError(f"norm_weight must be a contiguous [{K}] tensor")
    out = torch.empty(*x.shape[:-1], rq + rk + rv, device=x.device, dtype=dt)
    o2 = _rows(out, "out")
    rc = _lib.load().fsvd_linear_rankkv_append(x2.data_ptr(), x2.stride(0), weight.data_ptr(), weight.stride(0), _ptr(norm_weight), float(eps),
                                               o2.data_ptr(), o2.stride(0), B, rq, rk, rv, K, pk_cache.data_ptr(), pk_cache.stride(0),
                                               pk_cache.stride(1), pv_cache.data_ptr(), pv_cache.stride(0), pv_cache.stride(1),
                                               positions.data_ptr(), int(pk_cache.shape[1]), code, _stream())
    _lib.check("fsvd_linear_rankkv_append", rc)
    return out


def swiglu_linear(p: torch.Tensor, gate_u: torch.Tensor, up_u: torch.Tensor, *, up_off: int, mode: int = 0,
                  out: Optional[torch.Tensor] = None, cfg: int = 0) -> torch.Tensor:
    """h = silu(p[..., :R] @ gate_u.T) * (p[..., up_off:up_off+R] @ up_u.T); gate_u/up_u are [D, R].
    Custom operator flashsvd_hip::swiglu_linear."""
    if out is None:
        return _OPS.swiglu_linear.default(p, gate_u, up_u, int(up_off), int(mode), int(cfg))
    return _OPS.swiglu_linear.out(p, gate_u, up_u, int(up_off), int(mode), int(cfg), out=out)


def _swiglu_linear_impl(p, gate_u, up_u, up_off, mode, out, cfg):
    dt, code = _elem(p, "p")
    _need(gate_u, "gate_u", dtype=dt); _need(up_u, "up_u", dtype=dt)
    if gate_u.dim() != 2 or gate_u.shape != up_u.shape or gate_u.stride() != up_u.stride() or gate_u.stride(1) != 1:
        raise ValueError(f"gate_u/up_u must be matching [D, R] weights, got {tuple(gate_u.shape)} / {tuple(up_u.shape)}")
    D, R = gate_u.shape
    p2 = _rows(p, "p")
    if p2.shape[1] < up_off + R:
        raise ValueError(f"p last dim {p2.shape[1]} too small for up_off {up_off} + R {R}")
    B = p2.shape[0]
    if out is None:
        out = torch.empty(*p.shape[:-1], D, device=p.device, dtype=dt)
    _need(out, "out", dtype=dt)
    o2 = _rows(out, "out")
    lib = _lib.load()
    if 3 <= B < 128:
        ensure_split_workspace(p.device)
    rc = lib.fsvd_swiglu_linear(p2.data_ptr(), p2.stride(0), int(up_off), gate_u.data_ptr(), up_u.data_ptr(),
                                gate_u.stride(0), o2.data_ptr(), o2.stride(0), B, D, R, int(mode), int(cfg), code, _stream())
    _lib.check("fsvd_swiglu_linear", rc)
    return out


def _q4_check(qweight, scales, zeros, N: int, K: int, group_size: int, name: str) -> int:
    """Validate one int4 matrix; returns the group width the kernel is given (0 = one group per row)."""
    if qweight.dtype != torch.uint8 or scales.dtype != torch.float16 or zeros.dtype != torch.int16:
        raise TypeError(f"{name}: expected uint8 weights, float16 scales and int16 zeros, got {qweight.dtype}, {scales.dtype}, "
                        f"{zeros.dtype}")
    if not (qweight.is_cuda and scales.is_cuda and zeros.is_cuda):
        raise ValueError(f"{name}: quantised buffers must be on the GPU")
    if qweight.dim() != 2 or qweight.shape != (N, (K + 1) // 2) or qweight.stride(1) != 1:
        raise ValueError(f"{name}: packed weight must be [{N}, {(K + 1) // 2}] bytes, got {tuple(qweight.shape)}")
    group = 0 if group_size <= 0 or group_size >= K else int(group_size)
    G = 1 if group == 0 else -(-K // group)
    if scales.shape != (N, G) or zeros.shape != (N, G) or scales.stride() != zeros.stride() or scales.stride(1) != 1:
        raise ValueError(f"{name}: scales / zeros must be matching [{N}, {G}] tensors, got {tuple(scales.shape)} / {tuple(zeros.shape)}")
    return group


def linear_q4(x: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, *, group_size: int,
              bias: Optional[torch.Tensor] = None, norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
              residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = (residual +) linear(rmsnorm?(x), s * (q - z), bias) on group-wise int4 weights [N, K/2] bytes."""
    dt, code = _elem(x, "x")
    N, K = qweight.shape[0], x.shape[-1]
    group = _q4_check(qweight, scales, zeros, N, K, group_size, "linear_q4")
    x2 = _rows(x, "x")
    B = x2.shape[0]
    if out is None:
        out = torch.empty(*x.shape[:-1], N, device=x.device, dtype=dt)
    _need(out, "out", dtype=dt)
    o2 = out if out.dim() == 2 else _rows(out, "out")
    if o2.shape != (B, N) or o2.stride(1) != 1:
        raise ValueError("out must be a [rows, N] tensor with unit inner stride matching x")
    r2 = None
    if residual is not None:
        _need(residual, "residual", dtype=dt)
        r2 = _rows(residual, "residual")
        if r2.shape != (B, N):
            raise ValueError(f"residual shape {tuple(residual.shape)} does not match output [{B}, {N}]")
    for t, nm, n in ((bias, "bias", N), (norm_weight, "norm_weight", K)):
        if t is not None:
            _need(t, nm, dtype=dt)
            if t.shape != (n,) or not t.is_contiguous():
                raise ValueError(f"{nm} must be a contiguous [{n}] tensor")
    lib = _lib.load()
    rc = lib.fsvd_linear_q4(x2.data_ptr(), x2.stride(0), qweight.data_ptr(), qweight.stride(0), scales.data_ptr(), zeros.data_ptr(),
                            scales.stride(0), group, _ptr(bias), _ptr(norm_weight), float(eps), _ptr(r2),
                            0 if r2 is None else r2.stride(0), o2.data_ptr(), o2.stride(0), B, N, K, code, _stream())
    _lib.check("fsvd_linear_q4", rc)
    return out


def swiglu_linear_q4(p: torch.Tensor, gate: tuple, up: tuple, *, up_off: int, group_size: int, mode: int = 0,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h = silu(p[..., :R] @ Wg.T) * (p[..., up_off:up_off+R] @ Wu.T); gate / up are (qweight, scales, zeros) of [D, R]."""
    dt, code = _elem(p, "p")
    (gq, gs, gz), (uq, us, uz) = gate, up
    D = gq.shape[0]
    R = 2 * gq.shape[1]
    p2 = _rows(p, "p")
    if p2.shape[1] < up_off + R:
        raise ValueError(f"p last dim {p2.shape[1]} too small for up_off {up_off} + R {R}")
    group = _q4_check(gq, gs, gz, D, R, group_size, "swiglu_linear_q4 gate")
    _q4_check(uq, us, uz, D, R, group_size, "swiglu_linear_q4 up")
    if gq.stride() != uq.stride() or gs.stride() != us.stride():
        raise ValueError("gate and up must share one layout")
    B = p2.shape[0]
    if out is None:
        out = torch.empty(*p.shape[:-1], D, device=p.device, dtype=dt)
    _need(out, "out", dtype=dt)
    o2 = _rows(out, "out")
    lib = _lib.load()
    rc = lib.fsvd_swiglu_linear_q4(p2.data_ptr(), p2.stride(0), int(up_off), gq.data_ptr(), gs.data_ptr(), gz.data_ptr(),
                                   uq.data_ptr(), us.data_ptr(), uz.data_ptr(), gq.stride(0), gs.stride(0), group,
                                   o2.data_ptr(), o2.stride(0), B, D, R, int(mode), code, _stream())
    _lib.check("fsvd_swiglu_linear_q4", rc)
    return out


def dequant_q4(qweight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, *, in_features: int, group_size: int,
               out: Optional[torch.Tensor] = None, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """[N, K] = s * (q - z), rounded once to ``dtype`` (bf16 or fp16; the type of ``out`` when that is given, else bf16)."""
    N, K = qweight.shape[0], int(in_features)
    group = _q4_check(qweight, scales, zeros, N, K, group_size, "dequant_q4")
    if out is None:
        out = torch.empty(N, K, device=qweight.device, dtype=dtype or _BF16)
    dt, code = _elem(out, "out")
    if out.shape != (N, K) or (dtype is not None and dt != dtype) or out.stride(1) != 1:
        raise ValueError(f"out must be a {dtype or 'bf16 / fp16'} [{N}, {K}] tensor with unit inner stride")
    lib = _lib.load()
    rc = lib.fsvd_dequant_q4(qweight.data_ptr(), qweight.stride(0), scales.data_ptr(), zeros.data_ptr(), scales.stride(0), group,
                             out.data_ptr(), out.stride(0), N, K, code, _stream())
    _lib.check("fsvd_dequant_q4", rc)
    return out


def qkv_rope_append(p: torch.Tensor, q_u: torch.Tensor, k_u: torch.Tensor, v_u: torch.Tensor,
                    cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
                    k_cache: torch.Tensor, v_cache: torch.Tensor, *, num_heads: int, num_kv_heads: int, head_dim: int,
                    q_out: Optional[torch.Tensor] = None, cfg: int = 0) -> torch.Tensor:
    """q (rotated) -> q_out [B,H,Dh]; rotated k and v written into the caches [B,S,Hk,Dh] at positions[b].
    Custom operator flashsvd_hip::qkv_rope_append (the caches are mutated arguments)."""
    a = (p, q_u, k_u, v_u, cos, sin, positions, k_cache, v_cache, int(num_heads), int(num_kv_heads), int(head_dim), int(cfg))
    return _OPS.qkv_rope_append.default(*a) if q_out is None else _OPS.qkv_rope_append.out(*a, q_out=q_out)


def _qkv_rope_append_impl(p, q_u, k_u, v_u, cos, sin, positions, k_cache, v_cache, num_heads, num_kv_heads, head_dim, q_out, cfg):
    dt, code = _elem(p, "p")
    for t, nm in ((q_u, "q_u"), (k_u, "k_u"), (v_u, "v_u"), (k_cache, "k_cache"), (v_cache, "v_cache")):
        _need(t, nm, dtype=dt)
    _need(positions, "positions", dtype=torch.int32)
    H, Hk, Dh = int(num_heads), int(num_kv_heads), int(head_dim)
    Rq, Rk, Rv = q_u.shape[1], k_u.shape[1], v_u.shape[1]
    if q_u.shape[0] != H * Dh or k_u.shape[0] != Hk * Dh or v_u.shape[0] != Hk * Dh:
        raise ValueError(f"u_proj rows do not match heads: {tuple(q_u.shape)}/{tuple(k_u.shape)}/{tuple(v_u.shape)} "
                         f"for H={H} Hk={Hk} Dh={Dh}")
    p2 = _rows(p, "p")
    B = p2.shape[0]
    if p2.shape[1] != Rq + Rk + Rv:
        raise ValueError(f"p last dim {p2.shape[1]} != Rq+Rk+Rv = {Rq + Rk + Rv}")
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.stride() != v_cache.stride() \
            or k_cache.shape[2:] != (Hk, Dh) or k_cache.shape[0] < B or k_cache.stride(3) != 1:
        raise ValueError(f"caches must be matching [B>={B}, S, {Hk}, {Dh}] tensors, got {tuple(k_cache.shape)}")
    if positions.numel() != B or not positions.is_contiguous():
        raise ValueError(f"positions must be a contiguous int32 [{B}] tensor")
    rope_len = 0
    if cos is not None:
        _need(cos, "cos", dtype=dt); _need(sin, "sin", dtype=dt)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != Dh // 2 or not cos.is_contiguous() or not sin.is_contiguous():
            raise ValueError(f"cos/sin must be contiguous [len, {Dh // 2}] tables")
        rope_len = cos.shape[0]
    if q_out is None:
        q_out = torch.empty(B, H, Dh, device=p.device, dtype=dt)
    elif q_out.shape != (B, H, Dh) or not q_out.is_contiguous() or q_out.dtype != dt:
        raise ValueError("q_out must be contiguous [B,H,Dh]")
    lib = _lib.load()
    rc = lib.fsvd_qkv_rope_append(p2.data_ptr(), p2.stride(0), q_u.data_ptr(), q_u.stride(0), k_u.data_ptr(), k_u.stride(0),
                                  v_u.data_ptr(), v_u.stride(0), _ptr(cos), _ptr(sin), rope_len, positions.data_ptr(),
                                  q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                  k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
                                  B, H, Hk, Dh, Rq, Rk, Rv, k_cache.shape[1], int(cfg), code, _stream())
    _lib.check("fsvd_qkv_rope_append", rc)
    return q_out


def pick_nsplit(max_len: int, batch: int, heads: int, head_dim: int = 128) -> int:
    """Key-axis split: about 128 keys per workgroup (one pass of loads in flight), bounded so that
    batch*heads*nsplit stays within ~2048 workgroups."""
    per_pass = 128 if head_dim >= 128 else 128
    n = max(1, math.ceil(max_len / per_pass))
    cap = max(1, 2048 // max(1, batch * heads))
    return int(max(1, min(n, cap)))


def attn_workspace(batch: int, heads: int, head_dim: int, nsplit: int, device) -> torch.Tensor:
    lib = _lib.load()
    nbytes = lib.fsvd_attn_decode_workspace_bytes(batch, heads, head_dim, nsplit)
    return torch.zeros(max(1, (nbytes + 3) // 4), dtype=torch.int32, device=device)


def attn_decode_densekv(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cache_seqlens: torch.Tensor, *,
                        k_new: Optional[torch.Tensor] = None, v_new: Optional[torch.Tensor] = None,
                        cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, seqlen_add: int = 0,
                        nsplit: Optional[int] = None, workspace: Optional[torch.Tensor] = None,
                        out: Optional[torch.Tensor] = None, softmax_scale: Optional[float] = None,
                        static_scratch: bool = False) -> torch.Tensor:
    """q [B,H,Dh] over caches [B,S,Hk,Dh]; see fsvd_attn_decode_densekv in include/flashsvd_hip.h.
    static_scratch=True takes fsvd_attn_decode_densekv_static (the library's own fixed scratch array).
    Custom operator flashsvd_hip::attn_decode_densekv."""
    a = (q, k_cache, v_cache, cache_seqlens, k_new, v_new, cos, sin, int(seqlen_add), None if nsplit is None else int(nsplit),
         workspace, None if not softmax_scale else float(softmax_scale), bool(static_scratch))
    return _OPS.attn_decode_densekv.default(*a) if out is None else _OPS.attn_decode_densekv.out(*a, out=out)


def _attn_decode_densekv_impl(q, k_cache, v_cache, cache_seqlens, k_new, v_new, cos, sin, seqlen_add, nsplit, workspace, out,
                              softmax_scale, static_scratch):
    dt, code = _elem(q, "q")
    _need(k_cache, "k_cache", dtype=dt); _need(v_cache, "v_cache", dtype=dt)
    _need(cache_seqlens, "cache_seqlens", dtype=torch.int32)
    if q.dim() != 3 or q.stride(2) != 1:
        raise ValueError(f"q must be [B,H,Dh] with unit inner stride, got {tuple(q.shape)}")
    B, H, Dh = q.shape
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.stride() != v_cache.stride() \
            or k_cache.shape[3] != Dh or k_cache.shape[0] < B or k_cache.stride(3) != 1:
        raise ValueError(f"caches must be matching [B>={B}, S, Hk, {Dh}] tensors, got {tuple(k_cache.shape)} / {tuple(v_cache.shape)}")
    S, Hk = k_cache.shape[1], k_cache.shape[2]
    if H % Hk != 0:
        raise ValueError(f"H={H} is not a multiple of Hk={Hk}")
    if cache_seqlens.numel() != B or not cache_seqlens.is_contiguous():
        raise ValueError(f"cache_seqlens must be a contiguous int32 [{B}] tensor")
    sk_b = sk_h = sv_b = sv_h = 0
    if k_new is not None:
        _need(k_new, "k_new", dtype=dt); _need(v_new, "v_new", dtype=dt)
        if k_new.shape != (B, Hk, Dh) or v_new.shape != (B, Hk, Dh) or k_new.stride(2) != 1 or v_new.stride(2) != 1:
            raise ValueError(f"k_new/v_new must be [B,Hk,Dh] tensors with unit inner stride, got {tuple(k_new.shape)} / {tuple(v_new.shape)}")
        sk_b, sk_h, sv_b, sv_h = k_new.stride(0), k_new.stride(1), v_new.stride(0), v_new.stride(1)
    rope_len = 0
    if cos is not None:
        _need(cos, "cos", dtype=dt); _need(sin, "sin", dtype=dt)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != Dh // 2 or not cos.is_contiguous() or not sin.is_contiguous():
            raise ValueError(f"cos/sin must be contiguous [len, {Dh // 2}] tables")
        rope_len = cos.shape[0]
    if nsplit is None:
        nsplit = pick_nsplit(S, B, H, Dh)
    if out is None:
        out = torch.empty(B, H, Dh, device=q.device, dtype=dt)
    elif out.shape != (B, H, Dh) or out.stride(2) != 1 or out.dtype != dt:
        raise ValueError("out must be [B,H,Dh] with unit inner stride")
    lib = _lib.load()
    if static_scratch:
        # library-owned scratch: no workspace tensor, nothing allocated inside the call (out must then be given too
        # by a caller that may not allocate)
        rc = lib.fsvd_attn_decode_densekv_static(q.data_ptr(), q.stride(0), q.stride(1), k_cache.data_ptr(), v_cache.data_ptr(),
                                                 k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
                                                 _ptr(k_new), sk_b, sk_h, _ptr(v_new), sv_b, sv_h, cache_seqlens.data_ptr(),
                                                 int(seqlen_add), _ptr(cos), _ptr(sin), rope_len, out.data_ptr(), out.stride(0),
                                                 out.stride(1), B, H, Hk, Dh, S, int(nsplit),
                                                 float(softmax_scale) if softmax_scale else 0.0, code, _stream())
        _lib.check("fsvd_attn_decode_densekv_static", rc)
        return out
    ws_ptr, ws_bytes = None, 0
    if nsplit > 1:
        if workspace is None:
            workspace = attn_workspace(B, H, Dh, nsplit, q.device)
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    rc = lib.fsvd_attn_decode_densekv(q.data_ptr(), q.stride(0), q.stride(1), k_cache.data_ptr(), v_cache.data_ptr(),
                                      k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
                                      _ptr(k_new), sk_b, sk_h, _ptr(v_new), sv_b, sv_h, cache_seqlens.data_ptr(), int(seqlen_add),
                                      _ptr(cos), _ptr(sin), rope_len, out.data_ptr(), out.stride(0), out.stride(1),
                                      ws_ptr, ws_bytes, B, H, Hk, Dh, S, int(nsplit),
                                      float(softmax_scale) if softmax_scale else 0.0, code, _stream())
    _lib.check("fsvd_attn_decode_densekv", rc)
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """w * bf16(x * rsqrt(mean(x^2) + eps)); custom operator flashsvd_hip::rmsnorm."""
    return _OPS.rmsnorm.default(x, weight, float(eps)) if out is None else _OPS.rmsnorm.out(x, weight, float(eps), out=out)


def _rmsnorm_impl(x, weight, eps, out):
    dt, code = _elem(x, "x")
    _need(weight, "weight", dtype=dt)
    K = x.shape[-1]
    if weight.shape != (K,) or not weight.is_contiguous():
        raise ValueError(f"weight must be contiguous [{K}]")
    x2 = _rows(x, "x")
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    _need(out, "out", dtype=dt)
    o2 = _rows(out, "out")
    lib = _lib.load()
    rc = lib.fsvd_rmsnorm(x2.data_ptr(), x2.stride(0), weight.data_ptr(), float(eps), o2.data_ptr(), o2.stride(0),
                          x2.shape[0], K, code, _stream())
    _lib.check("fsvd_rmsnorm", rc)
    return out


def _expand_operands(p, u, heads, Dh, out, bias, head_stride):
    """Checks of one head expansion; returns (B, M, R, coefficient strides, element code)."""
    dt, code = _elem(p, "p")
    _need(u, "u", dtype=dt); _need(out, "out", dtype=dt)
    if p.dim() == 3:
        B, M, R = p.shape
        sp = (p.stride(0), p.stride(1), 0 if head_stride is None else int(head_stride))
    elif p.dim() == 4:
        B, M, hp, R = p.shape
        if hp != heads:
            raise ValueError(f"p has {hp} heads, expected {heads}")
        sp = (p.stride(0), p.stride(1), p.stride(2))
    else:
        raise ValueError(f"p must be [B,M,R] or [B,M,heads,R], got {tuple(p.shape)}")
    if p.stride(-1) != 1 or u.stride(1) != 1 or out.stride(-1) != 1:
        raise ValueError("p, u and out need unit stride on the last axis")
    if u.shape != (heads * Dh, R):
        raise ValueError(f"u must be [{heads * Dh}, {R}], got {tuple(u.shape)}")
    if out.dim() != 4 or out.shape[0] < B or out.shape[2] != heads or out.shape[3] != Dh:
        raise ValueError(f"out must be [B>={B}, rows, {heads}, {Dh}], got {tuple(out.shape)}")
    if bias is not None:
        _need(bias, "bias", dtype=dt)
        if bias.numel() != heads * Dh or not bias.is_contiguous():
            raise ValueError(f"bias must be contiguous [{heads * Dh}]")
    return B, M, R, sp, code


def _rope_tables(cos, sin, Dh, dt):
    if cos is None:
        return 0
    _need(cos, "cos", dtype=dt); _need(sin, "sin", dtype=dt)
    if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != Dh // 2 or not cos.is_contiguous() or not sin.is_contiguous():
        raise ValueError(f"cos/sin must be contiguous [len, {Dh // 2}] tables")
    return cos.shape[0]


def lowrank_expand_heads(p: torch.Tensor, u: torch.Tensor, *, num_heads: int, head_dim: int, out: torch.Tensor,
                         cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                         positions: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                         dst_by_position: bool = False, head_stride: Optional[int] = None) -> torch.Tensor:
    """out[b, row, h, :] = rope(p[b, m, (h), :] @ u[h*Dh:(h+1)*Dh].T + bias); see fsvd_lowrank_expand_heads.
    p is [B, M, R] (shared by all heads) or [B, M, heads, R]; out is [B, rows, heads, Dh].
    Custom operator flashsvd_hip::lowrank_expand_heads (``out`` is the mutated argument)."""
    _OPS.lowrank_expand_heads.default(p, u, int(num_heads), int(head_dim), out, cos, sin, positions, bias, bool(dst_by_position),
                                      None if head_stride is None else int(head_stride))
    return out


def _lowrank_expand_heads_impl(p, u, num_heads, head_dim, out, cos, sin, positions, bias, dst_by_position, head_stride):
    heads, Dh = int(num_heads), int(head_dim)
    B, M, R, sp, code = _expand_operands(p, u, heads, Dh, out, bias, head_stride)
    rope_len = _rope_tables(cos, sin, Dh, p.dtype)
    if positions is not None:
        _need(positions, "positions", dtype=torch.int32)
        if positions.numel() != B:
            raise ValueError(f"positions must be int32 [{B}]")
    lib = _lib.load()
    rc = lib.fsvd_lowrank_expand_heads(p.data_ptr(), sp[0], sp[1], sp[2], u.data_ptr(), u.stride(0), _ptr(bias), _ptr(cos), _ptr(sin),
                                       rope_len, _ptr(positions), out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
                                       int(bool(dst_by_position)), out.shape[1], B, M, heads, Dh, R, code, _stream())
    _lib.check("fsvd_lowrank_expand_heads", rc)
    return out


def prefill_head_groups(B: int, M: int, n_ctx: int, H: int, Hk: int, Dh: int, itemsize: int = 2) -> int:
    """How many kv heads (with their query heads) the expand-then-attend prompt pass takes at a time.

    The pass rebuilds q [B,M,H,Dh] and K, V [B,n_ctx,Hk,Dh] from rank coefficients into temporaries and runs the prompt
    attention over them; nothing forces all heads to exist at once.  The largest group of kv heads whose temporaries
    fit FLASHSVD_AMD_PREFILL_TEMP_BYTES (default 1 GiB) is taken, at least one; 0 or a negative budget means all heads in
    one pass.  Groups cost a few per cent of the pass (8 x 2048 tokens at rank 1664: +4 % at 64 MiB, five kv heads per
    group), so the default only bounds the temporaries of very long batches."""
    import os
    budget = int(float(os.getenv("FLASHSVD_AMD_PREFILL_TEMP_BYTES", str(1 << 30))))
    if budget <= 0:
        return Hk
    per_kv_head = (B * M * (H // Hk) + 2 * B * n_ctx) * Dh * itemsize
    return max(1, min(Hk, budget // max(per_kv_head, 1)))


def lowrank_expand_heads_multi(items, *, head_dim: int, cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                               positions: Optional[torch.Tensor] = None) -> None:
    """The q / k / v expansions of one prompt pass in one call (fsvd_lowrank_expand_heads_multi): ``items`` is a list of one
    to three dicts with the keyword arguments of :func:`lowrank_expand_heads` for one expansion (``p``, ``u``,
    ``num_heads``, ``out``, optional ``bias``, ``dst_by_position``, ``head_stride``) plus ``rotate`` (apply cos / sin).
    The same results as separate calls; a single launch when every expansion takes the tiled kernel."""
    Dh = int(head_dim)
    if not 1 <= len(items) <= 3:
        raise ValueError(f"{len(items)} expansions (1..3)")
    rope_len = _rope_tables(cos, sin, Dh, items[0]["p"].dtype)
    descs = (_lib.ExpandDesc * len(items))()
    shape = code = None
    for d, it in zip(descs, items):
        heads, out, bias = int(it["num_heads"]), it["out"], it.get("bias")
        B, M, R, sp, c = _expand_operands(it["p"], it["u"], heads, Dh, out, bias, it.get("head_stride"))
        if shape is None:
            shape, code = (B, M), c
        elif shape != (B, M):
            raise ValueError(f"expansions of one call cover the same token rows: {shape} vs {(B, M)}")
        elif c != code:
            raise ValueError("expansions of one call are of one element type")
        if it.get("rotate") and cos is None:
            raise ValueError("rotate asked for without cos / sin")
        d.p, d.sp_b, d.sp_m, d.sp_h = it["p"].data_ptr(), sp[0], sp[1], sp[2]
        d.u, d.ldu, d.bias = it["u"].data_ptr(), it["u"].stride(0), _ptr(bias)
        d.y, d.sy_b, d.sy_m, d.sy_h = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
        d.heads, d.R, d.rotate = heads, R, int(bool(it.get("rotate")))
        d.dst_by_position, d.dst_rows, d.rsv0 = int(bool(it.get("dst_by_position"))), out.shape[1], 0
    B, M = shape
    if positions is not None:
        _need(positions, "positions", dtype=torch.int32)
        if positions.numel() != B:
            raise ValueError(f"positions must be int32 [{B}]")
    lib = _lib.load()
    rc = lib.fsvd_lowrank_expand_heads_multi(descs, len(items), _ptr(cos), _ptr(sin), rope_len, _ptr(positions), B, M, Dh, code, _stream())
    _lib.check("fsvd_lowrank_expand_heads_multi", rc)


def attn_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, q_pos0: Optional[torch.Tensor] = None, causal: bool = True,
                 pad_mask: Optional[torch.Tensor] = None, add_mask: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None, softmax_scale: Optional[float] = None) -> torch.Tensor:
    """q [B,M,H,Dh] (rotated), k/v [B,S,Hk,Dh] -> out [B,M,H,Dh]; keys n < q_pos0[b]+M, causal n <= q_pos0[b]+m.
    Custom operator flashsvd_hip::rope_attn_prefill."""
    a = (q, k, v, q_pos0, bool(causal), pad_mask, add_mask, None if not softmax_scale else float(softmax_scale))
    return _OPS.rope_attn_prefill.default(*a) if out is None else _OPS.rope_attn_prefill.out(*a, out=out)


def _attn_prefill_impl(q, k, v, q_pos0, causal, pad_mask, add_mask, out, softmax_scale):
    dt, code = _elem(q, "q")
    _need(k, "k", dtype=dt); _need(v, "v", dtype=dt)
    if q.dim() != 4 or k.dim() != 4 or k.shape != v.shape or k.stride() != v.stride():
        raise ValueError(f"q must be [B,M,H,Dh] and k/v matching [B,S,Hk,Dh], got {tuple(q.shape)} {tuple(k.shape)} {tuple(v.shape)}")
    B, M, H, Dh = q.shape
    S, Hk = k.shape[1], k.shape[2]
    if k.shape[0] < B or k.shape[3] != Dh or H % Hk:
        raise ValueError("k/v do not match q")
    if q.stride(3) != 1 or k.stride(3) != 1:
        raise ValueError("q, k, v need unit stride on the last axis")
    if out is None:
        out = torch.empty(B, M, H, Dh, device=q.device, dtype=dt)
    _need(out, "out", dtype=dt)
    spm = sam_b = sam_q = 0
    if pad_mask is not None:
        if pad_mask.dtype != torch.uint8 or pad_mask.dim() != 2 or pad_mask.shape[0] != B or pad_mask.stride(1) != 1:
            raise ValueError("pad_mask must be uint8 [B, keys]")
        spm = pad_mask.stride(0)
    if add_mask is not None:
        if add_mask.dtype != torch.float32 or add_mask.dim() != 3 or add_mask.shape[0] != B or add_mask.shape[1] != M or add_mask.stride(2) != 1:
            raise ValueError("add_mask must be float32 [B, M, keys]")
        sam_b, sam_q = add_mask.stride(0), add_mask.stride(1)
    if q_pos0 is not None:
        _need(q_pos0, "q_pos0", dtype=torch.int32)
    lib = _lib.load()
    rc = lib.fsvd_attn_prefill(q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), k.data_ptr(), v.data_ptr(), k.stride(0),
                               k.stride(1), k.stride(2), _ptr(q_pos0), _ptr(pad_mask), spm, _ptr(add_mask), sam_b, sam_q,
                               out.data_ptr(), out.stride(0), out.stride(1), out.stride(2), B, M, H, Hk, Dh, S, int(bool(causal)),
                               float(softmax_scale) if softmax_scale else 0.0, code, _stream())
    _lib.check("fsvd_attn_prefill", rc)
    return out
