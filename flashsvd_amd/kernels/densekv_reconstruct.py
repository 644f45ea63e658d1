"""Current-token Q/K/V reconstruction from rank coefficients (decode, q_len == 1).

Same function names, argument order, return values and error behaviour as the reference module
kernels/attn/decode/densekv_reconstruct_triton.py (wrappers at :360-760); the Triton tiling
keywords (BD, BR, num_warps, num_stages) are accepted and ignored.  All variants run one HIP
launch of the input-major GEMV in libflashsvd_hip (q, k and v as three problems of one grid)."""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ..torch_ops import ops as _OPS
from ._common import check, dtype_code, inner_contig, scratch, stream


def _all_cuda(*ts) -> bool:
    return all(t.is_cuda for t in ts)


def _bias_ok(b: Optional[torch.Tensor], name: str, heads: int, dh: int) -> Optional[torch.Tensor]:
    if b is None:
        return None
    if tuple(b.shape) != (heads, dh):
        raise ValueError(f"Expected {name} shape {(heads, dh)}, got {tuple(b.shape)}")
    return inner_contig(b)


def _launch(Pq, Pk, Pv, sP, Vq, Vk, Vv, bq, bk, bv, B, H, Hk, Dh, Rq, Rk, Rv):
    """sP: per matrix (stride_b, stride_h, stride_r) of the coefficient tensors.  Goes through the custom operator
    flashsvd_hip::reconstruct_qkv_token, which takes head-wise views [B, heads, R] (a head stride of 0 = shared)."""
    views = [P.as_strided((B, h, r), st) for P, h, r, st in ((Pq, H, Rq, sP[0]), (Pk, Hk, Rk, sP[1]), (Pv, Hk, Rv, sP[2]))]
    return _OPS.reconstruct_qkv_token.default(*views, Vq, Vk, Vv, bq, bk, bv)


def _heads_as_linear_layout(V: torch.Tensor) -> torch.Tensor:
    """[heads, R, Dh] basis -> nn.Linear layout [heads*Dh, R], built once per tensor (see rank_decode._as_linear_layout)."""
    from .rank_decode import _as_linear_layout
    return _as_linear_layout(V)


def _reconstruct_fast(Pq, Pk, Pv, Vq, Vk, Vv, bq, bk, bv):
    """Shared coefficients (head stride 0), bf16 or fp16: the head expansion of the product path on nn.Linear-layout twins of the
    bases — one launch (fsvd_qkv_rope_append without rotation, K and V written to one-row "caches") when there are no
    biases, else one fused-bias projection per matrix.  Same arithmetic as the reference kernels: fp32 sum (+ bias), one
    rounding (kernels/attn/decode/densekv_reconstruct_triton.py:170-237)."""
    import os
    from .. import hip_ops
    B, H, Rq = Pq.shape
    Hk, Rk, Rv, Dh = Pk.shape[1], Pk.shape[2], Pv.shape[2], Vq.shape[2]
    if os.getenv("FLASHSVD_AMD_REFERENCE_LAYOUT_FAST", "1") == "0" or Dh not in (64, 128):
        return None
    if Pq.dtype not in (torch.bfloat16, torch.float16) or any(t.dtype != Pq.dtype for t in (Pk, Pv, Vq, Vk, Vv, bq, bk, bv) if t is not None) or any(t.stride(1) != 0 or t.stride(2) != 1 for t in (Pq, Pk, Pv)):
        return None
    if Rq % 8 or Rk % 8 or Rv % 8:
        return None
    uq, uk, uv = _heads_as_linear_layout(Vq), _heads_as_linear_layout(Vk), _heads_as_linear_layout(Vv)
    pq, pk, pv = (t.as_strided((B, r), (t.stride(0), 1)) for t, r in ((Pq, Rq), (Pk, Rk), (Pv, Rv)))
    if bq is not None or bk is not None or bv is not None:
        flat = lambda b: None if b is None else b.reshape(-1).contiguous()
        return (hip_ops.linear(pq, uq, flat(bq)).view(B, H, Dh), hip_ops.linear(pk, uk, flat(bk)).view(B, Hk, Dh),
                hip_ops.linear(pv, uv, flat(bv)).view(B, Hk, Dh))
    adjacent = pk.data_ptr() == pq.data_ptr() + Rq * 2 and pv.data_ptr() == pk.data_ptr() + Rk * 2 and \
        pq.stride(0) == pk.stride(0) == pv.stride(0) >= Rq + Rk + Rv
    p = pq.as_strided((B, Rq + Rk + Rv), (pq.stride(0), 1)) if adjacent else torch.cat([pq, pk, pv], dim=1)
    K = torch.empty((B, 1, Hk, Dh), device=Pq.device, dtype=Pq.dtype)
    V = torch.empty_like(K)
    pos = scratch(Pq.device, 4096, "reconstruct_pos")[:B]          # zeros: every row writes its one cache slot
    Q = hip_ops.qkv_rope_append(p, uq, uk, uv, None, None, pos, K, V, num_heads=H, num_kv_heads=Hk, head_dim=Dh)
    return Q, K.view(B, Hk, Dh), V.view(B, Hk, Dh)


def _reconstruct_impl(Pq, Pk, Pv, Vq, Vk, Vv, bq, bk, bv):
    B, H, Rq = Pq.shape
    Hk, Rk, Rv, Dh = Pk.shape[1], Pk.shape[2], Pv.shape[2], Vq.shape[2]
    if B <= 64:       # decode batches; more rows take the input-major kernel below
        fast = _reconstruct_fast(Pq, Pk, Pv, Vq, Vk, Vv, bq, bk, bv)
        if fast is not None:
            return fast
    sP = [tuple(t.stride()) for t in (Pq, Pk, Pv)]
    Vq, Vk, Vv = inner_contig(Vq), inner_contig(Vk), inner_contig(Vv)
    for t, nm in ((Pk, "Pk"), (Pv, "Pv"), (Vq, "Vq"), (Vk, "Vk"), (Vv, "Vv")):
        if t.dtype != Pq.dtype:
            raise ValueError(f"{nm} has dtype {t.dtype}, expected {Pq.dtype}")
    dt = dtype_code(Pq)
    Q = torch.empty((B, H, Dh), device=Pq.device, dtype=Pq.dtype)
    K = torch.empty((B, Hk, Dh), device=Pq.device, dtype=Pq.dtype)
    V = torch.empty((B, Hk, Dh), device=Pq.device, dtype=Pq.dtype)
    lib = _lib.load()
    ws = scratch(Pq.device, lib.fsvd_reconstruct_qkv_workspace_bytes(B, H, Hk, Dh, Rq, Rk, Rv, dt), "reconstruct")

    def bias(b):
        return (None, 0) if b is None else (b.data_ptr(), b.stride(0))

    rc = lib.fsvd_reconstruct_qkv_token(
        Pq.data_ptr(), *sP[0], Pk.data_ptr(), *sP[1], Pv.data_ptr(), *sP[2],
        Vq.data_ptr(), Vq.stride(0), Vq.stride(1), Vk.data_ptr(), Vk.stride(0), Vk.stride(1),
        Vv.data_ptr(), Vv.stride(0), Vv.stride(1), *bias(bq), *bias(bk), *bias(bv),
        Q.data_ptr(), Q.stride(0), Q.stride(1), K.data_ptr(), K.stride(0), K.stride(1), V.data_ptr(), V.stride(0), V.stride(1),
        B, H, Hk, Dh, Rq, Rk, Rv, dt, ws.data_ptr(), ws.numel() * 4, stream())
    check("fsvd_reconstruct_qkv_token", rc)
    return Q, K, V


def reconstruct_qkv_token(Pq, Pk, Pv, Vq, Vk, Vv, *, bq=None, bk=None, bv=None, BD: int = 64, BR: int = 64,
                          num_warps: int = 4, num_stages: int = 2):
    """Head-wise coefficients: Pq [B,H,R], Pk/Pv [B,Hk,R]; bases Vq [H,R,Dh], Vk/Vv [Hk,R,Dh].
    Returns Q [B,H,Dh], K [B,Hk,Dh], V [B,Hk,Dh]."""
    if not _all_cuda(Pq, Pk, Pv, Vq, Vk, Vv):
        raise ValueError("reconstruct_qkv_token expects all tensors on CUDA.")
    if Pq.ndim != 3 or Pk.ndim != 3 or Pv.ndim != 3:
        raise ValueError(f"Expected Pq/Pk/Pv to be 3D [B,H|Hk,R], got {tuple(Pq.shape)}/{tuple(Pk.shape)}/{tuple(Pv.shape)}")
    if Vq.ndim != 3 or Vk.ndim != 3 or Vv.ndim != 3:
        raise ValueError(f"Expected Vq/Vk/Vv to be 3D [H|Hk,R,Dh], got {tuple(Vq.shape)}/{tuple(Vk.shape)}/{tuple(Vv.shape)}")
    B, H, R = Pq.shape
    Hk = Pk.shape[1]
    if Pk.shape[0] != B or Pv.shape[0] != B or Pv.shape[1] != Hk or Pk.shape[2] != R or Pv.shape[2] != R:
        raise ValueError("Mismatched token-factor shapes.")
    if Vq.shape[0] != H or Vk.shape[0] != Hk or Vv.shape[0] != Hk:
        raise ValueError("Mismatched basis head dimensions.")
    if Vq.shape[1] != R or Vk.shape[1] != R or Vv.shape[1] != R:
        raise ValueError("Mismatched rank dimension between P* and V*.")
    Dh = int(Vq.shape[2])
    if Vk.shape[2] != Dh or Vv.shape[2] != Dh:
        raise ValueError("All bases must share the same head_dim.")
    bq, bk, bv = _bias_ok(bq, "bq", H, Dh), _bias_ok(bk, "bk", Hk, Dh), _bias_ok(bv, "bv", Hk, Dh)
    sP = [tuple(t.stride()) for t in (Pq, Pk, Pv)]
    return _launch(Pq, Pk, Pv, sP, Vq, Vk, Vv, bq, bk, bv, B, H, Hk, Dh, R, R, R)


def reconstruct_qkv_token_shared_hetero(Pq, Pk, Pv, Vq, Vk, Vv, *, bq=None, bk=None, bv=None, BD: int = 64, BR: int = 64,
                                        num_warps: int = 4, num_stages: int = 2):
    """One coefficient vector per token shared by all heads, ranks may differ:
    Pq [B,Rq], Pk [B,Rk], Pv [B,Rv]; Vq [H,Rq,Dh], Vk [Hk,Rk,Dh], Vv [Hk,Rv,Dh]."""
    if not _all_cuda(Pq, Pk, Pv, Vq, Vk, Vv):
        raise ValueError("reconstruct_qkv_token_shared_hetero expects all tensors on CUDA.")
    if Pq.ndim != 2 or Pk.ndim != 2 or Pv.ndim != 2:
        raise ValueError(f"Expected Pq/Pk/Pv to be 2D [B,R*], got {tuple(Pq.shape)}/{tuple(Pk.shape)}/{tuple(Pv.shape)}")
    if Vq.ndim != 3 or Vk.ndim != 3 or Vv.ndim != 3:
        raise ValueError(f"Expected Vq/Vk/Vv to be 3D [H|Hk,R*,Dh], got {tuple(Vq.shape)}/{tuple(Vk.shape)}/{tuple(Vv.shape)}")
    B, Rq = Pq.shape
    Rk, Rv = int(Pk.shape[1]), int(Pv.shape[1])
    if Pk.shape[0] != B or Pv.shape[0] != B:
        raise ValueError("Mismatched batch dimension across Pq/Pk/Pv.")
    H, Hk, Dh = int(Vq.shape[0]), int(Vk.shape[0]), int(Vq.shape[2])
    for nm, V, r in (("Vq", Vq, Rq), ("Vk", Vk, Rk), ("Vv", Vv, Rv)):
        if V.shape[1] != r:
            raise ValueError(f"Expected {nm} rank {r}, got {int(V.shape[1])}")
    if Vv.shape[0] != Hk or Vk.shape[2] != Dh or Vv.shape[2] != Dh:
        raise ValueError("All bases must share the same head_dim.")
    bq, bk, bv = _bias_ok(bq, "bq", H, Dh), _bias_ok(bk, "bk", Hk, Dh), _bias_ok(bv, "bv", Hk, Dh)
    sP = [(t.stride(0), 0, t.stride(1)) for t in (Pq, Pk, Pv)]
    return _launch(Pq, Pk, Pv, sP, Vq, Vk, Vv, bq, bk, bv, B, H, Hk, Dh, Rq, Rk, Rv)


def reconstruct_qkv_token_shared(Pq, Pk, Pv, Vq, Vk, Vv, *, bq=None, bk=None, bv=None, BD: int = 64, BR: int = 64,
                                 num_warps: int = 4, num_stages: int = 2):
    """Shared global-rank coefficients with one common rank: Pq/Pk/Pv [B,R]."""
    if not _all_cuda(Pq, Pk, Pv, Vq, Vk, Vv):
        raise ValueError("reconstruct_qkv_token_shared expects all tensors on CUDA.")
    if Pq.ndim != 2 or Pk.ndim != 2 or Pv.ndim != 2:
        raise ValueError(f"Expected Pq/Pk/Pv to be 2D [B,R*], got {tuple(Pq.shape)}/{tuple(Pk.shape)}/{tuple(Pv.shape)}")
    if Vq.ndim != 3 or Vk.ndim != 3 or Vv.ndim != 3:
        raise ValueError(f"Expected Vq/Vk/Vv to be 3D [H|Hk,R,Dh], got {tuple(Vq.shape)}/{tuple(Vk.shape)}/{tuple(Vv.shape)}")
    B, R = Pq.shape
    if tuple(Pk.shape) != (B, R) or tuple(Pv.shape) != (B, R):
        raise ValueError("Mismatched shared factor shapes.")
    Dh = int(Vq.shape[2])
    if Vq.shape[1] != R or Vk.shape[1] != R or Vv.shape[1] != R or Vk.shape[2] != Dh or Vv.shape[2] != Dh:
        raise ValueError("Mismatched basis shapes for shared factor reconstruction.")
    return reconstruct_qkv_token_shared_hetero(Pq, Pk, Pv, Vq, Vk, Vv, bq=bq, bk=bk, bv=bv)


def pack_qkv_shared_bases(Vq, Vk, Vv):
    """[H|Hk, R, Dh] -> [R, H*Dh] / [R, Hk*Dh]: one-time repack for decode loops that reuse the bases."""
    if not _all_cuda(Vq, Vk, Vv):
        raise ValueError("pack_qkv_shared_bases expects CUDA tensors.")
    if Vq.ndim != 3 or Vk.ndim != 3 or Vv.ndim != 3:
        raise ValueError(f"Expected Vq/Vk/Vv to be 3D [H|Hk,R,Dh], got {tuple(Vq.shape)}/{tuple(Vk.shape)}/{tuple(Vv.shape)}")
    Dh = int(Vq.shape[2])
    if Vk.shape[2] != Dh or Vv.shape[2] != Dh:
        raise ValueError("All bases must share the same head_dim.")

    def flat(V):
        heads, r, _ = V.shape
        return V.transpose(0, 1).reshape(r, heads * Dh).contiguous()
    return flat(Vq), flat(Vk), flat(Vv)


def _xw(x: torch.Tensor, W: torch.Tensor, bias: Optional[torch.Tensor], bias_post: bool) -> torch.Tensor:
    """Custom operator flashsvd_hip::xw_linear."""
    return _OPS.xw_linear.default(x, W, bias, bool(bias_post))


def _xw_impl(x, W, bias, bias_post):
    lib = _lib.load()
    B, K = x.shape
    N = W.shape[1]
    W = inner_contig(W)
    y = torch.empty((B, N), device=x.device, dtype=x.dtype)
    dt = dtype_code(x)
    ws = scratch(x.device, lib.fsvd_xw_linear_workspace_bytes(B, K, N, dt), "xw_linear")
    rc = lib.fsvd_xw_linear(x.data_ptr(), x.stride(0), x.stride(1), 0, W.data_ptr(), W.stride(0),
                            None if bias is None else bias.data_ptr(), int(bias_post), y.data_ptr(), y.stride(0), 0,
                            B, K, N, dt, ws.data_ptr(), ws.numel() * 4, stream())
    check("fsvd_xw_linear", rc)
    return y


def xw_linear(x: torch.Tensor, W: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ W`` for x [B,K] and a row-major [K,N] matrix such as the packed rank projection
    (the product the reference issues as torch.matmul, benchmark/attn/decode_compare.py:1538)."""
    if not _all_cuda(x, W):
        raise ValueError("xw_linear expects all tensors on CUDA.")
    if x.ndim != 2 or W.ndim != 2 or x.shape[1] != W.shape[0]:
        raise ValueError(f"xw_linear: x {tuple(x.shape)} does not chain with W {tuple(W.shape)}")
    return _xw(x, W, bias, False)


def reconstruct_qkv_token_shared_prepacked(Pq, Pk, Pv, Vq_flat, Vk_flat, Vv_flat, *, H: int, Hk: int, Dh: int,
                                           bq=None, bk=None, bv=None):
    """Q = Pq @ Vq_flat etc. on the prepacked [R, heads*Dh] bases; the bias is added after the
    product has been rounded, as the reference does with a separate add."""
    if not _all_cuda(Pq, Pk, Pv, Vq_flat, Vk_flat, Vv_flat):
        raise ValueError("reconstruct_qkv_token_shared_prepacked expects all tensors on CUDA.")
    if Pq.ndim != 2 or Pk.ndim != 2 or Pv.ndim != 2:
        raise ValueError(f"Expected shared Pq/Pk/Pv to be 2D [B,R], got {tuple(Pq.shape)}/{tuple(Pk.shape)}/{tuple(Pv.shape)}")
    if Vq_flat.ndim != 2 or Vk_flat.ndim != 2 or Vv_flat.ndim != 2:
        raise ValueError(f"Expected prepacked bases to be 2D [R,N], got {tuple(Vq_flat.shape)}/{tuple(Vk_flat.shape)}/{tuple(Vv_flat.shape)}")
    B, Rq = Pq.shape
    Rk, Rv = int(Pk.shape[1]), int(Pv.shape[1])
    if Pk.shape[0] != B or Pv.shape[0] != B:
        raise ValueError("Mismatched batch dimension across Pq/Pk/Pv.")
    for nm, Vf, shp in (("Vq_flat", Vq_flat, (Rq, H * Dh)), ("Vk_flat", Vk_flat, (Rk, Hk * Dh)), ("Vv_flat", Vv_flat, (Rv, Hk * Dh))):
        if tuple(Vf.shape) != shp:
            raise ValueError(f"Expected {nm} shape {shp}, got {tuple(Vf.shape)}")
    bq, bk, bv = _bias_ok(bq, "bq", H, Dh), _bias_ok(bk, "bk", Hk, Dh), _bias_ok(bv, "bv", Hk, Dh)

    def one(P, Vf, b, heads):
        bias = None if b is None else b.reshape(heads * Dh).contiguous()
        return _xw(P, Vf, bias, True).reshape(B, heads, Dh)
    return one(Pq, Vq_flat, bq, H), one(Pk, Vk_flat, bk, Hk), one(Pv, Vv_flat, bv, Hk)


__all__ = ["reconstruct_qkv_token", "reconstruct_qkv_token_shared", "reconstruct_qkv_token_shared_hetero",
           "pack_qkv_shared_bases", "reconstruct_qkv_token_shared_prepacked", "xw_linear"]
