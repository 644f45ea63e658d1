"""Decode attention over the rank-space KV cache.

The reference resolves these entry points from kernel files that are not part of its checkout
(runtime/attn/decode_registry.py:38-150); their call contract is the one its benchmark drives
(benchmark/attn/decode_compare.py:823-948): ``DecodePackedFactors`` holds the query's rank
coefficients Pq [B,H,R], the cached Pk/Pv [B,L,Hk,R] (shared-rank caches arrive as zero-stride
expands over the head axis) and the per-head bases Vq/Vk/Vv [heads,R,Dh];
``flashsvd_attn_decode_packed(factors, cos_half, sin_half, seqlen_k=..., workspace=(M,L,Acc),
out=...)`` returns the attention output [B,H,Dh].  Semantics follow the pure-torch streaming
reference, decode_compare.py:586-750.  Tiling keywords (bn, br, num_warps_*, num_stages_*,
pad_to_16, writethrough, vk_resident) are accepted and ignored."""
from __future__ import annotations

import math
import weakref
from dataclasses import dataclass
from typing import Optional

import torch

from .. import _lib
from ..torch_ops import ops as _OPS
from ._common import check, stream


@dataclass
class DecodePackedFactors:
    Pq: torch.Tensor
    Pk: torch.Tensor
    Pv: torch.Tensor
    Vq: torch.Tensor
    Vk: torch.Tensor
    Vv: torch.Tensor
    bq: Optional[torch.Tensor] = None
    bk: Optional[torch.Tensor] = None
    bv: Optional[torch.Tensor] = None


_LINEAR_LAYOUT: dict = {}


def _as_linear_layout(V: torch.Tensor) -> torch.Tensor:
    """[heads, R, Dh] basis -> [heads*Dh, R] (nn.Linear layout, contiguous along R), cached per tensor."""
    key = (V.data_ptr(), tuple(V.shape), tuple(V.stride()), V._version)
    hit = _LINEAR_LAYOUT.get(key)
    if hit is not None and hit[0]() is V:
        return hit[1]
    heads, r, dh = V.shape
    out = V.transpose(1, 2).reshape(heads * dh, r).contiguous()
    if len(_LINEAR_LAYOUT) > 256:
        _LINEAR_LAYOUT.clear()
    _LINEAR_LAYOUT[key] = (weakref.ref(V), out)
    return out


# test hooks: force the one-kernel form for every shape; a list that receives the score buffer of each call (or None)
_FORCE_ONE_KERNEL = False
_KEEP_SCORES: Optional[list] = None


def rank_decode(q: torch.Tensor, pk_cache: torch.Tensor, pv_cache: torch.Tensor, k_u: torch.Tensor, v_u: torch.Tensor,
                cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], seqlens: torch.Tensor, *, num_kv_heads: int,
                seqlen_add: int = 0, rotate_q: bool = False, bv: Optional[torch.Tensor] = None, nsplit: Optional[int] = None,
                workspace=None, out: Optional[torch.Tensor] = None, softmax_scale: Optional[float] = None) -> torch.Tensor:
    """q [B,H,Dh]; pk_cache/pv_cache [B,S,R] (shared) or [B,S,Hk,R]; k_u/v_u nn.Linear weights [Hk*Dh,R].
    Custom operator flashsvd_hip::attn_decode_rankkv; ``workspace`` = (M, L, Acc)."""
    ws_m, ws_l, ws_acc = workspace if workspace is not None else (None, None, None)
    a = (q, pk_cache, pv_cache, k_u, v_u, cos, sin, seqlens, int(num_kv_heads), int(seqlen_add), bool(rotate_q), bv,
         None if nsplit is None else int(nsplit), ws_m, ws_l, ws_acc, None if not softmax_scale else float(softmax_scale))
    return _OPS.attn_decode_rankkv.default(*a) if out is None else _OPS.attn_decode_rankkv.out(*a, out=out)


def _rank_decode_impl(q, pk_cache, pv_cache, k_u, v_u, cos, sin, seqlens, num_kv_heads, seqlen_add, rotate_q, bv, nsplit,
                      ws_m, ws_l, ws_acc, out, softmax_scale):
    workspace = None if ws_m is None else (ws_m, ws_l, ws_acc)
    codes = {torch.bfloat16: 0, torch.float16: 1}      # FSVD_BF16, FSVD_FP16: q names the element type of the call
    if q.dtype not in codes:
        raise ValueError(f"rank-space decode computes in bfloat16 or float16; q is {q.dtype}")
    for t, nm in ((q, "q"), (pk_cache, "pk_cache"), (pv_cache, "pv_cache"), (k_u, "k_u"), (v_u, "v_u"), (bv, "bv"), (cos, "cos"), (sin, "sin")):
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError(f"{nm} must be a GPU tensor")
        if t.dtype != q.dtype:
            raise ValueError(f"rank-space decode: {nm} is {t.dtype}, q is {q.dtype}")
    B, H, Dh = q.shape
    Hk = int(num_kv_heads)
    if pk_cache.dim() == 3:
        spk = (pk_cache.stride(0), pk_cache.stride(1), 0)
        spv = (pv_cache.stride(0), pv_cache.stride(1), 0)
    elif pk_cache.dim() == 4:
        spk = (pk_cache.stride(0), pk_cache.stride(1), pk_cache.stride(2))
        spv = (pv_cache.stride(0), pv_cache.stride(1), pv_cache.stride(2))
    else:
        raise ValueError(f"coefficient caches must be [B,S,R] or [B,S,Hk,R], got {tuple(pk_cache.shape)}")
    S, Rk, Rv = pk_cache.shape[1], pk_cache.shape[-1], pv_cache.shape[-1]
    if pk_cache.stride(-1) != 1 or pv_cache.stride(-1) != 1 or q.stride(-1) != 1:
        raise ValueError("q and the coefficient caches need unit stride on the last axis")
    if k_u.shape != (Hk * Dh, Rk) or v_u.shape != (Hk * Dh, Rv) or k_u.stride(1) != 1 or v_u.stride(1) != 1:
        raise ValueError(f"k_u/v_u must be [Hk*Dh, R] weights, got {tuple(k_u.shape)} / {tuple(v_u.shape)}")
    if seqlens.dtype != torch.int32 or seqlens.numel() != B:
        raise ValueError(f"seqlens must be int32 [{B}]")
    if nsplit is None:
        nsplit = max(1, min(math.ceil(S / 64), max(1, 1024 // max(1, B * Hk))))
    if workspace is None:
        M = torch.empty(B, H, nsplit, device=q.device, dtype=torch.float32)
        L = torch.empty_like(M)
        Acc = torch.empty(B, H, nsplit, Rv, device=q.device, dtype=torch.float32)
    else:
        M, L, Acc = workspace
        nsplit = int(M.shape[2])
        if tuple(M.shape) != (B, H, nsplit) or tuple(L.shape) != (B, H, nsplit) or tuple(Acc.shape) != (B, H, nsplit, Rv):
            raise ValueError(f"workspace must be (M,L [B,H,S], Acc [B,H,S,R]) with matching shapes, got "
                             f"{tuple(M.shape)} {tuple(L.shape)} {tuple(Acc.shape)}")
        for t in (M, L, Acc):
            if t.dtype != torch.float32 or not t.is_contiguous():
                raise ValueError("workspace tensors must be contiguous float32")
    if out is None:
        out = torch.empty(B, H, Dh, device=q.device, dtype=q.dtype)
    rope_len = 0 if cos is None else int(cos.shape[0])
    lib = _lib.load()
    # long caches shared by the heads: the library runs score / softmax / accumulation launches when the call brings a
    # buffer for its scores; the size query depends on the shape alone, so a captured graph and an eager call of the
    # same shape take the same form, and the buffer is the call's own (nothing shared between streams)
    need = 0 if _FORCE_ONE_KERNEL else int(lib.fsvd_attn_decode_rankkv_scores_bytes(B, H, S, 1 if spv[2] == 0 else 0))
    scores = torch.empty(need // 4, device=q.device, dtype=torch.float32) if need else None
    if _KEEP_SCORES is not None:
        _KEEP_SCORES.append(scores)
    rc = lib.fsvd_attn_decode_rankkv(
        q.data_ptr(), q.stride(0), q.stride(1), pk_cache.data_ptr(), *spk, pv_cache.data_ptr(), *spv,
        k_u.data_ptr(), k_u.stride(0), v_u.data_ptr(), v_u.stride(0), None if bv is None else bv.data_ptr(),
        None if cos is None else cos.data_ptr(), None if sin is None else sin.data_ptr(), rope_len, int(bool(rotate_q)),
        seqlens.data_ptr(), int(seqlen_add), M.data_ptr(), L.data_ptr(), Acc.data_ptr(), out.data_ptr(), out.stride(0),
        out.stride(1), B, H, Hk, Dh, S, Rk, Rv, int(nsplit), float(softmax_scale) if softmax_scale else 0.0,
        None if scores is None else scores.data_ptr(), need, codes[q.dtype], stream())
    check("fsvd_attn_decode_rankkv", rc)
    return out


def rankkv_append(pk: torch.Tensor, pv: torch.Tensor, pk_cache: torch.Tensor, pv_cache: torch.Tensor, positions: torch.Tensor) -> None:
    """pk_cache[b, positions[b]] = pk[b], pv_cache[b, positions[b]] = pv[b] in one launch: the one-token case of
    FlashSVDLegacySparseKVCache.update (runtime/cache/attn_legacy_sparse_kv.py:113-169).  pk / pv [B,R] (row views of a
    wider buffer are fine), caches [>=B,S,R] bf16, positions int32 [B] on the device; positions outside the cache are dropped.
    Custom operator flashsvd_hip::rankkv_append."""
    _OPS.rankkv_append.default(pk, pv, pk_cache, pv_cache, positions)


def _rankkv_append_impl(pk, pv, pk_cache, pv_cache, positions):
    for t, nm in ((pk, "pk"), (pv, "pv"), (pk_cache, "pk_cache"), (pv_cache, "pv_cache")):
        if not t.is_cuda or t.dtype not in (torch.bfloat16, torch.float16) or t.dtype != pk.dtype:
            raise ValueError(f"{nm} must be a bfloat16 or float16 GPU tensor of the rows' type")
        if t.stride(-1) != 1:
            raise ValueError(f"{nm} needs unit stride on the last axis")
    B, Rk = pk.shape
    Rv = pv.shape[1]
    if pv.shape[0] != B or pk_cache.dim() != 3 or pv_cache.dim() != 3 or pk_cache.shape[0] < B or pv_cache.shape[0] < B:
        raise ValueError(f"shapes do not agree: pk {tuple(pk.shape)} pv {tuple(pv.shape)} caches {tuple(pk_cache.shape)} / {tuple(pv_cache.shape)}")
    if pk_cache.shape[2] != Rk or pv_cache.shape[2] != Rv or pk_cache.shape[1] != pv_cache.shape[1]:
        raise ValueError(f"cache ranks / lengths do not match the rows: {tuple(pk_cache.shape)} / {tuple(pv_cache.shape)} for ranks {Rk} / {Rv}")
    if positions.dtype != torch.int32 or positions.numel() != B or not positions.is_cuda:
        raise ValueError(f"positions must be int32 [{B}] on the device")
    lib = _lib.load()
    rc = lib.fsvd_rankkv_append(pk.data_ptr(), pk.stride(0), pv.data_ptr(), pv.stride(0), pk_cache.data_ptr(), pk_cache.stride(0),
                                pk_cache.stride(1), pv_cache.data_ptr(), pv_cache.stride(0), pv_cache.stride(1), positions.data_ptr(),
                                B, int(pk_cache.shape[1]), Rk, Rv, stream())
    check("fsvd_rankkv_append", rc)


def flashsvd_attn_decode_packed(factors: DecodePackedFactors, cos_half: Optional[torch.Tensor], sin_half: Optional[torch.Tensor], *,
                                seqlen_k: Optional[int] = None, causal: bool = True, split_k: int = 512, bn: int = 64,
                                br: int = 64, num_warps_stage1: int = 4, num_stages_stage1: int = 2, num_warps_stage2: int = 4,
                                num_stages_stage2: int = 2, workspace=None, out: Optional[torch.Tensor] = None,
                                q_buffers=None, precompute_q: bool = True, pad_to_16: bool = True, writethrough: bool = True,
                                vk_resident: bool = True) -> torch.Tensor:
    """Attention of the token at position seqlen_k-1 over keys [0, seqlen_k): returns [B,H,Dh]."""
    f = factors
    if f.Pq.dim() != 3:
        raise ValueError(f"Pq must be [B,H,R], got {tuple(f.Pq.shape)}")
    if f.Pk.dim() != 4 or f.Pv.dim() != 4:
        raise ValueError(f"Pk/Pv must be [B,L,Hk,R], got {tuple(f.Pk.shape)} / {tuple(f.Pv.shape)}")
    B, H, Rq = f.Pq.shape
    _, L, Hk, Rk = f.Pk.shape
    Dh = int(f.Vq.shape[2])
    if seqlen_k is None:
        seqlen_k = L
    if not 0 < int(seqlen_k) <= L:
        raise ValueError(f"seqlen_k={seqlen_k} outside (0, {L}]")
    # query: rebuilt from its rank coefficients with the head-wise reconstruct kernel (its k/v outputs are unused)
    from .densekv_reconstruct import reconstruct_qkv_token
    Q, _, _ = reconstruct_qkv_token(f.Pq, f.Pq[:, :1], f.Pq[:, :1], f.Vq, f.Vq[:1], f.Vq[:1], bq=f.bq)
    shared = f.Pk.stride(2) == 0 and f.Pv.stride(2) == 0
    pk = f.Pk[:, :, 0] if shared else f.Pk
    pv = f.Pv[:, :, 0] if shared else f.Pv
    if f.bk is not None:
        raise NotImplementedError("a key bias does not commute with in-kernel RoPE reconstruction; fold it into the cache")
    seqlens = torch.full((B,), int(seqlen_k), dtype=torch.int32, device=f.Pq.device)
    bv = None if f.bv is None else f.bv.reshape(-1).contiguous()
    return rank_decode(Q, pk, pv, _as_linear_layout(f.Vk), _as_linear_layout(f.Vv), cos_half, sin_half, seqlens,
                       num_kv_heads=Hk, rotate_q=cos_half is not None, bv=bv, workspace=workspace, out=out)


flashsvd_attn_decode_packed_v1 = flashsvd_attn_decode_packed

__all__ = ["DecodePackedFactors", "flashsvd_attn_decode_packed", "flashsvd_attn_decode_packed_v1", "rank_decode", "rankkv_append"]
