"""Fused low-rank RoPE attention for full sequences (prefill): the public module of the
reference's kernels/attn/prefill/rope_sdpa.py, re-exported there as kernels/flashsvdropeattn.py.

``FlashSVDRoPEAttention(num_heads, head_dim, rotary_emb).forward(QKVFactors, attention_mask,
position_ids)`` returns O [B,M,H,dh].  Q, K and V are rebuilt from the rank coefficients on the
matrix cores exactly once per token (fsvd_lowrank_expand_heads, rotation fused), then a causal
flash-attention pass runs over them (fsvd_attn_prefill).  Arithmetic is bf16 storage with fp32
accumulation; the Triton tile sizes (bm, bn, bdh, br) are accepted and ignored."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
from torch import nn

from .. import hip_ops
from .rank_decode import _as_linear_layout


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_bmhd(x_bmhd: torch.Tensor, cos_bmhd: torch.Tensor, sin_bmhd: torch.Tensor) -> torch.Tensor:
    """Rotate the two halves of the last axis with the first-half angles of cos/sin."""
    x1, x2 = x_bmhd.chunk(2, dim=-1)
    half = x1.shape[-1]
    c, s = cos_bmhd[..., :half], sin_bmhd[..., :half]
    return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1)


@dataclass
class QKVFactors:
    """Pq [B,H,M,R]; Pk,Pv [B,Hk,M,R]; Vq [H,R,dh]; Vk,Vv [Hk,R,dh]; optional biases [H*dh]."""
    Pq: torch.Tensor
    Pk: torch.Tensor
    Pv: torch.Tensor
    Vq: torch.Tensor
    Vk: torch.Tensor
    Vv: torch.Tensor
    bq: Optional[torch.Tensor] = None
    bk: Optional[torch.Tensor] = None
    bv: Optional[torch.Tensor] = None


class FlashSVDRoPEAttention(nn.Module):
    def __init__(self, num_heads: int, head_dim: int, rotary_emb, *, bm=64, bn=64, bdh=None, br=64):
        super().__init__()
        self.num_heads, self.head_dim, self.rotary_emb = num_heads, head_dim, rotary_emb
        self.bm, self.bn, self.br = bm, bn, br
        self.bdh = head_dim if bdh is None else bdh
        assert self.bdh == head_dim, "Kernel currently expects BDH == dh."
        self.causal = True   # decoder-only

    def _tables(self, B: int, M: int, dh: int, position_ids, device, dtype):
        """Per-token cos/sin rows [rows, dh/2] and the row offset of each batch entry."""
        if position_ids is None:
            position_ids = torch.arange(M, device=device, dtype=torch.long).unsqueeze(0)
        if position_ids.dim() == 1:
            position_ids = position_ids.unsqueeze(0)
        if position_ids.shape[-1] != M:
            raise ValueError(f"position_ids last dim {position_ids.shape[-1]} != M {M}")
        if position_ids.shape[0] not in (1, B):
            raise ValueError(f"position_ids batch dim {position_ids.shape[0]} != B {B}")
        inv = getattr(self.rotary_emb, "inv_freq", None)
        if inv is not None:
            ang = position_ids.to(device=device, dtype=torch.float32)[..., None] * inv.to(device=device, dtype=torch.float32)
            cos, sin = torch.cos(ang).to(dtype), torch.sin(ang).to(dtype)          # [Bpos, M, dh/2]
        else:
            dummy = torch.empty((position_ids.shape[0], M, dh), device=device, dtype=dtype)
            try:
                cos, sin = self.rotary_emb(dummy, position_ids)
            except TypeError:
                cos, sin = self.rotary_emb(dummy, seq_len=M)
                if cos.dim() == 4:
                    cos, sin = cos[:, 0], sin[:, 0]
            cos, sin = cos[..., : dh // 2].to(dtype), sin[..., : dh // 2].to(dtype)
        shared = cos.shape[0] == 1
        offs = torch.zeros(B, dtype=torch.int32, device=device) if shared else \
            torch.arange(B, dtype=torch.int32, device=device) * M
        return cos.reshape(-1, dh // 2).contiguous(), sin.reshape(-1, dh // 2).contiguous(), offs

    @torch.no_grad()
    def forward(self, qkv_factors: QKVFactors, attention_mask: Optional[torch.Tensor], position_ids: torch.Tensor,
                sliding_window_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        f = qkv_factors
        H, dh = self.num_heads, self.head_dim
        if f.Pq.dim() != 4:
            raise ValueError(f"FlashSVDRoPEAttention expects Pq [B,H,M,R], got {tuple(f.Pq.shape)}")
        B, Hq, M, R = f.Pq.shape
        if Hq != H:
            raise ValueError(f"Pq has {Hq} heads, expected {H}")
        if f.Pk.dim() != 4 or f.Pv.dim() != 4:
            raise ValueError(f"Expected Pk/Pv [B,Hk,M,R], got {tuple(f.Pk.shape)}/{tuple(f.Pv.shape)}")
        Bk, Hk, Mk, Rk = f.Pk.shape
        assert Bk == B and Mk == M and Rk == R, "Pk shape mismatch vs Pq"
        if f.Pq.dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"the MI355X prefill kernels compute in bfloat16 or float16; got {f.Pq.dtype}")
        if (f.bk is not None or f.bv is not None) and Hk != H:
            raise NotImplementedError("key/value biases indexed by query head need H == Hk")
        dev, dt = f.Pq.device, f.Pq.dtype
        cos, sin, offs = self._tables(B, M, dh, position_ids, dev, dt)

        def coeff(P):   # [B,h,M,R] -> view [B,M,h,R] without copying (head stride may be 0)
            P = P if P.stride(-1) == 1 else P.contiguous()
            return P.permute(0, 2, 1, 3)

        def bias(b, heads):
            return None if b is None else b.reshape(-1)[: heads * dh].to(dt).contiguous()

        uq, uk, uv = _as_linear_layout(f.Vq), _as_linear_layout(f.Vk), _as_linear_layout(f.Vv)
        Pq, Pk, Pv = coeff(f.Pq), coeff(f.Pk), coeff(f.Pv)
        bq, bk, bv = bias(f.bq, H), bias(f.bk, Hk), bias(f.bv, Hk)
        pad = add = None
        if attention_mask is not None:
            if attention_mask.dim() == 2:
                pad = (attention_mask != 0).to(torch.uint8).contiguous()
            elif attention_mask.dim() == 4:
                add = attention_mask[:, 0].to(torch.float32).expand(B, M, M).contiguous()
            else:
                raise ValueError(f"Unsupported attention_mask shape: {attention_mask.shape}")
        if sliding_window_mask is not None:
            add = sliding_window_mask[:, 0].to(torch.float32).expand(B, M, M).contiguous()
        # q, K, V are rebuilt and consumed one group of kv heads at a time (hip_ops.prefill_head_groups): the temporaries of
        # a group are reused by the next, so the pass never holds q / k / v of all heads (the activation-memory property of
        # the reference's kernel, which rebuilds its tiles inside the attention loop, without its rebuild per query tile)
        G = H // Hk
        gk = hip_ops.prefill_head_groups(B, M, M, H, Hk, dh)
        q = torch.empty(B, M, gk * G, dh, device=dev, dtype=dt)
        k = torch.empty(B, M, gk, dh, device=dev, dtype=dt)
        v = torch.empty_like(k)
        out = torch.empty(B, M, H, dh, device=dev, dtype=dt)

        def rows(t, r0, r1):
            return None if t is None else t[r0:r1]

        for k0 in range(0, Hk, gk):
            k1 = min(k0 + gk, Hk)
            nk, nq = k1 - k0, (k1 - k0) * G
            hip_ops.lowrank_expand_heads_multi(
                [dict(p=Pq[:, :, k0 * G:k1 * G], u=uq[k0 * G * dh:k1 * G * dh], num_heads=nq, out=q[:, :, :nq], rotate=True,
                      bias=rows(bq, k0 * G * dh, k1 * G * dh)),
                 dict(p=Pk[:, :, k0:k1], u=uk[k0 * dh:k1 * dh], num_heads=nk, out=k[:, :, :nk], rotate=True, bias=rows(bk, k0 * dh, k1 * dh)),
                 dict(p=Pv[:, :, k0:k1], u=uv[k0 * dh:k1 * dh], num_heads=nk, out=v[:, :, :nk], bias=rows(bv, k0 * dh, k1 * dh))],
                head_dim=dh, cos=cos, sin=sin, positions=offs)
            hip_ops.attn_prefill(q[:, :, :nq], k[:, :, :nk], v[:, :, :nk], causal=self.causal, pad_mask=pad, add_mask=add,
                                 out=out[:, :, k0 * G:k1 * G])
        return out


__all__ = ["FlashSVDRoPEAttention", "QKVFactors", "apply_rotary_bmhd", "rotate_half"]
