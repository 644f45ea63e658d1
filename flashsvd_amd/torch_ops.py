"""PyTorch custom operators ``flashsvd_hip::*`` over the C ABI of libflashsvd_hip.

Every hot entry point of the library is a dispatcher-visible operator with a schema (mutated arguments are
annotated), a device implementation that checks its operands and makes the ctypes call, and a fake / meta
implementation that only derives output shapes — so the operators can be traced, compiled around and run on fake
tensors.  ``flashsvd_amd.hip_ops`` and the modules under ``flashsvd_amd.kernels`` call them through ``torch.ops``.

  linear / linear.out                 fsvd_linear            rank projections, factor pairs, fused RMSNorm / residual
  swiglu_linear / .out                fsvd_swiglu_linear     gate_u / up_u pair + SwiGLU
  rmsnorm / .out                      fsvd_rmsnorm
  qkv_rope_append / .out              fsvd_qkv_rope_append   head expansion + RoPE + dense-cache append
  attn_decode_densekv / .out          fsvd_attn_decode_densekv(_static)   the flash_attn_with_kvcache role
  attn_decode_rankkv / .out           fsvd_attn_decode_rankkv             decode over the rank-space cache
  rankkv_append                       fsvd_rankkv_append
  lowrank_expand_heads                fsvd_lowrank_expand_heads           prompt-pass head expansion (+ RoPE)
  rope_attn_prefill / .out            fsvd_attn_prefill                   causal prompt attention
  reconstruct_qkv_token               fsvd_reconstruct_qkv_token          reference-layout current-token q / k / v
  xw_linear                           fsvd_xw_linear                      reference-layout x @ W
  mlp_dual_split                      fsvd_mlp_dual_split                 reference-layout dual-split MLP

The implementations are registered for every backend key (the Python bodies raise ``ValueError`` for tensors that
are not on the GPU, as the reference's wrappers do); the Meta key carries the shape functions.
"""
from __future__ import annotations

from typing import Optional

import torch

NS = "flashsvd_hip"
_lib = torch.library.Library(NS, "DEF")
_BF16 = torch.bfloat16


def _define(schema: str, impl, fake) -> None:
    name = schema.split("(", 1)[0]
    _lib.define(schema)
    _lib.impl(name, impl, "CompositeExplicitAutograd")
    torch.library.register_fake(f"{NS}::{name}", fake, lib=_lib)


# ------------------------------------------------------------------ linear
def _linear(x, weight, bias=None, norm_weight=None, eps=1e-6, residual=None, cfg=0):
    from . import hip_ops
    return hip_ops._linear_impl(x, weight, bias, norm_weight, eps, residual, None, cfg)


def _linear_out(x, weight, bias=None, norm_weight=None, eps=1e-6, residual=None, cfg=0, *, out):
    from . import hip_ops
    return hip_ops._linear_impl(x, weight, bias, norm_weight, eps, residual, out, cfg)


def _linear_fake(x, weight, bias=None, norm_weight=None, eps=1e-6, residual=None, cfg=0):
    return x.new_empty((*x.shape[:-1], weight.shape[0]))


_define("linear(Tensor x, Tensor weight, Tensor? bias=None, Tensor? norm_weight=None, float eps=1e-6, Tensor? residual=None, "
        "int cfg=0) -> Tensor", _linear, _linear_fake)
_define("linear.out(Tensor x, Tensor weight, Tensor? bias=None, Tensor? norm_weight=None, float eps=1e-6, Tensor? residual=None, "
        "int cfg=0, *, Tensor(a!) out) -> Tensor(a!)", _linear_out, lambda *a, out, **k: out)


# ------------------------------------------------------------------ SwiGLU pair
def _swiglu(p, gate_u, up_u, up_off, mode=0, cfg=0):
    from . import hip_ops
    return hip_ops._swiglu_linear_impl(p, gate_u, up_u, up_off, mode, None, cfg)


def _swiglu_out(p, gate_u, up_u, up_off, mode=0, cfg=0, *, out):
    from . import hip_ops
    return hip_ops._swiglu_linear_impl(p, gate_u, up_u, up_off, mode, out, cfg)


_define("swiglu_linear(Tensor p, Tensor gate_u, Tensor up_u, int up_off, int mode=0, int cfg=0) -> Tensor", _swiglu,
        lambda p, gate_u, up_u, up_off, mode=0, cfg=0: p.new_empty((*p.shape[:-1], gate_u.shape[0])))
_define("swiglu_linear.out(Tensor p, Tensor gate_u, Tensor up_u, int up_off, int mode=0, int cfg=0, *, Tensor(a!) out) -> Tensor(a!)",
        _swiglu_out, lambda *a, out, **k: out)


# ------------------------------------------------------------------ RMSNorm
def _rmsnorm(x, weight, eps=1e-6):
    from . import hip_ops
    return hip_ops._rmsnorm_impl(x, weight, eps, None)


def _rmsnorm_out(x, weight, eps=1e-6, *, out):
    from . import hip_ops
    return hip_ops._rmsnorm_impl(x, weight, eps, out)


_define("rmsnorm(Tensor x, Tensor weight, float eps=1e-6) -> Tensor", _rmsnorm,
        lambda x, weight, eps=1e-6: torch.empty_like(x, memory_format=torch.contiguous_format))
_define("rmsnorm.out(Tensor x, Tensor weight, float eps=1e-6, *, Tensor(a!) out) -> Tensor(a!)", _rmsnorm_out,
        lambda *a, out, **k: out)


# ------------------------------------------------------------------ q / k / v expansion + RoPE + cache append
def _qkv(p, q_u, k_u, v_u, cos, sin, positions, k_cache, v_cache, num_heads, num_kv_heads, head_dim, cfg=0):
    from . import hip_ops
    return hip_ops._qkv_rope_append_impl(p, q_u, k_u, v_u, cos, sin, positions, k_cache, v_cache, num_heads, num_kv_heads,
                                         head_dim, None, cfg)


def _qkv_out(p, q_u, k_u, v_u, cos, sin, positions, k_cache, v_cache, num_heads, num_kv_heads, head_dim, cfg=0, *, q_out):
    from . import hip_ops
    return hip_ops._qkv_rope_append_impl(p, q_u, k_u, v_u, cos, sin, positions, k_cache, v_cache, num_heads, num_kv_heads,
                                         head_dim, q_out, cfg)


def _qkv_fake(p, q_u, k_u, v_u, cos, sin, positions, k_cache, v_cache, num_heads, num_kv_heads, head_dim, cfg=0):
    rows = p.numel() // p.shape[-1]
    return p.new_empty((rows, num_heads, head_dim))


_QKV_ARGS = ("Tensor p, Tensor q_u, Tensor k_u, Tensor v_u, Tensor? cos, Tensor? sin, Tensor positions, Tensor(a!) k_cache, "
             "Tensor(b!) v_cache, int num_heads, int num_kv_heads, int head_dim, int cfg=0")
_define(f"qkv_rope_append({_QKV_ARGS}) -> Tensor", _qkv, _qkv_fake)
_define(f"qkv_rope_append.out({_QKV_ARGS}, *, Tensor(c!) q_out) -> Tensor(c!)", _qkv_out, lambda *a, q_out, **k: q_out)


# ------------------------------------------------------------------ decode attention, dense cache
def _attn_dense(q, k_cache, v_cache, cache_seqlens, k_new=None, v_new=None, cos=None, sin=None, seqlen_add=0, nsplit=None,
                workspace=None, softmax_scale=None, static_scratch=False):
    from . import hip_ops
    return hip_ops._attn_decode_densekv_impl(q, k_cache, v_cache, cache_seqlens, k_new, v_new, cos, sin, seqlen_add, nsplit,
                                             workspace, None, softmax_scale, static_scratch)


def _attn_dense_out(q, k_cache, v_cache, cache_seqlens, k_new=None, v_new=None, cos=None, sin=None, seqlen_add=0, nsplit=None,
                    workspace=None, softmax_scale=None, static_scratch=False, *, out):
    from . import hip_ops
    return hip_ops._attn_decode_densekv_impl(q, k_cache, v_cache, cache_seqlens, k_new, v_new, cos, sin, seqlen_add, nsplit,
                                             workspace, out, softmax_scale, static_scratch)


_AD_ARGS = ("Tensor q, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor cache_seqlens, Tensor? k_new=None, Tensor? v_new=None, "
            "Tensor? cos=None, Tensor? sin=None, int seqlen_add=0, int? nsplit=None, Tensor(c!)? workspace=None, "
            "float? softmax_scale=None, bool static_scratch=False")
_define(f"attn_decode_densekv({_AD_ARGS}) -> Tensor", _attn_dense, lambda q, *a, **k: q.new_empty(q.shape))
_define(f"attn_decode_densekv.out({_AD_ARGS}, *, Tensor(d!) out) -> Tensor(d!)", _attn_dense_out, lambda *a, out, **k: out)


# ------------------------------------------------------------------ decode attention, rank-space cache
def _attn_rank(q, pk_cache, pv_cache, k_u, v_u, cos, sin, seqlens, num_kv_heads, seqlen_add=0, rotate_q=False, bv=None, nsplit=None,
               ws_m=None, ws_l=None, ws_acc=None, softmax_scale=None):
    from .kernels import rank_decode as RD
    return RD._rank_decode_impl(q, pk_cache, pv_cache, k_u, v_u, cos, sin, seqlens, num_kv_heads, seqlen_add, rotate_q, bv, nsplit,
                                ws_m, ws_l, ws_acc, None, softmax_scale)


def _attn_rank_out(q, pk_cache, pv_cache, k_u, v_u, cos, sin, seqlens, num_kv_heads, seqlen_add=0, rotate_q=False, bv=None,
                   nsplit=None, ws_m=None, ws_l=None, ws_acc=None, softmax_scale=None, *, out):
    from .kernels import rank_decode as RD
    return RD._rank_decode_impl(q, pk_cache, pv_cache, k_u, v_u, cos, sin, seqlens, num_kv_heads, seqlen_add, rotate_q, bv, nsplit,
                                ws_m, ws_l, ws_acc, out, softmax_scale)


_AR_ARGS = ("Tensor q, Tensor pk_cache, Tensor pv_cache, Tensor k_u, Tensor v_u, Tensor? cos, Tensor? sin, Tensor seqlens, "
            "int num_kv_heads, int seqlen_add=0, bool rotate_q=False, Tensor? bv=None, int? nsplit=None, Tensor(a!)? ws_m=None, "
            "Tensor(b!)? ws_l=None, Tensor(c!)? ws_acc=None, float? softmax_scale=None")
_define(f"attn_decode_rankkv({_AR_ARGS}) -> Tensor", _attn_rank, lambda q, *a, **k: torch.empty_like(q, memory_format=torch.contiguous_format))
_define(f"attn_decode_rankkv.out({_AR_ARGS}, *, Tensor(d!) out) -> Tensor(d!)", _attn_rank_out, lambda *a, out, **k: out)


def _linear_rankkv_append(x, weight, pk_cache, pv_cache, positions, rq, rk, rv, norm_weight=None, eps=1e-6):
    from . import hip_ops
    return hip_ops._linear_rankkv_append_impl(x, weight, pk_cache, pv_cache, positions, rq, rk, rv, norm_weight, eps)


_define("linear_rankkv_append(Tensor x, Tensor weight, Tensor(a!) pk_cache, Tensor(b!) pv_cache, Tensor positions, int rq, int rk, int rv, "
        "Tensor? norm_weight=None, float eps=1e-6) -> Tensor", _linear_rankkv_append,
        lambda x, weight, *a, **k: x.new_empty((*x.shape[:-1], weight.shape[0])))


def _rankkv_append(pk, pv, pk_cache, pv_cache, positions):
    from .kernels import rank_decode as RD
    RD._rankkv_append_impl(pk, pv, pk_cache, pv_cache, positions)


_define("rankkv_append(Tensor pk, Tensor pv, Tensor(a!) pk_cache, Tensor(b!) pv_cache, Tensor positions) -> ()", _rankkv_append,
        lambda *a, **k: None)


# ------------------------------------------------------------------ prompt pass
def _expand(p, u, num_heads, head_dim, out, cos=None, sin=None, positions=None, bias=None, dst_by_position=False, head_stride=None):
    from . import hip_ops
    hip_ops._lowrank_expand_heads_impl(p, u, num_heads, head_dim, out, cos, sin, positions, bias, dst_by_position, head_stride)


_define("lowrank_expand_heads(Tensor p, Tensor u, int num_heads, int head_dim, Tensor(a!) out, Tensor? cos=None, Tensor? sin=None, "
        "Tensor? positions=None, Tensor? bias=None, bool dst_by_position=False, int? head_stride=None) -> ()", _expand,
        lambda *a, **k: None)


def _prefill(q, k, v, q_pos0=None, causal=True, pad_mask=None, add_mask=None, softmax_scale=None):
    from . import hip_ops
    return hip_ops._attn_prefill_impl(q, k, v, q_pos0, causal, pad_mask, add_mask, None, softmax_scale)


def _prefill_out(q, k, v, q_pos0=None, causal=True, pad_mask=None, add_mask=None, softmax_scale=None, *, out):
    from . import hip_ops
    return hip_ops._attn_prefill_impl(q, k, v, q_pos0, causal, pad_mask, add_mask, out, softmax_scale)


_PF_ARGS = ("Tensor q, Tensor k, Tensor v, Tensor? q_pos0=None, bool causal=True, Tensor? pad_mask=None, Tensor? add_mask=None, "
            "float? softmax_scale=None")
_define(f"rope_attn_prefill({_PF_ARGS}) -> Tensor", _prefill, lambda q, *a, **k: q.new_empty(q.shape))
_define(f"rope_attn_prefill.out({_PF_ARGS}, *, Tensor(a!) out) -> Tensor(a!)", _prefill_out, lambda *a, out, **k: out)


# ------------------------------------------------------------------ reference operand layouts
def _reconstruct(Pq, Pk, Pv, Vq, Vk, Vv, bq=None, bk=None, bv=None):
    from .kernels import densekv_reconstruct as DR
    return DR._reconstruct_impl(Pq, Pk, Pv, Vq, Vk, Vv, bq, bk, bv)


def _reconstruct_fake(Pq, Pk, Pv, Vq, Vk, Vv, bq=None, bk=None, bv=None):
    B, H, Hk, Dh = Pq.shape[0], Vq.shape[0], Vk.shape[0], Vq.shape[2]
    return Pq.new_empty((B, H, Dh)), Pq.new_empty((B, Hk, Dh)), Pq.new_empty((B, Hk, Dh))


_define("reconstruct_qkv_token(Tensor Pq, Tensor Pk, Tensor Pv, Tensor Vq, Tensor Vk, Tensor Vv, Tensor? bq=None, Tensor? bk=None, "
        "Tensor? bv=None) -> (Tensor, Tensor, Tensor)", _reconstruct, _reconstruct_fake)


def _xw(x, W, bias=None, bias_post=False):
    from .kernels import densekv_reconstruct as DR
    return DR._xw_impl(x, W, bias, bias_post)


_define("xw_linear(Tensor x, Tensor W, Tensor? bias=None, bool bias_post=False) -> Tensor", _xw,
        lambda x, W, bias=None, bias_post=False: x.new_empty((x.shape[0], W.shape[1])))


def _dual_split(PUp, PGate, GateU, UpU, DownV, DownU, b2, variant, BD, partials_fp32=True, s_out=None):
    from .kernels import dual_split as DS
    return DS._run_impl(PUp, PGate, GateU, UpU, DownV, DownU, b2, variant, BD, partials_fp32, s_out)


_define("mlp_dual_split(Tensor PUp, Tensor PGate, Tensor GateU, Tensor UpU, Tensor DownV, Tensor DownU, Tensor? b2, int variant, "
        "int BD, bool partials_fp32=True, Tensor(a!)? s_out=None) -> Tensor", _dual_split,
        lambda PUp, PGate, GateU, UpU, DownV, DownU, b2, variant, BD, partials_fp32=True, s_out=None:
        PUp.new_empty((PUp.shape[0], DownU.shape[1])))

ops = getattr(torch.ops, NS)
OP_NAMES = ("linear", "swiglu_linear", "rmsnorm", "qkv_rope_append", "attn_decode_densekv", "attn_decode_rankkv", "rankkv_append", "linear_rankkv_append",
            "lowrank_expand_heads", "rope_attn_prefill", "reconstruct_qkv_token", "xw_linear", "mlp_dual_split")
