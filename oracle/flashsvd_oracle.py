"""CPU oracle for the low-rank Llama decode hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file; it is
used by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` as the checker / the reported CPU figure, never as the product path.

It is a plain PyTorch-on-CPU restatement (no custom kernels) of the algorithms the
reference implements with Triton kernels, cuBLAS calls and flash-attn, with every
floating-point rounding point written out.  Each function names the reference
file:line it follows (paths relative to the reference checkout).

Arithmetic contract used everywhere ("dtype" is torch.float32, torch.bfloat16 or torch.float16):
  * every matrix product accumulates in fp32 and is rounded once to ``dtype``
    (what a chain of ``nn.Linear`` modules does on an accelerator);
  * element-wise ops on ``dtype`` tensors round after every op, like eager PyTorch;
  * softmax runs in fp32.

Pinning status (see tests/test_oracle_pins.py):
  lin / lowrank_pair         closed form in float64, dense special case
  rms_norm                   transformers LlamaRMSNorm
  rope_tables / apply_rope   closed form, norm preservation, relative-position
                             invariance, transformers apply_rotary_pos_emb
  reconstruct_qkv_token*     flat-GEMM identity, all four variants agree
  dense_decode_attn          torch scaled_dot_product_attention
  flash_attn_with_kvcache    append-then-attend == last row of causal SDPA
  rank_decode_attn           == dense decode on reconstructed K/V, block-size
                             invariance, V-absorption identity
  rope_sdpa_prefill          == reconstruct -> RoPE -> causal SDPA; padded rows -> 0
  dual_split_mlp             closed form, D-tile partition invariance, HF LlamaMLP
  LowRankLlama (block/model) transformers LlamaForCausalLM built from W = U @ V
  greedy_decode              cached decode == full-sequence recompute
  pack_int4 / quantize_weight / dequantize_weight / quant_linear
                             hand-worked vectors, pack/unpack round trip, |w - dequant| <= scale/2,
                             symmetric zero point, all-zero group, fp64 closed form of the linear
  exact mode (act_dtype=fp64) same functions on fp64 activations: equals an independent float64 restatement with
                             numpy loops on a small block; a bf16 run stays within the bf16 rounding budget of it
Where this restatement is deliberately finer than the reference's own torch code: ``rank_decode_attn`` keeps the
rebuilt K (and V) tiles in fp32, while the reference's streaming function rounds each einsum result to the input
dtype first (benchmark/attn/decode_compare.py:718-721); the absent fused kernels keep them in registers, and the
difference (one bf16 rounding of K before the scores) is inside the decode tolerance.
parity unpinned (source absent from the reference checkout, behaviour defined here):
  the op order / rounding points of models/llama.py (SVD_LlamaAttention.forward,
  SVD_LlamaMLP.forward) and the bit-level behaviour of flash-attn 2.8.3.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------
# primitives
# ----------------------------------------------------------------------------
def _ct(x: torch.Tensor) -> torch.dtype:
    """Accumulation type: fp32, or fp64 when the activations themselves are fp64 (the exact mode below)."""
    return torch.float64 if x.dtype == torch.float64 else torch.float32


def lin(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``nn.Linear``: y = x @ w.T (+ bias), w is [out, in]; fp32 accumulate, one rounding.

    Follows the chain-of-linears reference at
    benchmark/attn/bench_real_checkpoint_decode_reconstruct.py:116-123.

    Exact mode: with fp32 or fp64 activations ``x`` and the same (bf16-valued) weights the final cast is
    a no-op, so a forward pass fed fp64 activations carries no intermediate rounding at all — the ground
    truth that two bf16 implementations with different fp32 summation orders are both measured against.
    """
    ct = _ct(x)
    y = x.to(ct) @ w.to(ct).t()
    if bias is not None:
        y = y + bias.to(ct)
    return y.to(x.dtype)


def lowrank_pair(x: torch.Tensor, v_w: torch.Tensor, u_w: torch.Tensor) -> torch.Tensor:
    """y = u_proj(v_proj(x)); v_w is [R, in] (applied first), u_w is [out, R].

    src/methods/svdllm/SVDLLM_flashsvd.py:292-294,324-350.
    """
    return lin(lin(x, v_w), u_w)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """benchmark/mlp/bench_svd_llama_decode_graph.py:78-83 (cast to input dtype, then * w)."""
    x32 = x.to(_ct(x))
    var = x32.pow(2).mean(-1, keepdim=True)
    return weight.to(x.dtype) * (x32 * torch.rsqrt(var + float(eps))).to(x.dtype)


def rope_tables(seqlen: int, head_dim: int, theta: float = 10000.0,
                dtype: torch.dtype = torch.float32) -> tuple[torch.Tensor, torch.Tensor]:
    """cos/sin [seqlen, head_dim/2]; fp32 angles then cast.  runtime/cache/attn_dense_kv.py:331-357."""
    half = head_dim // 2
    pos = torch.arange(seqlen, dtype=torch.float32)
    inv_freq = 1.0 / (float(theta) ** (torch.arange(0, half, dtype=torch.float32) / half))
    ang = pos[:, None] * inv_freq[None, :]
    return torch.cos(ang).to(dtype).contiguous(), torch.sin(ang).to(dtype).contiguous()


def apply_rope(x: torch.Tensor, cos_half: torch.Tensor, sin_half: torch.Tensor) -> torch.Tensor:
    """Rotate-half RoPE in eager-PyTorch arithmetic (rounds after each op in x.dtype).

    x [..., Dh]; cos_half/sin_half broadcastable to [..., Dh/2].
    out = [x0*cos - x1*sin , x1*cos + x0*sin]  — the element-wise form of
    ``x*cos + rotate_half(x)*sin`` (kernels/attn/prefill/rope_sdpa.py:29-37).
    """
    half = x.shape[-1] // 2
    x0, x1 = x[..., :half], x[..., half:]
    c = cos_half.to(x.dtype)
    s = sin_half.to(x.dtype)
    return torch.cat([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1)


def apply_rope_fp32(x: torch.Tensor, cos_half: torch.Tensor, sin_half: torch.Tensor) -> torch.Tensor:
    """Same rotation computed in fp32 with a single final rounding (what a fused
    attention kernel does to q and k_new; benchmark/attn/decode_compare.py:773-802)."""
    half = x.shape[-1] // 2
    x0, x1 = x[..., :half].float(), x[..., half:].float()
    c, s = cos_half.float(), sin_half.float()
    return torch.cat([x0 * c - x1 * s, x0 * s + x1 * c], dim=-1).to(x.dtype)


# ----------------------------------------------------------------------------
# current-token Q/K/V reconstruction (reference kernel-level API)
# ----------------------------------------------------------------------------
def _bias(y: torch.Tensor, b: Optional[torch.Tensor]) -> torch.Tensor:
    return y if b is None else y + b.float()[None]


def reconstruct_qkv_token(Pq, Pk, Pv, Vq, Vk, Vv, bq=None, bk=None, bv=None):
    """Headwise P: Q[b,h,:] = Pq[b,h,:] @ Vq[h]; fp32 accumulate, store in P dtype.
    kernels/attn/decode/densekv_reconstruct_triton.py:11-123,360-461."""
    dt = Pq.dtype
    Q = _bias(torch.einsum("bhr,hrd->bhd", Pq.float(), Vq.float()), bq).to(dt)
    K = _bias(torch.einsum("bhr,hrd->bhd", Pk.float(), Vk.float()), bk).to(dt)
    V = _bias(torch.einsum("bhr,hrd->bhd", Pv.float(), Vv.float()), bv).to(dt)
    return Q, K, V


def reconstruct_qkv_token_shared_hetero(Pq, Pk, Pv, Vq, Vk, Vv, bq=None, bk=None, bv=None):
    """Shared-rank P [B,R*] against per-head bases [H,R*,Dh], ranks may differ.
    kernels/attn/decode/densekv_reconstruct_triton.py:241-357,559-659."""
    dt = Pq.dtype
    Q = _bias(torch.einsum("br,hrd->bhd", Pq.float(), Vq.float()), bq).to(dt)
    K = _bias(torch.einsum("br,hrd->bhd", Pk.float(), Vk.float()), bk).to(dt)
    V = _bias(torch.einsum("br,hrd->bhd", Pv.float(), Vv.float()), bv).to(dt)
    return Q, K, V


def reconstruct_qkv_token_shared(Pq, Pk, Pv, Vq, Vk, Vv, bq=None, bk=None, bv=None):
    """Equal-rank case.  kernels/attn/decode/densekv_reconstruct_triton.py:126-238,464-556."""
    return reconstruct_qkv_token_shared_hetero(Pq, Pk, Pv, Vq, Vk, Vv, bq, bk, bv)


def pack_qkv_shared_bases(Vq, Vk, Vv):
    """[H,R,Dh] -> [R,H*Dh].  kernels/attn/decode/densekv_reconstruct_triton.py:662-690."""
    def flat(V):
        h, r, d = V.shape
        return V.permute(1, 0, 2).reshape(r, h * d).contiguous()
    return flat(Vq), flat(Vk), flat(Vv)


def reconstruct_qkv_token_shared_prepacked(Pq, Pk, Pv, Vq_flat, Vk_flat, Vv_flat, *, H, Hk, Dh,
                                           bq=None, bk=None, bv=None):
    """Q = Pq @ Vq_flat (rounded), then bias added in P dtype.
    kernels/attn/decode/densekv_reconstruct_triton.py:693-760."""
    B = Pq.shape[0]
    dt = Pq.dtype
    Q = (Pq.float() @ Vq_flat.float()).to(dt).reshape(B, H, Dh)
    K = (Pk.float() @ Vk_flat.float()).to(dt).reshape(B, Hk, Dh)
    V = (Pv.float() @ Vv_flat.float()).to(dt).reshape(B, Hk, Dh)
    if bq is not None:
        Q = Q + bq[None]
    if bk is not None:
        K = K + bk[None]
    if bv is not None:
        V = V + bv[None]
    return Q.contiguous(), K.contiguous(), V.contiguous()


# ----------------------------------------------------------------------------
# decode attention
# ----------------------------------------------------------------------------
def dense_decode_attn(q_bhd: torch.Tensor, k_blhd: torch.Tensor, v_blhd: torch.Tensor) -> torch.Tensor:
    """softmax(q K^T / sqrt(Dh)) V for one query token over L cached keys, GQA aware.

    q [B,H,Dh] (already rotated), k/v [B,L,Hk,Dh] (k already rotated) -> [B,H,Dh].
    benchmark/attn/decode_compare.py:569-583.
    """
    B, H, Dh = q_bhd.shape
    Hk = k_blhd.shape[2]
    rep = H // Hk
    q = q_bhd.float().reshape(B, Hk, rep, Dh)
    k = k_blhd.float().permute(0, 2, 1, 3)  # [B,Hk,L,Dh]
    v = v_blhd.float().permute(0, 2, 1, 3)
    scores = torch.einsum("bkgd,bkld->bkgl", q, k) * (1.0 / math.sqrt(Dh))
    p = torch.softmax(scores, dim=-1)
    out = torch.einsum("bkgl,bkld->bkgd", p, v)
    return out.reshape(B, H, Dh).to(q_bhd.dtype)


def flash_attn_with_kvcache(q, k_cache, v_cache, k=None, v=None, cache_seqlens=None,
                            rotary_cos=None, rotary_sin=None, causal=True,
                            rotary_interleaved=False, softmax_scale=None):
    """The call contract of flash-attn 2.8.3 ``flash_attn_with_kvcache`` as the reference
    uses it (runtime/attn/decode_registry.py:177-211), q_len == 1.

    q [B,1,H,Dh]; caches [B,S,Hk,Dh] (mutated in place); k,v [B,1,Hk,Dh];
    cache_seqlens int32 [B]; rotary_cos/sin [S', Dh/2].  q and k are rotated at position
    cache_seqlens[b] (non-interleaved), k/v are written at that position, attention runs
    over cache_seqlens[b]+1 keys.  Returns [B,1,H,Dh].
    """
    assert not rotary_interleaved and q.shape[1] == 1
    B, _, H, Dh = q.shape
    out = torch.empty_like(q)
    for b in range(B):
        n = int(cache_seqlens[b]) if cache_seqlens is not None else 0
        qb = q[b, 0]
        if k is not None:
            kb, vb = k[b, 0], v[b, 0]
            if rotary_cos is not None:
                kb = apply_rope_fp32(kb, rotary_cos[n], rotary_sin[n])
            k_cache[b, n] = kb
            v_cache[b, n] = vb
            n_keys = n + 1
        else:
            n_keys = n
        if rotary_cos is not None:
            qb = apply_rope_fp32(qb, rotary_cos[n], rotary_sin[n])
        o = dense_decode_attn(qb[None], k_cache[b:b + 1, :n_keys], v_cache[b:b + 1, :n_keys])
        out[b, 0] = o[0]
    return out


def rank_decode_attn(q_bhd, Pk_blr, Pv_blr, Vk_hrd, Vv_hrd, cos_half=None, sin_half=None, BN: int = 64):
    """Streaming decode over a rank-space KV cache, shared-rank layout.

    q [B,H,Dh] already rotated at its own position; Pk/Pv [B,L,R] pre-RoPE rank
    coefficients; Vk/Vv [Hk,R,Dh].  Per block of BN keys: K = Pk @ Vk[h] (fp32),
    rotate-half RoPE at absolute positions, online softmax, V = Pv @ Vv[h],
    out = acc / max(l, 1e-20).  benchmark/attn/decode_compare.py:675-750.
    """
    B, H, Dh = q_bhd.shape
    Hk = Vk_hrd.shape[0]
    rep = H // Hk
    L = Pk_blr.shape[1]
    half = Dh // 2
    scale = 1.0 / math.sqrt(Dh)
    q = q_bhd.float().reshape(B, Hk, rep, Dh)
    m_i = torch.full((B, Hk, rep), -float("inf"))
    l_i = torch.zeros((B, Hk, rep))
    acc = torch.zeros((B, Hk, rep, Dh))
    for n0 in range(0, L, BN):
        n1 = min(L, n0 + BN)
        Kb = torch.einsum("blr,krd->bkld", Pk_blr[:, n0:n1].float(), Vk_hrd.float())
        Vb = torch.einsum("blr,krd->bkld", Pv_blr[:, n0:n1].float(), Vv_hrd.float())
        if cos_half is not None:
            c = cos_half[n0:n1].float()[None, None]
            s = sin_half[n0:n1].float()[None, None]
            k0, k1 = Kb[..., :half], Kb[..., half:]
            Kb = torch.cat([k0 * c - k1 * s, k0 * s + k1 * c], dim=-1)
        scores = torch.einsum("bkgd,bknd->bkgn", q, Kb) * scale
        m_new = torch.maximum(m_i, scores.max(dim=-1).values)
        alpha = torch.exp(m_i - m_new)
        p = torch.exp(scores - m_new[..., None])
        l_i = l_i * alpha + p.sum(-1)
        acc = acc * alpha[..., None] + torch.einsum("bkgn,bknd->bkgd", p, Vb)
        m_i = m_new
    out = acc / l_i[..., None].clamp_min(1e-20)
    return out.reshape(B, H, Dh).to(q_bhd.dtype)


def rank_decode_attn_headwise(q_bhd, Pk_blhr, Pv_blhr, Vk_hrd, Vv_hrd, cos_half=None, sin_half=None, BN: int = 64):
    """Per-head rank coefficients Pk/Pv [B,L,Hk,R].  benchmark/attn/decode_compare.py:586-672."""
    B, H, Dh = q_bhd.shape
    Hk = Vk_hrd.shape[0]
    K = torch.einsum("blhr,hrd->blhd", Pk_blhr.float(), Vk_hrd.float())
    V = torch.einsum("blhr,hrd->blhd", Pv_blhr.float(), Vv_hrd.float())
    if cos_half is not None:
        K = apply_rope_fp32(K, cos_half[None, :, None, :], sin_half[None, :, None, :])
    return dense_decode_attn(q_bhd.float(), K, V).to(q_bhd.dtype)


# ----------------------------------------------------------------------------
# fused low-rank RoPE attention, full sequence (prefill)
# ----------------------------------------------------------------------------
def rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos_half, sin_half, *, bq=None, bk=None, bv=None,
                      pad_mask: Optional[torch.Tensor] = None,
                      add_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """O [B,M,H,dh] of the fused prefill kernel.  kernels/attn/prefill/rope_sdpa.py:67-248.

    Pq [B,H,M,R], Pk/Pv [B,Hk,M,R], V* [H|Hk,R,dh], cos/sin [M,dh/2] (or [B,M,dh/2]);
    q,k,v tiles are P @ V in fp32 (+bias), rotate-half RoPE with first-half angles
    (:185-189), causal (:195-197), scale 1/sqrt(dh) applied after the causal fill
    (:200), pad mask on keys / additive mask (:203-209), online softmax in fp32,
    fully masked rows give 0 (:244-246); output in P dtype.
    """
    B, H, M, R = Pq.shape
    Hk = Pk.shape[1]
    dh = Vq.shape[2]
    rep = H // Hk
    half = dh // 2
    q = torch.einsum("bhmr,hrd->bhmd", Pq.float(), Vq.float())
    k = torch.einsum("bhmr,hrd->bhmd", Pk.float(), Vk.float())
    v = torch.einsum("bhmr,hrd->bhmd", Pv.float(), Vv.float())
    if bq is not None:
        q = q + bq.float().reshape(1, H, 1, dh)
    # the kernel indexes bk/bv with the *query* head id (rope_sdpa.py:181-183,229-230)
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    if bk is not None:
        k = k + bk.float().reshape(1, -1, 1, dh)[:, :H]
    if bv is not None:
        v = v + bv.float().reshape(1, -1, 1, dh)[:, :H]
    c = cos_half.float()
    s = sin_half.float()
    if c.dim() == 2:
        c, s = c[None], s[None]
    c, s = c[:, None], s[:, None]  # [B|1,1,M,half]

    def rot(x):
        x0, x1 = x[..., :half], x[..., half:]
        return torch.cat([x0 * c - x1 * s, x0 * s + x1 * c], dim=-1)

    q, k = rot(q), rot(k)
    scores = torch.einsum("bhmd,bhnd->bhmn", q, k)
    causal = torch.ones(M, M, dtype=torch.bool).tril()
    scores = scores.masked_fill(~causal, -float("inf")) * (1.0 / math.sqrt(dh))
    if pad_mask is not None:
        scores = scores.masked_fill(~pad_mask.bool()[:, None, None, :], -float("inf"))
    if add_mask is not None:
        scores = scores + add_mask.float().reshape(B, 1, M, M)
    m = scores.max(dim=-1, keepdim=True).values
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    p = torch.exp(scores - m)
    l = p.sum(-1, keepdim=True)
    o = torch.einsum("bhmn,bhnd->bhmd", p, v) / torch.where(l > 0, l, torch.ones_like(l))
    o = torch.where(l > 0, o, torch.zeros_like(o))
    return o.permute(0, 2, 1, 3).contiguous().to(Pq.dtype)


# ----------------------------------------------------------------------------
# dual-split low-rank SwiGLU MLP (reference kernel-level API)
# ----------------------------------------------------------------------------
def dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2=None, *, BD: Optional[int] = None,
                   variant: str = "v2", work_dtype: Optional[torch.dtype] = None):
    """Y = ((silu(PGate@GateU) * (PUp@UpU)) @ DownV) @ DownU (+ b2).

    PUp/PGate [B,L,R]; GateU/UpU [R,D]; DownV [D,R]; DownU [R,Hd].
    Rounding points of the Triton kernels: g,u stay fp32; h is rounded to the input
    dtype (kernels/mlp/decode/dual_split_triton.py:207); per-D-tile partials of
    h@DownV are fp32 and summed (v1: through a workspace of ``work_dtype`` then
    ``.sum(1)`` :586-622; v2: fp32 atomics :311); S is rounded to the input dtype
    before the DownU GEMM (:719-721); b2 is added inside the GEMM (addmm).
    ``BD`` only changes the summation grouping.
    """
    dt = PUp.dtype
    B, L, R = PUp.shape
    T = B * L
    D = GateU.shape[1]
    pu = PUp.reshape(T, R).float()
    pg = PGate.reshape(T, R).float()
    g = pg @ GateU.float()
    u = pu @ UpU.float()
    h = ((g * torch.sigmoid(g)) * u).to(dt).float()
    if BD is None:
        S = h @ DownV.float()
    else:
        parts = [h[:, d0:d0 + BD] @ DownV[d0:d0 + BD].float() for d0 in range(0, D, BD)]
        if variant == "v1" and work_dtype is not None:
            work = torch.stack([p.to(work_dtype) for p in parts], dim=1)
            S = work.sum(dim=1).float()
        else:
            S = torch.stack(parts, dim=1).sum(dim=1)
    S = S.to(dt)
    Y = S.float() @ DownU.float()
    if b2 is not None:
        Y = Y + b2.float()
    return Y.to(dt).reshape(B, L, DownU.shape[1])


def dual_split_mlp_pcat(PCat, GateU, UpU, DownV, DownU, b2=None):
    """Packed input PCat[..., :R] = PUp, PCat[..., R:] = PGate.
    kernels/mlp/decode/dual_split_triton_pcat_s.py:81-90,123-218."""
    R = PCat.shape[-1] // 2
    return dual_split_mlp(PCat[..., :R], PCat[..., R:], GateU, UpU, DownV, DownU, b2)


def dual_split_mlp_v3(PUp, PGate, GateU, UpU, DownV, DownU, b2=None, *, BD: int = 128, BR2: int = 128):
    """v3 fuses DownU: per D-tile and per BR2 slice, s = h@DownV is rounded to the input
    dtype before being multiplied by DownU; partial Y's are summed in fp32 and rounded
    once; b2 added afterwards in the input dtype.
    kernels/mlp/decode/dual_split_triton.py:427-532,858-966."""
    dt = PUp.dtype
    B, L, R = PUp.shape
    T = B * L
    D = GateU.shape[1]
    g = PGate.reshape(T, R).float() @ GateU.float()
    u = PUp.reshape(T, R).float() @ UpU.float()
    h = ((g * torch.sigmoid(g)) * u).to(dt).float()
    Y = torch.zeros(T, DownU.shape[1])
    for d0 in range(0, D, BD):
        for r0 in range(0, R, BR2):
            s = (h[:, d0:d0 + BD] @ DownV[d0:d0 + BD, r0:r0 + BR2].float()).to(dt).float()
            Y += s @ DownU[r0:r0 + BR2].float()
    Y = Y.to(dt)
    if b2 is not None:
        Y = Y + b2
    return Y.reshape(B, L, -1)


# ----------------------------------------------------------------------------
# one low-rank Llama block and the model around it
# ----------------------------------------------------------------------------
@dataclass
class BlockWeights:
    """nn.Linear-layout factors: *_v [R,in] applied first, *_u [out,R]."""
    q_v: torch.Tensor; q_u: torch.Tensor
    k_v: torch.Tensor; k_u: torch.Tensor
    v_v: torch.Tensor; v_u: torch.Tensor
    o_v: torch.Tensor; o_u: torch.Tensor
    gate_v: torch.Tensor; gate_u: torch.Tensor
    up_v: torch.Tensor; up_u: torch.Tensor
    down_v: torch.Tensor; down_u: torch.Tensor
    ln1: torch.Tensor; ln2: torch.Tensor


@dataclass
class ModelWeights:
    embed: torch.Tensor            # [vocab, d]
    blocks: list
    norm: torch.Tensor             # [d]
    lm_head: torch.Tensor          # [vocab, d]
    n_heads: int
    n_kv_heads: int
    head_dim: int
    rope_theta: float = 10000.0
    eps: float = 1e-6
    meta: dict = field(default_factory=dict)


def make_model(*, d: int, n_heads: int, n_kv_heads: int, head_dim: int, ffn: int, attn_rank: int,
               mlp_rank: int, n_layers: int, vocab: int, dtype: torch.dtype, seed: int = 0,
               std: float = 0.02, theta: float = 10000.0) -> ModelWeights:
    """Seeded synthetic weights.  Draw order under ``torch.manual_seed(seed)`` on the CPU
    generator, all fp32 N(0, std) then cast: embed; per layer q_v,q_u,k_v,k_u,v_v,v_u,o_v,
    o_u,gate_v,gate_u,up_v,up_u,down_v,down_u; lm_head (separate matrix, not tied).
    RMSNorm weights are 1; a final RMSNorm is present."""
    g = torch.Generator().manual_seed(seed)

    def rn(*shape):
        return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(dtype)

    embed = rn(vocab, d)
    blocks = []
    qd, kvd = n_heads * head_dim, n_kv_heads * head_dim
    for _ in range(n_layers):
        blocks.append(BlockWeights(
            q_v=rn(attn_rank, d), q_u=rn(qd, attn_rank),
            k_v=rn(attn_rank, d), k_u=rn(kvd, attn_rank),
            v_v=rn(attn_rank, d), v_u=rn(kvd, attn_rank),
            o_v=rn(attn_rank, qd), o_u=rn(d, attn_rank),
            gate_v=rn(mlp_rank, d), gate_u=rn(ffn, mlp_rank),
            up_v=rn(mlp_rank, d), up_u=rn(ffn, mlp_rank),
            down_v=rn(mlp_rank, ffn), down_u=rn(d, mlp_rank),
            ln1=torch.ones(d, dtype=dtype), ln2=torch.ones(d, dtype=dtype)))
    lm_head = rn(vocab, d)
    return ModelWeights(embed=embed, blocks=blocks, norm=torch.ones(d, dtype=dtype), lm_head=lm_head,
                        n_heads=n_heads, n_kv_heads=n_kv_heads, head_dim=head_dim, rope_theta=theta,
                        meta=dict(d=d, ffn=ffn, attn_rank=attn_rank, mlp_rank=mlp_rank, vocab=vocab,
                                  n_layers=n_layers, seed=seed, std=std))


def hold_weights_as(mw: ModelWeights, dtype: torch.dtype) -> ModelWeights:
    """The same model with every factor and the lm_head held in ``dtype`` (values unchanged: widening bf16 is exact).
    The embedding and the norm weights keep their dtype, which is what names the activation dtype.  Results are
    bit-identical to those of ``mw``; the per-call widening of every weight is what goes away (decode steps of a deep
    model are several times faster on the host)."""
    import dataclasses
    blocks = [BlockWeights(**{f.name: (getattr(b, f.name) if f.name in ("ln1", "ln2") else getattr(b, f.name).to(dtype))
                              for f in dataclasses.fields(BlockWeights)}) for b in mw.blocks]
    return dataclasses.replace(mw, blocks=blocks, lm_head=mw.lm_head.to(dtype))


def mlp_forward(bw: BlockWeights, h2: torch.Tensor) -> torch.Tensor:
    """Chain-of-linears SwiGLU: down(silu(gate(x)) * up(x)), every op rounded in dtype.
    src/legacy/FlashSVD-V1/decoders/llama/profile_asvd_llama_decode.py:311-314."""
    g = lowrank_pair(h2, bw.gate_v, bw.gate_u)
    u = lowrank_pair(h2, bw.up_v, bw.up_u)
    return lowrank_pair(F.silu(g) * u, bw.down_v, bw.down_u)


def _attend(q, k, v, q_pos0: int) -> torch.Tensor:
    """q [B,T,H,Dh] at absolute positions q_pos0.., k/v [B,Lk,Hk,Dh] -> [B,T,H*Dh]; causal."""
    B, T, H, Dh = q.shape
    Lk, Hk = k.shape[1], k.shape[2]
    rep = H // Hk
    ct = _ct(q)
    qf = q.to(ct).permute(0, 2, 1, 3).reshape(B, Hk, rep, T, Dh)
    kf = k.to(ct).permute(0, 2, 1, 3)
    vf = v.to(ct).permute(0, 2, 1, 3)
    scores = torch.einsum("bkgtd,bkld->bkgtl", qf, kf) * (1.0 / math.sqrt(Dh))
    qpos = torch.arange(T)[:, None] + q_pos0
    kpos = torch.arange(Lk)[None, :]
    scores = scores.masked_fill(~(kpos <= qpos), -float("inf"))
    p = torch.softmax(scores, dim=-1)
    o = torch.einsum("bkgtl,bkld->bkgtd", p, vf)
    return o.reshape(B, H, T, Dh).permute(0, 2, 1, 3).reshape(B, T, H * Dh).to(q.dtype)


class DenseCache:
    """Per layer K (post-RoPE) and V, [B,S,Hk,Dh].  runtime/cache/attn_dense_kv.py:7-357."""

    def __init__(self, mw: ModelWeights, batch: int, max_len: int, dtype):
        n = len(mw.blocks)
        self.k = [torch.zeros(batch, max_len, mw.n_kv_heads, mw.head_dim, dtype=dtype) for _ in range(n)]
        self.v = [torch.zeros(batch, max_len, mw.n_kv_heads, mw.head_dim, dtype=dtype) for _ in range(n)]


class RankCache:
    """Per layer pre-RoPE Pk, Pv [B,S,R].  runtime/cache/attn_legacy_sparse_kv.py:22-182."""

    def __init__(self, mw: ModelWeights, batch: int, max_len: int, dtype):
        self.pk = [torch.zeros(batch, max_len, b.k_v.shape[0], dtype=dtype) for b in mw.blocks]
        self.pv = [torch.zeros(batch, max_len, b.v_v.shape[0], dtype=dtype) for b in mw.blocks]


def block_forward(mw: ModelWeights, li: int, x: torch.Tensor, pos0: int, cache, cos, sin) -> torch.Tensor:
    """x [B,T,d] at absolute positions pos0..pos0+T-1; the cache already holds pos0 earlier
    tokens and is extended in place.  Pre-norm block: x + o_u(o_v(attn(...))) then x + down(swiglu(...)); op order of an HF
    LlamaDecoderLayer with factored linears (utils/model_utils.py:586-671)."""
    bw = mw.blocks[li]
    B, T, d = x.shape
    H, Hk, Dh = mw.n_heads, mw.n_kv_heads, mw.head_dim
    h1 = rms_norm(x, bw.ln1, mw.eps)
    q = lowrank_pair(h1, bw.q_v, bw.q_u).reshape(B, T, H, Dh)
    c = cos[pos0:pos0 + T][None, :, None, :]
    s = sin[pos0:pos0 + T][None, :, None, :]
    q = apply_rope(q, c, s)
    L = pos0 + T
    if isinstance(cache, RankCache):
        cache.pk[li][:B, pos0:L] = lin(h1, bw.k_v)
        cache.pv[li][:B, pos0:L] = lin(h1, bw.v_v)
        k = lin(cache.pk[li][:B, :L], bw.k_u).reshape(B, L, Hk, Dh)
        v = lin(cache.pv[li][:B, :L], bw.v_u).reshape(B, L, Hk, Dh)
        k = apply_rope(k, cos[:L][None, :, None, :], sin[:L][None, :, None, :])
    else:
        k_new = lowrank_pair(h1, bw.k_v, bw.k_u).reshape(B, T, Hk, Dh)
        v_new = lowrank_pair(h1, bw.v_v, bw.v_u).reshape(B, T, Hk, Dh)
        k_new = apply_rope(k_new, c, s)
        if cache is not None:
            cache.k[li][:B, pos0:L] = k_new
            cache.v[li][:B, pos0:L] = v_new
            k, v = cache.k[li][:B, :L], cache.v[li][:B, :L]
        else:
            assert pos0 == 0
            k, v = k_new, v_new
    attn = _attend(q, k, v, pos0)
    x2 = x + lowrank_pair(attn, bw.o_v, bw.o_u)
    h2 = rms_norm(x2, bw.ln2, mw.eps)
    return x2 + mlp_forward(bw, h2)


def model_forward(mw: ModelWeights, ids: torch.Tensor, pos0: int = 0, cache=None,
                  cos=None, sin=None, last_only: bool = True, return_hidden: bool = False,
                  act_dtype: Optional[torch.dtype] = None, layer_inputs: Optional[list] = None):
    """embed -> blocks -> final RMSNorm -> lm_head.  utils/evaluator.py:50-82.

    ``act_dtype`` (fp32 / fp64) runs the exact mode: the stored weights and rotation tables as they are,
    activations and caches in ``act_dtype``, no rounding between operators.  ``layer_inputs``, if a list,
    receives the input of every block and, last, the output of the final block."""
    dtype = mw.embed.dtype
    if cos is None:
        cos, sin = rope_tables(pos0 + ids.shape[1], mw.head_dim, mw.rope_theta, dtype)
    x = mw.embed[ids]
    if act_dtype is not None:
        x = x.to(act_dtype)
    for li in range(len(mw.blocks)):
        if layer_inputs is not None:
            layer_inputs.append(x)
        x = block_forward(mw, li, x, pos0, cache, cos, sin)
    if layer_inputs is not None:
        layer_inputs.append(x)
    hidden = x
    xn = rms_norm(x[:, -1:] if last_only else x, mw.norm, mw.eps)
    logits = lin(xn, mw.lm_head)
    return (logits, hidden) if return_hidden else logits


def greedy_decode(mw: ModelWeights, prompt: torch.Tensor, n_new: int, cache_kind: str = "dense",
                  return_hidden: bool = False, return_logits: bool = False,
                  act_dtype: Optional[torch.dtype] = None, forced: Optional[torch.Tensor] = None,
                  layer_trace: Optional[list] = None):
    """Prefill yields token 0; each later token is one decode forward at
    cache_position = prompt_len + step.  scripts/demo_support/api.py:285-312,
    benchmark/decode/check_flashsvd_decode_correctness.py:277-322.

    ``act_dtype``: exact mode (see model_forward).  ``forced`` [B, n_new]: teacher forcing — the token fed
    at step s is ``forced[:, s-1]`` instead of this run's own argmax (the teacher-forced protocol of
    check_flashsvd_decode_correctness.py:220-265).  ``layer_trace``, if a list, receives per decode step the
    list of block inputs (+ the last block's output) of that step."""
    dtype = mw.embed.dtype
    B, Lp = prompt.shape
    max_len = Lp + n_new + 4
    cache = (RankCache if cache_kind == "rank" else DenseCache)(mw, B, max_len, act_dtype or dtype)
    cos, sin = rope_tables(max_len, mw.head_dim, mw.rope_theta, dtype)
    logits, hid = model_forward(mw, prompt, 0, cache, cos, sin, return_hidden=True, act_dtype=act_dtype)
    hiddens = [hid[:, -1]]
    all_logits = [logits[:, -1]]
    tok = logits[:, -1].float().argmax(-1, keepdim=True)
    toks = [tok]
    for step in range(n_new - 1):
        feed = tok if forced is None else forced[:, step:step + 1]
        li = [] if layer_trace is not None else None
        logits, hid = model_forward(mw, feed, Lp + step, cache, cos, sin, return_hidden=True, act_dtype=act_dtype,
                                    layer_inputs=li)
        if layer_trace is not None:
            layer_trace.append(li)
        hiddens.append(hid[:, -1])
        all_logits.append(logits[:, -1])
        tok = logits[:, -1].float().argmax(-1, keepdim=True)
        toks.append(tok)
    out = torch.cat(toks, dim=1)
    if return_logits:
        return out, torch.stack(hiddens, dim=1), cache, torch.stack(all_logits, dim=1)
    return (out, torch.stack(hiddens, dim=1), cache) if return_hidden else out


# ----------------------------------------------------------------------------
# group-wise int4 / int8 weights (src/quant/packed_quant_linear.py)
# ----------------------------------------------------------------------------
def pack_int4(q: torch.Tensor) -> torch.Tensor:
    """[N, K] values 0..15 -> [N, ceil(K/2)] bytes, even column in the low nibble.
    src/quant/packed_quant_linear.py:18-26."""
    q = q.to(torch.uint8)
    if q.shape[1] % 2:
        q = torch.cat([q, torch.zeros((q.shape[0], 1), dtype=torch.uint8)], dim=1)
    return (q[:, 0::2] & 0x0F) | ((q[:, 1::2] & 0x0F) << 4)


def unpack_int4(packed: torch.Tensor, in_features: int) -> torch.Tensor:
    """src/quant/packed_quant_linear.py:29-36."""
    out = torch.empty((packed.shape[0], packed.shape[1] * 2), dtype=torch.uint8)
    out[:, 0::2] = packed & 0x0F
    out[:, 1::2] = (packed >> 4) & 0x0F
    return out[:, :in_features]


def quantize_weight(weight: torch.Tensor, *, bits: int = 4, group_size: int = 128, sym: bool = False):
    """Min/max group quantisation of an nn.Linear weight [N, K] along K.
    Returns (qweight uint8 [N, K/2] for 4 bits or [N, K] for 8, scales fp16 [N, G], zeros int16 [N, G]);
    w ~= scale * (q - zero).  An all-zero group is given the range [-1, 1]; ``sym`` centres the range and fixes
    zero = 2^(bits-1).  src/quant/packed_quant_linear.py:126-172."""
    w = weight.detach().to(torch.float32)
    N, K = w.shape
    group = K if group_size <= 0 else int(group_size)
    maxq = float((1 << bits) - 1)
    qs, ss, zs = [], [], []
    for g0 in range(0, K, group):
        chunk = w[:, g0:min(K, g0 + group)]
        xmin, xmax = chunk.min(dim=1).values, chunk.max(dim=1).values
        if sym:
            xmax = torch.maximum(xmax.abs(), xmin.abs())
            xmin = -xmax
        dead = (xmin == 0) & (xmax == 0)
        xmin = torch.where(dead, torch.full_like(xmin, -1.0), xmin)
        xmax = torch.where(dead, torch.full_like(xmax, 1.0), xmax)
        scale = (xmax - xmin) / maxq
        scale = torch.where(scale == 0, torch.ones_like(scale), scale)
        zero = torch.full_like(scale, int((maxq + 1) / 2)) if sym else torch.round(-xmin / scale)
        qs.append(torch.clamp(torch.round(chunk / scale.unsqueeze(1)) + zero.unsqueeze(1), 0, maxq).to(torch.uint8))
        ss.append(scale.to(torch.float16))
        zs.append(zero.to(torch.int16))
    q = torch.cat(qs, dim=1).contiguous()
    return (pack_int4(q) if bits == 4 else q), torch.stack(ss, dim=1).contiguous(), torch.stack(zs, dim=1).contiguous()


def dequantize_weight(qweight, scales, zeros, *, in_features: int, bits: int = 4, group_size: int = 128,
                      dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """scale * (q - zero) in fp32, then ONE rounding to ``dtype``.  src/quant/packed_quant_linear.py:284-299."""
    q = (unpack_int4(qweight, in_features) if bits == 4 else qweight).to(torch.float32)
    group = in_features if group_size <= 0 else int(group_size)
    cols = []
    for gi in range(scales.shape[1]):
        g0, g1 = gi * group, min(in_features, (gi + 1) * group)
        cols.append(scales[:, gi].float().unsqueeze(1) * (q[:, g0:g1] - zeros[:, gi].float().unsqueeze(1)))
    return torch.cat(cols, dim=1).to(dtype)


def quant_linear(x, qweight, scales, zeros, bias=None, *, bits: int = 4, group_size: int = 128) -> torch.Tensor:
    """The module's reference forward: dequantise to the activation dtype, then an ordinary linear.
    src/quant/packed_quant_linear.py:301-312."""
    w = dequantize_weight(qweight, scales, zeros, in_features=x.shape[-1], bits=bits, group_size=group_size, dtype=x.dtype)
    return lin(x, w, bias)


# ----------------------------------------------------------------------------
# the synthetic configurations the benchmark contract names
# ----------------------------------------------------------------------------
def config_c1(dtype=torch.float32):
    """One Llama-style low-rank block, d=512, 8x64 heads, ffn 1376, attention rank 128,
    MLP rank 256, vocab 32000, seed 0; prompt = 128 ids from a second generator seeded 1."""
    mw = make_model(d=512, n_heads=8, n_kv_heads=8, head_dim=64, ffn=1376, attn_rank=128, mlp_rank=256,
                    n_layers=1, vocab=32000, dtype=dtype, seed=0)
    prompt = torch.randint(0, 32000, (1, 128), generator=torch.Generator().manual_seed(1))
    return mw, prompt
