"""Low-rank Llama modules on top of libflashsvd_hip.

The reference keeps these classes in ``models/llama.py``, which is not part of its checkout;
their surface is reconstructed from the callers (utils/model_utils.py:409-464,586-671,
benchmark/attn/bench_real_checkpoint_decode_reconstruct.py:90-180,
benchmark/attn/generate_dense_decode_plan.py:196-256,
benchmark/mlp/bench_svd_llama_decode_graph.py:88-200).  Every dense ``W[out,in]`` is held as
``v_proj: in->R`` (weight [R,in], applied first) and ``u_proj: R->out`` (weight [out,R]).

Arithmetic contract: bf16 storage, fp32 accumulation, one rounding after every linear,
RMSNorm, rotary op and SwiGLU op — what a chain of bf16 ``nn.Linear`` modules computes.
All compute goes through the HIP library; a module asked to run on CPU tensors raises.
"""
from __future__ import annotations

import os
from types import SimpleNamespace
from typing import Optional

import torch
from torch import nn

from . import hip_ops
from .runtime.cache import FlashSVDLegacySparseKVCache, FlashSVDV15DenseKVCache

_TRUE = {"1", "true", "yes", "y", "on"}
# set by api.enable_flashsvd_llama_layer_tail_cuda_graph(); read at call time together with the env flags
LAYER_TAIL_GRAPH_ENABLED = False


def _env_truthy(name: str) -> bool:
    return os.getenv(name, "").strip().lower() in _TRUE


def lowrank_rank(out_features: int, in_features: int, ratio: float) -> int:
    """Rank that keeps ``ratio`` of the dense parameter count: int(out*in*ratio/(out+in)).
    src/methods/svdllm/SVDLLM_flashsvd.py:286."""
    return int(out_features * in_features * float(ratio) / (out_features + in_features))


def _require_gpu(t: torch.Tensor, who: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{who} runs only on a GPU through libflashsvd_hip (got a {t.device} tensor); "
                           "there is no CPU path in this package")
    if t.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError(f"{who} computes in bfloat16 or float16, got {t.dtype}")


class LlamaRMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)
        self.variance_epsilon = float(eps)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        _require_gpu(hidden_states, "LlamaRMSNorm")
        return hip_ops.rmsnorm(hidden_states, self.weight, self.variance_epsilon)


class LlamaRotaryEmbedding(nn.Module):
    """Rotary tables with the legacy call forms the fused prefill wrapper accepts:
    ``forward(x, position_ids)`` -> cos,sin [B,T,Dh] and ``forward(x, seq_len=)`` -> [1,1,T,Dh]
    (kernels/attn/prefill/rope_sdpa.py:317-339)."""

    def __init__(self, head_dim: int, max_position_embeddings: int = 4096, base: float = 10000.0, device=None):
        super().__init__()
        self.dim = int(head_dim)
        self.max_position_embeddings = int(max_position_embeddings)
        self.base = float(base)
        half = self.dim // 2
        inv_freq = 1.0 / (self.base ** (torch.arange(0, half, dtype=torch.float32, device=device) / half))
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    @torch.no_grad()
    def forward(self, x: torch.Tensor, position_ids: Optional[torch.Tensor] = None, seq_len: Optional[int] = None):
        if position_ids is None:
            n = int(seq_len if seq_len is not None else x.shape[-2])
            ang = torch.arange(n, device=x.device, dtype=torch.float32)[:, None] * self.inv_freq.to(x.device)[None, :]
            emb = torch.cat((ang, ang), dim=-1)
            return emb.cos()[None, None].to(x.dtype), emb.sin()[None, None].to(x.dtype)
        ang = position_ids.to(torch.float32)[..., None] * self.inv_freq.to(position_ids.device)
        emb = torch.cat((ang, ang), dim=-1)
        return emb.cos().to(x.dtype), emb.sin().to(x.dtype)


def _packed_rows(mods: list[nn.Linear]) -> torch.Tensor:
    """One [sum(R_i), in] buffer whose row slices replace the modules' weights (no duplicate copy)."""
    ws = [m.weight.data for m in mods]
    base = ws[0]
    row = 0
    contiguous_already = True
    for w in ws:
        if w.untyped_storage().data_ptr() != base.untyped_storage().data_ptr() or \
                w.storage_offset() != base.storage_offset() + row * base.shape[1] or not w.is_contiguous():
            contiguous_already = False
            break
        row += w.shape[0]
    if contiguous_already:
        return torch.as_strided(base, (row, base.shape[1]), (base.shape[1], 1), base.storage_offset())
    packed = torch.cat(ws, dim=0).contiguous()
    row = 0
    for m in mods:
        r = m.weight.shape[0]
        m.weight.data = packed[row:row + r]
        row += r
    return packed


class SVD_LlamaAttention(nn.Module):
    """Low-rank attention: q/k/v/o each as v_proj (in->R) then u_proj (R->out)."""

    def __init__(self, config=None, ratio: float = 1.0, layer_idx: int = 0, ranks: Optional[dict] = None):
        super().__init__()
        self.config = config
        self.layer_idx = int(layer_idx)
        self.hidden_size = int(config.hidden_size)
        self.num_heads = int(config.num_attention_heads)
        self.num_key_value_heads = int(getattr(config, "num_key_value_heads", None) or self.num_heads)
        self.head_dim = int(getattr(config, "head_dim", None) or self.hidden_size // self.num_heads)
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.max_position_embeddings = int(getattr(config, "max_position_embeddings", 4096))
        self.ratio = float(ratio)
        qd, kvd, d = self.num_heads * self.head_dim, self.num_key_value_heads * self.head_dim, self.hidden_size
        ranks = dict(ranks or {})
        rq = int(ranks.get("q", lowrank_rank(qd, d, ratio)))
        rk = int(ranks.get("k", lowrank_rank(kvd, d, ratio)))
        rv = int(ranks.get("v", lowrank_rank(kvd, d, ratio)))
        ro = int(ranks.get("o", lowrank_rank(d, qd, ratio)))
        self.low_rank = rk
        self.use_lowrank_cache = bool(getattr(config, "flash_svd_use_lowrank_cache", False))
        self.q_v_proj = nn.Linear(d, rq, bias=False)
        self.q_u_proj = nn.Linear(rq, qd, bias=False)
        self.k_v_proj = nn.Linear(d, rk, bias=False)
        self.k_u_proj = nn.Linear(rk, kvd, bias=False)
        self.v_v_proj = nn.Linear(d, rv, bias=False)
        self.v_u_proj = nn.Linear(rv, kvd, bias=False)
        self.o_v_proj = nn.Linear(qd, ro, bias=False)
        self.o_u_proj = nn.Linear(ro, d, bias=False)
        self.rotary_emb = LlamaRotaryEmbedding(self.head_dim, self.max_position_embeddings,
                                               float(getattr(config, "rope_theta", 10000.0)))
        self._reset_runtime_state()

    # ---- runtime state (derived tensors, rebuilt lazily) -----------------------------------
    def _reset_runtime_state(self) -> None:
        self._decode_Vq = self._decode_Vk = self._decode_Vv = None
        self._decode_ptrs = None
        self._dense_decode_prepacked_cache: dict = {}
        self._dense_decode_backend_cache: dict = {}
        self._packed_qkv_v = None

    def _factor_modules(self):
        return (self.q_v_proj, self.q_u_proj, self.k_v_proj, self.k_u_proj, self.v_v_proj, self.v_u_proj, self.o_v_proj,
                self.o_u_proj)

    def _ensure_runtime_state(self) -> None:
        """Idempotent.  Packs [q_v; k_v; v_v] into one row-contiguous buffer (the module weights
        become views of it) so the three rank projections are a single weight stream."""
        for name in ("_decode_Vq", "_decode_Vk", "_decode_Vv", "_decode_ptrs", "_packed_qkv_v"):
            if not hasattr(self, name):
                setattr(self, name, None)
        for name in ("_dense_decode_prepacked_cache", "_dense_decode_backend_cache"):
            if not isinstance(getattr(self, name, None), dict):
                setattr(self, name, {})
        from .quant import is_quantized, pack_quant_rows
        if is_quantized(*self._factor_modules()):
            # int4 factors: the three rank projections share their input, so their rows are packed into one stream
            mods = [self.q_v_proj, self.k_v_proj, self.v_v_proj]
            key = tuple(m.qweight.data_ptr() if is_quantized(m) else m.weight.data_ptr() for m in mods)
            if getattr(self, "_q4_key", None) != key:
                self._q4_qkv_v = pack_quant_rows(mods)
                self._q4_key = tuple(m.qweight.data_ptr() if is_quantized(m) else m.weight.data_ptr() for m in mods)
            return
        mods = [self.q_v_proj, self.k_v_proj, self.v_v_proj]
        key = tuple((m.weight.data_ptr(), m.weight.dtype, m.weight.device) for m in mods)
        if self._packed_qkv_v is None or self._decode_ptrs != key:
            self._packed_qkv_v = _packed_rows(mods)
            self._decode_ptrs = tuple((m.weight.data_ptr(), m.weight.dtype, m.weight.device) for m in mods)
            self._decode_Vq = self._decode_Vk = self._decode_Vv = None
            self._dense_decode_prepacked_cache.clear()

    def _qkv_rank_tuple(self) -> tuple[int, int, int]:
        return (int(self.q_v_proj.out_features), int(self.k_v_proj.out_features), int(self.v_v_proj.out_features))

    def _get_decode_factors(self):
        """(Vq [H,Rq,Dh], Vk [Hk,Rk,Dh], Vv [Hk,Rv,Dh]): u_proj.weight [H*Dh,R] viewed [H,Dh,R] and
        transposed — the per-head bases of the reference's reconstruct kernels."""
        self._ensure_runtime_state()
        if self._decode_Vq is None:
            def basis(lin: nn.Linear, heads: int) -> torch.Tensor:
                return lin.weight.data.view(heads, self.head_dim, -1).transpose(1, 2).contiguous()
            self._decode_Vq = basis(self.q_u_proj, self.num_heads)
            self._decode_Vk = basis(self.k_u_proj, self.num_key_value_heads)
            self._decode_Vv = basis(self.v_u_proj, self.num_key_value_heads)
        return self._decode_Vq, self._decode_Vk, self._decode_Vv

    def _get_dense_decode_tensors(self, device=None, dtype=None, past_key_value=None, cache_position=None):
        """(packed_qkv_rank [d, Rq+Rk+Rv], vq_flat [Rq,H*Dh], vk_flat [Rk,Hk*Dh], vv_flat [Rv,Hk*Dh],
        split_sizes) in the reference's x@W layouts, cached per (device, dtype).  Ranks are padded
        with zero rows/columns to FLASH_SVD_DENSE_DECODE_RANK_PAD_MULTIPLE when it is set."""
        self._ensure_runtime_state()
        w = self._packed_qkv_v
        device = w.device if device is None else torch.device(device)
        dtype = w.dtype if dtype is None else dtype
        try:
            mult = max(1, int(os.getenv("FLASH_SVD_DENSE_DECODE_RANK_PAD_MULTIPLE", "1") or "1"))
        except ValueError:
            mult = 1
        mode = os.getenv("FLASH_SVD_DENSE_DECODE_PAD_MODE", "independent").strip().lower()
        key = (str(device), dtype, mult, mode)
        hit = self._dense_decode_prepacked_cache.get(key)
        if hit is not None:
            return hit
        ranks = list(self._qkv_rank_tuple())
        padded = [(r + mult - 1) // mult * mult for r in ranks]
        if mode == "uniform_layer":
            padded = [max(padded)] * 3
        vs = [self.q_v_proj.weight.data, self.k_v_proj.weight.data, self.v_v_proj.weight.data]
        us = [self.q_u_proj.weight.data, self.k_u_proj.weight.data, self.v_u_proj.weight.data]
        cols, flats = [], []
        for v, u, r, rp in zip(vs, us, ranks, padded):
            vt = v.t().to(device=device, dtype=dtype)          # [d, R]
            ut = u.t().to(device=device, dtype=dtype)          # [R, out]
            if rp != r:
                vt = torch.cat([vt, vt.new_zeros(vt.shape[0], rp - r)], dim=1)
                ut = torch.cat([ut, ut.new_zeros(rp - r, ut.shape[1])], dim=0)
            cols.append(vt)
            flats.append(ut.contiguous())
        out = (torch.cat(cols, dim=1).contiguous(), flats[0], flats[1], flats[2], tuple(padded))
        self._dense_decode_prepacked_cache[key] = out
        return out

    # ---- decode ---------------------------------------------------------------------------------
    def _dense_decode_backend(self, cache=None) -> str:
        """"exact" or "packed" for the current token: the entry an applied decode plan holds for this layer
        (per bucket of cached keys, read from the cache's host-side count, so a captured graph keeps the
        choice it was captured with), else FLASH_SVD_DENSE_DECODE_BACKEND (auto = packed)."""
        entry = getattr(self, "_dense_decode_plan", None)
        if entry:
            from .plan import plan_choice
            past = None
            if cache is not None and isinstance(entry.get("buckets"), dict):
                past = int(cache.get_seq_length())
            return plan_choice(entry, past)
        raw = os.getenv("FLASH_SVD_DENSE_DECODE_BACKEND", "auto").strip().lower() or "auto"
        if raw not in ("auto", "exact", "packed"):
            raise ValueError(f"FLASH_SVD_DENSE_DECODE_BACKEND={raw!r}: expected auto, exact or packed")
        return "exact" if raw == "exact" else "packed"

    def _positions_for(self, cache, batch: int, cache_position, device) -> torch.Tensor:
        """int32 [B] device tensor holding the write position of the current token."""
        if isinstance(cache_position, torch.Tensor) and cache_position.is_cuda and cache_position.dtype == torch.int32 \
                and cache_position.numel() == batch and cache_position.is_contiguous():
            return cache_position
        buf = cache._seqlens_buffer(self.layer_idx, batch) if hasattr(cache, "_seqlens_buffer") else \
            torch.empty(batch, dtype=torch.int32, device=device)
        if cache_position is None:
            start = int(cache.get_seq_length())
        elif isinstance(cache_position, torch.Tensor):
            if cache_position.is_cuda:
                pos = cache_position.reshape(-1).to(torch.int32)
                buf.copy_(pos.expand(batch) if pos.numel() == 1 else pos[:batch])
                return buf
            start = int(cache_position.reshape(-1)[0])
        else:
            start = int(cache_position)
        if start < 0 or start + 1 > cache.max_cache_len:
            raise IndexError(f"{type(cache).__name__} write position out of range: start={start} q_len=1 "
                             f"max={cache.max_cache_len}")
        buf.fill_(start)
        return buf

    def decode_token(self, x: torch.Tensor, cache, positions: torch.Tensor, *, norm_weight=None, eps: float = 1e-6,
                     residual: Optional[torch.Tensor] = None, rope=None, attn_ws=None, nsplit: Optional[int] = None):
        """One token per batch row.  x [B,d]; ``norm_weight`` fuses the input RMSNorm; ``residual``
        is added to the output projection.  K/V of the token are appended to ``cache`` at
        ``positions`` (int32 [B], device) and attention runs over positions+1 keys."""
        self._ensure_runtime_state()
        B = x.shape[0]
        H, Hk, Dh = self.num_heads, self.num_key_value_heads, self.head_dim
        if isinstance(cache, FlashSVDLegacySparseKVCache):
            return self._decode_token_rank(x, cache, positions, norm_weight=norm_weight, eps=eps, residual=residual, rope=rope)
        if not isinstance(cache, FlashSVDV15DenseKVCache):
            raise TypeError(f"decode needs a FlashSVDV15DenseKVCache or FlashSVDLegacySparseKVCache, got {type(cache).__name__}")
        cache._ensure_layer_spec(self.layer_idx, h=Hk, dh=Dh)
        kc, vc = cache.key_cache[self.layer_idx], cache.value_cache[self.layer_idx]
        if rope is None:
            rope = cache.get_rope_tables(seqlen=cache.max_cache_len, head_dim=Dh, device=x.device, dtype=x.dtype)
        if nsplit is None:
            nsplit = hip_ops.pick_nsplit(cache.max_cache_len, B, H, Dh)
        from .quant import apply_linear, is_quantized
        quantized = is_quantized(*self._factor_modules())
        if quantized or self._dense_decode_backend(cache) == "exact":
            # module by module: three rank projections, three head expansions, rotary + append inside attention
            # (the only form for int4 factors, whose bytes cannot be row-packed with their neighbours')
            pk = getattr(self, "_q4_qkv_v", None) if quantized else None
            if pk is not None and self.q_v_proj.streams_int4(B):
                rq, rk, rv = self._qkv_rank_tuple()
                p = hip_ops.linear_q4(x, *pk, group_size=self.q_v_proj.group_size, norm_weight=norm_weight, eps=eps)
                pq, pkk, pv = p[:, :rq], p[:, rq:rq + rk], p[:, rq + rk:]
            else:
                xn = x if norm_weight is None else hip_ops.rmsnorm(x, norm_weight, eps)
                pq, pkk, pv = (apply_linear(m, xn) for m in (self.q_v_proj, self.k_v_proj, self.v_v_proj))
            q = apply_linear(self.q_u_proj, pq).view(B, H, Dh)
            k = apply_linear(self.k_u_proj, pkk).view(B, Hk, Dh)
            v = apply_linear(self.v_u_proj, pv).view(B, Hk, Dh)
            a = hip_ops.attn_decode_densekv(q, kc[:B], vc[:B], positions, k_new=k, v_new=v, cos=rope[0], sin=rope[1],
                                            nsplit=nsplit, workspace=attn_ws)
            cache._layer_initialized[self.layer_idx] = True
            po = apply_linear(self.o_v_proj, a.view(B, H * Dh))
            return apply_linear(self.o_u_proj, po, residual=residual)
        else:
            p = hip_ops.linear(x, self._packed_qkv_v, norm_weight=norm_weight, eps=eps)
            q = hip_ops.qkv_rope_append(p, self.q_u_proj.weight, self.k_u_proj.weight, self.v_u_proj.weight, rope[0], rope[1],
                                        positions, kc[:B], vc[:B], num_heads=H, num_kv_heads=Hk, head_dim=Dh)
            cache._layer_initialized[self.layer_idx] = True
            a = hip_ops.attn_decode_densekv(q, kc[:B], vc[:B], positions, seqlen_add=1, nsplit=nsplit, workspace=attn_ws)
        po = hip_ops.linear(a.view(B, H * Dh), self.o_v_proj.weight)
        return hip_ops.linear(po, self.o_u_proj.weight, residual=residual)

    def _decode_token_rank(self, x, cache, positions, *, norm_weight=None, eps=1e-6, residual=None, rope=None):
        """Rank-space cache: append Pk, Pv (pre-RoPE coefficients) and attend with in-kernel K rebuild."""
        from .kernels.rank_decode import rank_decode, rankkv_append
        from .quant import is_quantized
        if is_quantized(*self._factor_modules()):
            raise NotImplementedError("the rank-space cache reads bf16 head bases; int4 factors decode through the dense cache")
        B = x.shape[0]
        H, Hk, Dh = self.num_heads, self.num_key_value_heads, self.head_dim
        rq, rk, rv = self._qkv_rank_tuple()
        cache.ensure_layer_ranks(self.layer_idx, rk, rv)
        pkc, pvc = cache.key_cache[self.layer_idx], cache.value_cache[self.layer_idx]
        if rope is None:
            rope = cache.get_rope_tables(seqlen=cache.max_cache_len, head_dim=Dh, device=x.device, dtype=x.dtype)
        if B <= 2 and positions.dtype == torch.int32 and positions.is_contiguous() and pkc.dim() == 3:
            # one or two tokens: the projection writes Pk | Pv into the cache rows from its own epilogue (one launch)
            p = hip_ops.linear_rankkv_append(x, self._packed_qkv_v, pkc, pvc, positions, ranks=(rq, rk, rv), norm_weight=norm_weight, eps=eps)
        elif rq % 8 == 0 and rk % 8 == 0 and rv % 8 == 0 and positions.dtype == torch.int32:
            p = hip_ops.linear(x, self._packed_qkv_v, norm_weight=norm_weight, eps=eps)       # [B, rq+rk+rv]
            rankkv_append(p[:, rq:rq + rk], p[:, rq + rk:], pkc, pvc, positions)      # one launch
        else:
            p = hip_ops.linear(x, self._packed_qkv_v, norm_weight=norm_weight, eps=eps)
            rows = torch.arange(B, device=x.device)
            pos = positions.long()
            pkc[rows, pos] = p[:, rq:rq + rk]    # device-side scatter of the new coefficients (data movement only)
            pvc[rows, pos] = p[:, rq + rk:]
        cache._layer_initialized[self.layer_idx] = True
        q = hip_ops.linear(p[:, :rq], self.q_u_proj.weight).view(B, H, Dh)
        a = rank_decode(q, pkc[:B], pvc[:B], self.k_u_proj.weight, self.v_u_proj.weight, rope[0], rope[1], positions,
                        num_kv_heads=Hk, seqlen_add=1, rotate_q=True)
        po = hip_ops.linear(a.view(B, H * Dh), self.o_v_proj.weight)
        return hip_ops.linear(po, self.o_u_proj.weight, residual=residual)

    def _flashsvd_dense_decode_token_from_hidden(self, x: torch.Tensor, cache, cache_position=None, cache_bindings=None,
                                                 advance_cache: bool = True) -> torch.Tensor:
        """x [B,1,d] (already normed) -> attention block output [B,1,d]."""
        _require_gpu(x, "SVD_LlamaAttention")
        if x.dim() != 3 or x.shape[1] != 1:
            raise ValueError(f"expected hidden states [B,1,d], got {tuple(x.shape)}")
        B = x.shape[0]
        bound = (cache_bindings or {}).get("positions") if isinstance(cache_bindings, dict) else None
        positions = bound if bound is not None else self._positions_for(cache, B, cache_position, x.device)
        ws = (cache_bindings or {}).get("attn_workspace") if isinstance(cache_bindings, dict) else None
        out = self.decode_token(x[:, 0], cache, positions, attn_ws=ws)
        if advance_cache:
            cache.advance_after_fa2(self.layer_idx, q_len=1, cache_position=cache_position)
        return out.unsqueeze(1)

    def forward(self, hidden_states: torch.Tensor, position_embeddings=None, attention_mask=None, position_ids=None,
                past_key_values=None, cache_position=None, **kwargs):
        """[B,T,d] -> ([B,T,d], None).  T tokens are appended at cache_position (default: after
        the tokens the cache has seen) and each attends causally to everything before it."""
        _require_gpu(hidden_states, "SVD_LlamaAttention")
        cache = past_key_values if past_key_values is not None else kwargs.get("past_key_value")
        B, T, d = hidden_states.shape
        if cache is None:
            cache = FlashSVDV15DenseKVCache(SimpleNamespace(num_hidden_layers=self.layer_idx + 1,
                                                            rope_theta=self.rotary_emb.base),
                                            max_batch_size=B, max_cache_len=T, device=hidden_states.device,
                                            dtype=hidden_states.dtype)
        if T == 1:
            return self._flashsvd_dense_decode_token_from_hidden(hidden_states, cache, cache_position=cache_position), None
        return self.prefill_tokens(hidden_states, cache, cache_position), None

    def prefill_tokens(self, x: torch.Tensor, cache, cache_position=None, *, norm_weight=None, eps: float = 1e-6,
                       residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Causal full-sequence pass; T tokens are appended at start..start+T-1.
        head_dim 128 with ranks that are multiples of 8 takes the matrix-core route (q/k/v rebuilt once
        per token with the rotation fused, then causal flash attention over the cache).  Other shapes
        (or FLASHSVD_AMD_PREFILL=decode) reuse the decode kernels: the T tokens of one sequence are the
        kernel's batch rows, all bound to the same cache row (batch stride 0), token t written at
        start+t and attending over start+t+1 keys."""
        self._ensure_runtime_state()
        B, T, d = x.shape
        H, Hk, Dh = self.num_heads, self.num_key_value_heads, self.head_dim
        if isinstance(cache, FlashSVDLegacySparseKVCache):
            return self._prefill_tokens_rank(x, cache, cache_position, norm_weight=norm_weight, eps=eps, residual=residual)
        # no cache_position means "prefill from slot 0", as in the reference caches' update()
        start = 0 if cache_position is None else int(cache_position.reshape(-1)[0])
        if start < 0 or start + T > cache.max_cache_len:
            raise IndexError(f"{type(cache).__name__} write position out of range: start={start} q_len={T} "
                             f"max={cache.max_cache_len}")
        cache._ensure_layer_spec(self.layer_idx, h=Hk, dh=Dh)
        kc, vc = cache.key_cache[self.layer_idx], cache.value_cache[self.layer_idx]
        rope = cache.get_rope_tables(seqlen=cache.max_cache_len, head_dim=Dh, device=x.device, dtype=x.dtype)
        from .quant import PackedQuantLinear, apply_linear, is_quantized
        if is_quantized(*self._factor_modules()):
            # int4 factors: rank projections module by module, head bases expanded to bf16 for this call
            xn = x if norm_weight is None else hip_ops.rmsnorm(x, norm_weight, eps)
            p = torch.cat([apply_linear(m, xn) for m in (self.q_v_proj, self.k_v_proj, self.v_v_proj)], dim=-1)
            wq, wk, wv = (m.dequantize(dtype=x.dtype) if isinstance(m, PackedQuantLinear) else m.weight
                          for m in (self.q_u_proj, self.k_u_proj, self.v_u_proj))
        else:
            p = hip_ops.linear(x, self._packed_qkv_v, norm_weight=norm_weight, eps=eps)   # [B,T,Rtot]
            wq, wk, wv = self.q_u_proj.weight, self.k_u_proj.weight, self.v_u_proj.weight
        rq, rk, rv = self._qkv_rank_tuple()
        mfma_ok = Dh == 128 and rq % 8 == 0 and rk % 8 == 0 and rv % 8 == 0 and T >= 16 \
            and os.getenv("FLASHSVD_AMD_PREFILL", "mfma").strip().lower() != "decode"
        a = torch.empty(B, T, H * Dh, device=x.device, dtype=x.dtype)
        if mfma_ok:
            # matrix-core route: q/k/v rebuilt once per token with the rotation fused (k, v land in the
            # cache rows start..start+T-1), then causal flash attention over the cache
            pos0 = torch.full((B,), start, device=x.device, dtype=torch.int32)
            q = torch.empty(B, T, H, Dh, device=x.device, dtype=x.dtype)
            hip_ops.lowrank_expand_heads_multi(
                [dict(p=p[..., :rq], u=wq, num_heads=H, out=q, rotate=True),
                 dict(p=p[..., rq:rq + rk], u=wk, num_heads=Hk, out=kc[:B], rotate=True, dst_by_position=True),
                 dict(p=p[..., rq + rk:], u=wv, num_heads=Hk, out=vc[:B], dst_by_position=True)],
                head_dim=Dh, cos=rope[0], sin=rope[1], positions=pos0)
            hip_ops.attn_prefill(q, kc[:B], vc[:B], q_pos0=pos0, causal=True, out=a.view(B, T, H, Dh))
        else:
            positions = torch.arange(start, start + T, device=x.device, dtype=torch.int32)
            nsplit = hip_ops.pick_nsplit(cache.max_cache_len, T, H, Dh)
            for b in range(B):
                kb, vb = kc[b:b + 1].expand(T, -1, -1, -1), vc[b:b + 1].expand(T, -1, -1, -1)
                q = hip_ops.qkv_rope_append(p[b], wq, wk, wv,
                                            rope[0], rope[1], positions, kb, vb, num_heads=H, num_kv_heads=Hk, head_dim=Dh)
                hip_ops.attn_decode_densekv(q, kb, vb, positions, seqlen_add=1, nsplit=nsplit, out=a[b].view(T, H, Dh))
        cache._layer_initialized[self.layer_idx] = True
        cache._note_seen(self.layer_idx, T, cache_position)
        po = apply_linear(self.o_v_proj, a)
        return apply_linear(self.o_u_proj, po, residual=residual)


def _prefill_tokens_rank(self, x, cache, cache_position=None, *, norm_weight=None, eps=1e-6, residual=None):
    """Rank-space prefill: the coefficients of all T tokens go into the cache.  head_dim 128 with ranks that are multiples
    of 8 (and T >= 16) then takes the matrix-core route of the dense-cache prompt pass: q of the new tokens and K / V of
    the whole context (cached coefficients included) are rebuilt ONCE into temporaries, rotation fused, and causal flash
    attention runs over them — K rounded to bf16 before the scores, as the reference's prompt kernel does
    (kernels/attn/prefill/rope_sdpa.py:133-199).  Other shapes (or FLASHSVD_AMD_PREFILL=decode) use the decode kernel:
    the tokens of a sequence are its batch rows bound to one cache row (batch stride 0) with key counts start+t+1, K
    tiles rebuilt per query — short prompts only."""
    from .kernels.rank_decode import rank_decode
    from .quant import is_quantized
    if is_quantized(*self._factor_modules()):
        raise NotImplementedError("the rank-space cache reads bf16 head bases; int4 factors decode through the dense cache")
    B, T, d = x.shape
    H, Hk, Dh = self.num_heads, self.num_key_value_heads, self.head_dim
    rq, rk, rv = self._qkv_rank_tuple()
    start = 0 if cache_position is None else int(cache_position.reshape(-1)[0])
    if start < 0 or start + T > cache.max_cache_len:
        raise IndexError(f"{type(cache).__name__} write position out of range: start={start} q_len={T} max={cache.max_cache_len}")
    cache.ensure_layer_ranks(self.layer_idx, rk, rv)
    pkc, pvc = cache.key_cache[self.layer_idx], cache.value_cache[self.layer_idx]
    rope = cache.get_rope_tables(seqlen=cache.max_cache_len, head_dim=Dh, device=x.device, dtype=x.dtype)
    p = hip_ops.linear(x, self._packed_qkv_v, norm_weight=norm_weight, eps=eps)           # [B,T,R*]
    pkc[:B, start:start + T] = p[..., rq:rq + rk]
    pvc[:B, start:start + T] = p[..., rq + rk:]
    cache._layer_initialized[self.layer_idx] = True
    cache._note_seen(self.layer_idx, T, cache_position)
    a = torch.empty(B, T, H * Dh, device=x.device, dtype=x.dtype)
    mfma_ok = Dh == 128 and rq % 8 == 0 and rk % 8 == 0 and rv % 8 == 0 and T >= 16 \
        and os.getenv("FLASHSVD_AMD_PREFILL", "mfma").strip().lower() != "decode"
    if mfma_ok:
        # q, K and V never exist for all heads at once: the heads are taken in groups whose temporaries stay inside a byte
        # budget (hip_ops.prefill_head_groups), each group expanded and attended before the next reuses the buffers
        n_ctx = start + T
        G = H // Hk
        gk = hip_ops.prefill_head_groups(B, T, n_ctx, H, Hk, Dh)
        q = torch.empty(B, T, gk * G, Dh, device=x.device, dtype=x.dtype)
        kt = torch.empty(B, n_ctx, gk, Dh, device=x.device, dtype=x.dtype)
        vt = torch.empty_like(kt)
        zero = torch.zeros(B, device=x.device, dtype=torch.int32)
        pos_q = torch.full((B,), start, device=x.device, dtype=torch.int32)
        wq, wk, wv = self.q_u_proj.weight, self.k_u_proj.weight, self.v_u_proj.weight
        av = a.view(B, T, H, Dh)
        for k0 in range(0, Hk, gk):
            k1 = min(k0 + gk, Hk)
            nk, nq = k1 - k0, (k1 - k0) * G
            qg, kg, vg = q[:, :, :nq], kt[:, :, :nk], vt[:, :, :nk]
            wqg, wkg, wvg = wq[k0 * G * Dh:k1 * G * Dh], wk[k0 * Dh:k1 * Dh], wv[k0 * Dh:k1 * Dh]
            if start == 0:
                hip_ops.lowrank_expand_heads_multi(
                    [dict(p=p[..., :rq], u=wqg, num_heads=nq, out=qg, rotate=True),
                     dict(p=p[..., rq:rq + rk], u=wkg, num_heads=nk, out=kg, rotate=True),
                     dict(p=p[..., rq + rk:], u=wvg, num_heads=nk, out=vg)],
                    head_dim=Dh, cos=rope[0], sin=rope[1], positions=zero)
            else:
                hip_ops.lowrank_expand_heads(p[..., :rq], wqg, num_heads=nq, head_dim=Dh, out=qg, cos=rope[0], sin=rope[1], positions=pos_q)
                hip_ops.lowrank_expand_heads_multi(
                    [dict(p=pkc[:B, :n_ctx], u=wkg, num_heads=nk, out=kg, rotate=True),
                     dict(p=pvc[:B, :n_ctx], u=wvg, num_heads=nk, out=vg)],
                    head_dim=Dh, cos=rope[0], sin=rope[1], positions=zero)
            hip_ops.attn_prefill(qg, kg, vg, q_pos0=pos_q, causal=True, out=av[:, :, k0 * G:k1 * G])
        po = hip_ops.linear(a, self.o_v_proj.weight)
        return hip_ops.linear(po, self.o_u_proj.weight, residual=residual)
    q = hip_ops.linear(p[..., :rq].contiguous(), self.q_u_proj.weight).view(B, T, H, Dh)
    lens = torch.arange(start + 1, start + T + 1, device=x.device, dtype=torch.int32)
    for b in range(B):
        # the rotation position of query t is its own key count - 1, which rotate_q uses
        rank_decode(q[b], pkc[b:b + 1].expand(T, -1, -1), pvc[b:b + 1].expand(T, -1, -1), self.k_u_proj.weight,
                    self.v_u_proj.weight, rope[0], rope[1], lens, num_kv_heads=Hk, rotate_q=True, out=a[b].view(T, H, Dh))
    po = hip_ops.linear(a, self.o_v_proj.weight)
    return hip_ops.linear(po, self.o_u_proj.weight, residual=residual)


SVD_LlamaAttention._prefill_tokens_rank = _prefill_tokens_rank

_FUSED_ROUNDING_BACKENDS = {
    "flashsvd_mlp_dual_split_prod", "flashsvd_mlp_dual_split_cutlass", "flashsvd_mlp_dual_split_triton_v1",
    "flashsvd_mlp_dual_split_triton_v2", "flashsvd_mlp_dual_split_triton_v2_sm80", "flashsvd_mlp_dual_split_triton_v3",
    "flashsvd_mlp_dual_split_triton_pcat_s", "dual_split_cublas", "dual_split_cutlass", "dual_split_kernel",
    "dual_split_kernel_v2", "dual_split_kernel_v2_sm80", "dual_split_kernel_v3",
}


def mlp_rounding_mode() -> int:
    """0: chain-of-linears rounding (backends ``auto``, ``*_exact_legacy``, or FFN kernels disabled);
    1: fused-kernel rounding, h = bf16(silu(g)*u) from fp32 g,u (the dual-split kernels)."""
    if _env_truthy("FLASH_SVD_DISABLE_FFN") or _env_truthy("SVDLLM_FLASH_FALLBACK"):
        return 0
    raw = os.getenv("FLASH_SVD_FFN_BACKEND", "auto").strip().lower().replace("-", "_")
    if raw in _FUSED_ROUNDING_BACKENDS and _env_truthy("FLASH_SVD_ENABLE_EXPERIMENTAL_FFN"):
        return 1
    return 0


class SVD_LlamaMLP(nn.Module):
    """SwiGLU MLP with gate/up/down each factored as v_proj then u_proj."""

    def __init__(self, hidden_size: int, intermediate_size: int, hidden_act: str = "silu", ratio: float = 1.0,
                 rank: Optional[int] = None):
        super().__init__()
        if hidden_act != "silu":
            raise ValueError(f"only the silu (SwiGLU) activation is implemented, got {hidden_act!r}")
        self.hidden_size, self.intermediate_size, self.ratio = int(hidden_size), int(intermediate_size), float(ratio)
        r = int(rank) if rank is not None else lowrank_rank(self.intermediate_size, self.hidden_size, ratio)
        self.gate_v_proj = nn.Linear(self.hidden_size, r, bias=False)
        self.gate_u_proj = nn.Linear(r, self.intermediate_size, bias=False)
        self.up_v_proj = nn.Linear(self.hidden_size, r, bias=False)
        self.up_u_proj = nn.Linear(r, self.intermediate_size, bias=False)
        self.down_v_proj = nn.Linear(self.intermediate_size, r, bias=False)
        self.down_u_proj = nn.Linear(r, self.hidden_size, bias=False)
        self._flashsvd_graph_cache: dict = {}
        self._flashsvd_layer_graph_cache: dict = {}
        self._packed_gu_v = None
        self._packed_key = None

    def _ensure_runtime_state(self) -> None:
        from .quant import is_quantized
        for name in ("_flashsvd_graph_cache", "_flashsvd_layer_graph_cache"):
            if not isinstance(getattr(self, name, None), dict):
                setattr(self, name, {})
        if is_quantized(*self._factor_modules()):
            from .quant import pack_quant_rows
            mods = [self.gate_v_proj, self.up_v_proj]
            key = tuple(m.qweight.data_ptr() if is_quantized(m) else m.weight.data_ptr() for m in mods)
            if getattr(self, "_q4_key", None) != key:
                self._q4_gu_v = pack_quant_rows(mods)       # gate and up rank projections as one int4 stream
                self._q4_key = tuple(m.qweight.data_ptr() if is_quantized(m) else m.weight.data_ptr() for m in mods)
            return
        mods = [self.gate_v_proj, self.up_v_proj]
        key = tuple((m.weight.data_ptr(), m.weight.dtype, m.weight.device) for m in mods)
        if getattr(self, "_packed_gu_v", None) is None or self._packed_key != key:
            if self.gate_v_proj.out_features != self.up_v_proj.out_features:
                raise ValueError("gate and up factors must share one rank for the packed rank projection")
            self._packed_gu_v = _packed_rows(mods)
            self._packed_key = tuple((m.weight.data_ptr(), m.weight.dtype, m.weight.device) for m in mods)
        for name in ("_flashsvd_graph_cache", "_flashsvd_layer_graph_cache"):
            if not isinstance(getattr(self, name, None), dict):
                setattr(self, name, {})

    def _factor_modules(self):
        return (self.gate_v_proj, self.gate_u_proj, self.up_v_proj, self.up_u_proj, self.down_v_proj, self.down_u_proj)

    def _run_quantized(self, x: torch.Tensor, *, norm_weight=None, eps: float = 1e-6, residual=None, mode: Optional[int] = None):
        """The same four stages with int4 factors: each projection through the kernel that fits its module."""
        from .quant import PackedQuantLinear, apply_linear
        gu, uu = self.gate_u_proj, self.up_u_proj
        r = int(self.gate_v_proj.out_features)
        if int(self.up_v_proj.out_features) != r:
            raise ValueError("gate and up factors must share one rank")
        self._ensure_runtime_state()
        rows = x.numel() // x.shape[-1]
        pk = getattr(self, "_q4_gu_v", None)
        if pk is not None and self.gate_v_proj.streams_int4(rows):
            p = hip_ops.linear_q4(x, *pk, group_size=self.gate_v_proj.group_size, norm_weight=norm_weight, eps=eps)
        else:
            xn = x if norm_weight is None else hip_ops.rmsnorm(x, norm_weight, eps)
            p = torch.empty(*x.shape[:-1], 2 * r, device=x.device, dtype=x.dtype)
            p2 = p.view(-1, 2 * r)
            apply_linear(self.gate_v_proj, xn.reshape(-1, xn.shape[-1]), out=p2[:, :r])
            apply_linear(self.up_v_proj, xn.reshape(-1, xn.shape[-1]), out=p2[:, r:])
        mode = mlp_rounding_mode() if mode is None else mode
        both_q = isinstance(gu, PackedQuantLinear) and isinstance(uu, PackedQuantLinear)
        if both_q and gu.streams_int4(rows) and uu.streams_int4(rows) and gu.group_size == uu.group_size:
            h = hip_ops.swiglu_linear_q4(p, (gu.qweight, gu.scales, gu.zeros), (uu.qweight, uu.scales, uu.zeros), up_off=r,
                                         group_size=gu.group_size, mode=mode)
        else:
            wg = gu.dequantize(dtype=x.dtype) if isinstance(gu, PackedQuantLinear) else gu.weight
            wu = uu.dequantize(dtype=x.dtype) if isinstance(uu, PackedQuantLinear) else uu.weight
            h = hip_ops.swiglu_linear(p, wg, wu, up_off=r, mode=mode)
        s = apply_linear(self.down_v_proj, h)
        return apply_linear(self.down_u_proj, s, residual=residual)

    def run(self, x: torch.Tensor, *, norm_weight=None, eps: float = 1e-6, residual=None, mode: Optional[int] = None):
        """x [..., d] -> (residual +) down_u(down_v(silu(gate(x)) * up(x))); four weight streams."""
        from .quant import is_quantized
        if is_quantized(*self._factor_modules()):
            return self._run_quantized(x, norm_weight=norm_weight, eps=eps, residual=residual, mode=mode)
        self._ensure_runtime_state()
        r = self.gate_v_proj.out_features
        p = hip_ops.linear(x, self._packed_gu_v, norm_weight=norm_weight, eps=eps)      # [.., 2R] = [PGate | PUp]
        h = hip_ops.swiglu_linear(p, self.gate_u_proj.weight, self.up_u_proj.weight, up_off=r,
                                  mode=mlp_rounding_mode() if mode is None else mode)
        s = hip_ops.linear(h, self.down_v_proj.weight)
        return hip_ops.linear(s, self.down_u_proj.weight, residual=residual)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        _require_gpu(x, "SVD_LlamaMLP")
        if _env_truthy("FLASH_SVD_MLP_CUDA_GRAPH") and x.dim() == 3 and x.shape[1] == 1 and not torch.cuda.is_current_stream_capturing():
            scope = os.getenv("FLASH_SVD_MLP_CUDA_GRAPH_SCOPE", "auto").strip().lower()
            if scope in ("auto", "mlp", "layer_tail"):
                return self._graphed(x)
        return self.run(x)

    def _graphed(self, x: torch.Tensor) -> torch.Tensor:
        """Replay a captured graph of ``run`` keyed by input shape and rounding mode."""
        from .graphs import GraphedCallable
        key = (tuple(x.shape), x.dtype, x.device, mlp_rounding_mode())
        g = self._flashsvd_graph_cache.get(key)
        if g is None:
            mode = key[-1]
            g = GraphedCallable(lambda t: self.run(t, mode=mode), x)
            self._flashsvd_graph_cache[key] = g
        out = g(x)
        return out if _env_truthy("FLASH_SVD_MLP_CUDA_GRAPH_ALIAS_OUTPUT") else out.clone()


class SVDLlamaDecoderLayer(nn.Module):
    def __init__(self, config, layer_idx: int, attn_ratio: float, mlp_ratio: float, attn_ranks=None, mlp_rank=None):
        super().__init__()
        self.layer_idx = int(layer_idx)
        eps = float(getattr(config, "rms_norm_eps", 1e-6))
        self.input_layernorm = LlamaRMSNorm(config.hidden_size, eps)
        self.self_attn = SVD_LlamaAttention(config, ratio=attn_ratio, layer_idx=layer_idx, ranks=attn_ranks)
        self.post_attention_layernorm = LlamaRMSNorm(config.hidden_size, eps)
        self.mlp = SVD_LlamaMLP(config.hidden_size, config.intermediate_size, getattr(config, "hidden_act", "silu"),
                                ratio=mlp_ratio, rank=mlp_rank)

    def decode_token(self, x: torch.Tensor, cache, positions: torch.Tensor, *, rope=None, attn_ws=None, nsplit=None):
        """x [B,d] -> [B,d]; both RMSNorms and both residual adds are fused into the projections."""
        return decoder_layer_decode_token(self, x, cache, positions, rope=rope, attn_ws=attn_ws, nsplit=nsplit)

    def _layer_tail(self, x2: torch.Tensor) -> torch.Tensor:
        return decoder_layer_tail(self, x2)

    def forward(self, hidden_states: torch.Tensor, attention_mask=None, position_ids=None, past_key_values=None,
                cache_position=None, position_embeddings=None, **kwargs):
        return decoder_layer_forward(self, hidden_states, past_key_values=past_key_values, cache_position=cache_position, **kwargs)


# The three functions below are the decoder layer.  They take any module that carries ``input_layernorm``, ``self_attn``
# (SVD_LlamaAttention), ``post_attention_layernorm`` and ``mlp`` (SVD_LlamaMLP): this package's SVDLlamaDecoderLayer, or an
# unmodified transformers LlamaDecoderLayer whose two sub-modules were swapped for the low-rank ones (the reference's
# arrangement, utils/model_utils.py:586-671), once enable_flashsvd_llama_layer_tail_cuda_graph() has patched that class.
def decoder_layer_decode_token(layer, x: torch.Tensor, cache, positions: torch.Tensor, *, rope=None, attn_ws=None, nsplit=None):
    n1 = layer.input_layernorm
    x2 = layer.self_attn.decode_token(x, cache, positions, norm_weight=n1.weight, eps=n1.variance_epsilon,
                                      residual=x, rope=rope, attn_ws=attn_ws, nsplit=nsplit)
    return decoder_layer_tail(layer, x2)


def decoder_layer_tail(layer, x2: torch.Tensor) -> torch.Tensor:
    """residual + post-attention norm + MLP + residual; replayed from a captured graph when the
    layer-tail scope is enabled and no outer capture is running."""
    n2, mlp = layer.post_attention_layernorm, layer.mlp
    want_graph = (LAYER_TAIL_GRAPH_ENABLED and _env_truthy("FLASH_SVD_MLP_CUDA_GRAPH")
                  and os.getenv("FLASH_SVD_MLP_CUDA_GRAPH_SCOPE", "auto").strip().lower() in ("auto", "layer_tail")
                  and not torch.cuda.is_current_stream_capturing())
    if not want_graph:
        return mlp.run(x2, norm_weight=n2.weight, eps=n2.variance_epsilon, residual=x2)
    from .graphs import GraphedCallable
    mode = mlp_rounding_mode()
    cache = mlp._flashsvd_layer_graph_cache
    key = (tuple(x2.shape), x2.dtype, x2.device, mode)
    g = cache.get(key)
    if g is None:
        g = GraphedCallable(lambda t: mlp.run(t, norm_weight=n2.weight, eps=n2.variance_epsilon, residual=t, mode=mode), x2)
        cache[key] = g
    out = g(x2)
    return out if _env_truthy("FLASH_SVD_MLP_CUDA_GRAPH_ALIAS_OUTPUT") else out.clone()


def decoder_layer_forward(layer, hidden_states: torch.Tensor, *, past_key_values=None, cache_position=None, **kwargs):
    _require_gpu(hidden_states, type(layer).__name__)
    attn = layer.self_attn
    cache = past_key_values if past_key_values is not None else kwargs.get("past_key_value")
    B, T, d = hidden_states.shape
    n1 = layer.input_layernorm
    if cache is None:
        cache = FlashSVDV15DenseKVCache(SimpleNamespace(num_hidden_layers=attn.layer_idx + 1, rope_theta=attn.rotary_emb.base),
                                        max_batch_size=B, max_cache_len=T, device=hidden_states.device, dtype=hidden_states.dtype)
    if T == 1:
        positions = attn._positions_for(cache, B, cache_position, hidden_states.device)
        out = decoder_layer_decode_token(layer, hidden_states[:, 0], cache, positions).unsqueeze(1)
        cache.advance_after_fa2(attn.layer_idx, q_len=1, cache_position=cache_position)
        return out
    x2 = attn.prefill_tokens(hidden_states, cache, cache_position, norm_weight=n1.weight, eps=n1.variance_epsilon,
                             residual=hidden_states)
    n2 = layer.post_attention_layernorm      # prompt rows: no graph (the captured tail is a decode-step device)
    return layer.mlp.run(x2, norm_weight=n2.weight, eps=n2.variance_epsilon, residual=x2)


_HF_PATCH = {}


def patch_hf_llama_decoder_layer() -> bool:
    """Idempotent, process-global: give transformers' LlamaDecoderLayer a forward that, for a layer whose ``mlp`` is an
    SVD_LlamaMLP, runs "residual + post-attention norm + MLP + residual" through the fused kernels (and from one captured
    graph under the layer_tail scope); when ``self_attn`` is an SVD_LlamaAttention too the whole layer takes the same
    route as SVDLlamaDecoderLayer, bit for bit.  Layers with other modules, and tensors that are not bf16 on the GPU, keep
    the original forward.  Returns False when transformers is not importable."""
    if _HF_PATCH:
        return True
    try:
        from transformers.models.llama.modeling_llama import LlamaDecoderLayer
    except Exception:
        return False
    orig = LlamaDecoderLayer.forward
    # Whether the installed transformers returns the hidden state itself or a 1-tuple: releases that return a tuple build
    # it as `outputs = (hidden_states,)` in the layer's forward; the return annotation is the fallback where the source
    # cannot be read.
    try:
        import inspect
        returns_tensor = "outputs = (hidden_states,)" not in inspect.getsource(orig)
    except (OSError, TypeError):
        returns_tensor = orig.__annotations__.get("return") in (torch.Tensor, "torch.Tensor")
    _cache_kw = {}

    def cache_kwarg(attn_mod) -> str:
        """The name under which this attention class takes the cache (`past_key_values` in transformers 4.56+ / 5.x,
        `past_key_value` before): passing it under the other name would drop it into **kwargs unnoticed."""
        cls = type(attn_mod)
        if cls not in _cache_kw:
            import inspect
            names = inspect.signature(cls.forward).parameters
            if "past_key_values" in names:
                _cache_kw[cls] = "past_key_values"
            elif "past_key_value" in names:
                _cache_kw[cls] = "past_key_value"
            elif any(p.kind is inspect.Parameter.VAR_KEYWORD for p in names.values()):
                _cache_kw[cls] = "past_key_values"       # an open signature: the spelling the installed layer itself uses
            else:
                raise TypeError(f"{cls.__name__}.forward takes neither past_key_values nor past_key_value")
        return _cache_kw[cls]

    def forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_values=None, use_cache=False,
                position_embeddings=None, **kwargs):
        if not isinstance(self.mlp, SVD_LlamaMLP) or not hidden_states.is_cuda or hidden_states.dtype not in (torch.bfloat16, torch.float16):
            return orig(self, hidden_states, attention_mask=attention_mask, position_ids=position_ids,
                        past_key_values=past_key_values, use_cache=use_cache, position_embeddings=position_embeddings, **kwargs)
        if _env_truthy("FLASH_SVD_MLP_CUDA_GRAPH") and os.getenv("FLASH_SVD_MLP_CUDA_GRAPH_SCOPE", "auto").strip().lower() == "mlp":
            # scope "mlp": the graph covers the MLP module alone (SVD_LlamaMLP.forward replays it); the layer around it
            # stays the original one
            return orig(self, hidden_states, attention_mask=attention_mask, position_ids=position_ids,
                        past_key_values=past_key_values, use_cache=use_cache, position_embeddings=position_embeddings, **kwargs)
        if past_key_values is None:
            past_key_values = kwargs.pop("past_key_value", None)
        if isinstance(self.self_attn, SVD_LlamaAttention) and \
                (past_key_values is None or isinstance(past_key_values, (FlashSVDV15DenseKVCache, FlashSVDLegacySparseKVCache))):
            out = decoder_layer_forward(self, hidden_states, past_key_values=past_key_values,
                                        cache_position=kwargs.get("cache_position"))
        else:
            # attention half as the unmodified layer runs it (any attention module), fused tail
            h = self.input_layernorm(hidden_states)
            h = self.self_attn(hidden_states=h, attention_mask=attention_mask, position_ids=position_ids, use_cache=use_cache,
                               position_embeddings=position_embeddings, **{cache_kwarg(self.self_attn): past_key_values}, **kwargs)
            h = h[0] if isinstance(h, (tuple, list)) else h
            x2 = hidden_states + h
            shape = x2.shape
            if x2.dim() == 3 and shape[1] == 1:
                out = decoder_layer_tail(self, x2.reshape(-1, shape[-1])).reshape(shape)
            else:
                # prompt rows: no graph (one would be captured and kept per prompt shape and layer), as decoder_layer_forward
                n2 = self.post_attention_layernorm
                out = self.mlp.run(x2, norm_weight=n2.weight, eps=n2.variance_epsilon, residual=x2)
        return out if returns_tensor else (out,)

    LlamaDecoderLayer.forward = forward
    _HF_PATCH.update(cls=LlamaDecoderLayer, orig=orig)
    return True


def unpatch_hf_llama_decoder_layer() -> None:
    """Put the original forward back (tests)."""
    if _HF_PATCH:
        _HF_PATCH["cls"].forward = _HF_PATCH["orig"]
        _HF_PATCH.clear()


class SVDLlamaModel(nn.Module):
    def __init__(self, config, attn_ratio: float, mlp_ratio: float, attn_ranks=None, mlp_rank=None):
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([
            SVDLlamaDecoderLayer(config, i, attn_ratio, mlp_ratio, attn_ranks, mlp_rank)
            for i in range(config.num_hidden_layers)])
        self.norm = LlamaRMSNorm(config.hidden_size, float(getattr(config, "rms_norm_eps", 1e-6)))
        hd = int(getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads)
        self.rotary_emb = LlamaRotaryEmbedding(hd, int(getattr(config, "max_position_embeddings", 4096)),
                                               float(getattr(config, "rope_theta", 10000.0)))


class SVDLlamaForCausalLM(nn.Module):
    """embed -> N low-rank decoder layers -> RMSNorm -> lm_head, with the attribute layout
    (``model.embed_tokens/layers/norm/rotary_emb``, ``lm_head``, ``config``) the reference's
    manual decode step walks (utils/evaluator.py:30-82)."""

    def __init__(self, config, attn_ratio: float = 1.0, mlp_ratio: float = 1.0, attn_ranks=None, mlp_rank=None):
        super().__init__()
        self.config = config
        self.model = SVDLlamaModel(config, attn_ratio, mlp_ratio, attn_ranks, mlp_rank)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        for p in self.parameters():
            p.requires_grad_(False)

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, past_key_values=None, cache_position=None, use_cache: bool = True,
                attention_mask=None, logits_to_keep: int = 0, **kwargs):
        if attention_mask is not None and not bool(torch.all(attention_mask != 0)):
            raise NotImplementedError("padded batches are not supported by the decode-kernel prefill")
        inner = self.model
        x = inner.embed_tokens(input_ids)
        _require_gpu(x, "SVDLlamaForCausalLM")
        B, T = input_ids.shape
        cache = past_key_values
        if cache is None:
            cache = FlashSVDV15DenseKVCache(self.config, max_batch_size=B, max_cache_len=T, device=x.device, dtype=x.dtype)
        for layer in inner.layers:
            x = layer(x, past_key_values=cache, cache_position=cache_position)
        keep = x if logits_to_keep == 0 else x[:, -int(logits_to_keep):]
        logits = hip_ops.linear(keep, self.lm_head.weight, norm_weight=inner.norm.weight, eps=inner.norm.variance_epsilon)
        return SimpleNamespace(logits=logits, past_key_values=cache, hidden_states=x)

    @torch.no_grad()
    def decode_step(self, input_ids: torch.Tensor, cache, positions: torch.Tensor, *, rope=None, attn_ws=None,
                    nsplit=None, return_hidden: bool = False):
        """One token per row: ids [B,1] -> logits [B,1,V].  ``positions`` int32 [B] on the device."""
        inner = self.model
        x = inner.embed_tokens(input_ids)[:, 0]
        for layer in inner.layers:
            x = layer.decode_token(x, cache, positions, rope=rope, attn_ws=attn_ws, nsplit=nsplit)
        logits = hip_ops.linear(x, self.lm_head.weight, norm_weight=inner.norm.weight, eps=inner.norm.variance_epsilon)
        out = logits.unsqueeze(1)
        return (out, x) if return_hidden else out


def build_model(*, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, intermediate_size: int,
                num_layers: int, vocab_size: int, attn_rank: int, mlp_rank: int, rope_theta: float = 10000.0,
                rms_norm_eps: float = 1e-6, max_position_embeddings: int = 4096) -> SVDLlamaForCausalLM:
    """Random-shaped model with explicit ranks (weights are left uninitialised: load or fill them)."""
    cfg = SimpleNamespace(hidden_size=hidden_size, num_attention_heads=num_heads, num_key_value_heads=num_kv_heads,
                          head_dim=head_dim, intermediate_size=intermediate_size, num_hidden_layers=num_layers,
                          vocab_size=vocab_size, rope_theta=rope_theta, rms_norm_eps=rms_norm_eps, hidden_act="silu",
                          max_position_embeddings=max_position_embeddings)
    with torch.device("meta"):
        model = SVDLlamaForCausalLM(cfg, attn_ranks=dict(q=attn_rank, k=attn_rank, v=attn_rank, o=attn_rank),
                                    mlp_rank=mlp_rank)
    return model


def materialize(model: SVDLlamaForCausalLM, device, dtype=torch.bfloat16, *, seed: Optional[int] = None,
                std: float = 0.02) -> SVDLlamaForCausalLM:
    """Give a meta-device model real storage on ``device``; with ``seed`` every matrix is filled with
    N(0, std) drawn on the device, RMSNorm weights with 1."""
    model = model.to(dtype=dtype).to_empty(device=device)
    gen = None
    if seed is not None:
        gen = torch.Generator(device=device)
        gen.manual_seed(int(seed))
    for mod in model.modules():
        if isinstance(mod, LlamaRotaryEmbedding):
            half = mod.dim // 2
            mod.inv_freq = 1.0 / (mod.base ** (torch.arange(0, half, dtype=torch.float32, device=device) / half))
        elif isinstance(mod, LlamaRMSNorm):
            mod.weight.data.fill_(1.0)
        elif isinstance(mod, (nn.Linear, nn.Embedding)) and gen is not None:
            w = mod.weight.data
            w.copy_(torch.randn(w.shape, generator=gen, device=device, dtype=torch.float32) * std)
    return model.eval()
