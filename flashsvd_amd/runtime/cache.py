"""KV caches of the decode path.

``FlashSVDV15DenseKVCache`` keeps post-RoPE K and V per layer as [Bmax, Smax, Hk, Dh]
(runtime/cache/attn_dense_kv.py:7-357 of the reference); ``FlashSVDLegacySparseKVCache`` keeps
the pre-RoPE rank coefficients Pk, Pv per layer as [Bmax, Smax, R]
(runtime/cache/attn_legacy_sparse_kv.py:22-257).  Both are plain Python objects (no dependency
on the transformers ``Cache`` base class) with the method names, return values and error
behaviour the reference's callers rely on.  Storage is allocated once at full size so that
decode kernels can write in place and a captured HIP graph keeps valid pointers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch


def _as_device(d) -> torch.device:
    return torch.device("cuda", d) if isinstance(d, int) else torch.device(d)


def _rope_tables(cache: dict, seqlen: int, head_dim: int, theta: float, device, dtype):
    key = (int(seqlen), int(head_dim), float(theta), dtype, torch.device(device))
    hit = cache.get(key)
    if hit is not None:
        return hit
    if head_dim % 2:
        raise ValueError(f"head_dim must be even, got {head_dim}")
    half = head_dim // 2
    pos = torch.arange(int(seqlen), device=device, dtype=torch.float32)
    inv_freq = 1.0 / (float(theta) ** (torch.arange(0, half, device=device, dtype=torch.float32) / half))
    ang = pos[:, None] * inv_freq[None, :]
    pair = (torch.cos(ang).to(dtype).contiguous(), torch.sin(ang).to(dtype).contiguous())
    cache[key] = pair
    return pair


class _CacheBase:
    is_compileable = False

    def __init__(self, config, max_batch_size: int, max_cache_len: int, device, dtype, layer_device_map):
        self._config = config
        self._max_batch_size = int(max_batch_size)
        self._max_cache_len = int(max_cache_len)
        self._dtype = dtype
        self._rope_theta = float(getattr(config, "rope_theta", 10000.0))
        self._seen_tokens = 0
        self._rope_cache: dict = {}
        n_layers = int(getattr(config, "num_hidden_layers", 0))
        base = torch.device(device) if device is not None else torch.device("cpu")
        self._layer_device = [
            _as_device(layer_device_map[i]) if layer_device_map is not None else base for i in range(n_layers)]
        self._layer_initialized = [False] * n_layers
        self.key_cache: list[torch.Tensor] = []
        self.value_cache: list[torch.Tensor] = []

    max_batch_size = property(lambda self: self._max_batch_size)
    max_cache_len = property(lambda self: self._max_cache_len)

    def __len__(self) -> int:
        return len(self.key_cache)

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        return int(self._seen_tokens)

    def get_max_cache_shape(self) -> Optional[int]:
        return self._max_cache_len

    def get_mask_sizes(self, cache_position: torch.Tensor, layer_idx: int) -> tuple[int, int]:
        return int(cache_position.shape[0]) + int(self._seen_tokens), 0

    def get_rope_tables(self, *, seqlen: int, head_dim: int, device, dtype):
        """(cos, sin), each [seqlen, head_dim/2]: fp32 angles pos * theta^(-i/half) cast to ``dtype``."""
        return _rope_tables(self._rope_cache, seqlen, head_dim, self._rope_theta, device, dtype)

    def _note_seen(self, layer_idx: int, q_len: int, cache_position) -> None:
        """Only layer 0 advances the token count; exact for host positions, sequential otherwise."""
        if int(layer_idx) != 0:
            return
        if cache_position is None:
            self._seen_tokens = max(self._seen_tokens, int(q_len))
        elif torch.is_tensor(cache_position) and not cache_position.is_cuda and cache_position.numel() > 0:
            self._seen_tokens = max(self._seen_tokens, int(cache_position.max()) + 1)
        else:
            self._seen_tokens = self._seen_tokens + int(q_len)

    def reset(self) -> None:
        self._seen_tokens = 0


class FlashSVDV15DenseKVCache(_CacheBase):
    """Dense KV cache, [B, S, Hk, Dh] per layer, K stored after RoPE."""

    def __init__(self, config, *, max_batch_size: int, max_cache_len: int, device=None,
                 dtype: torch.dtype = torch.float16, layer_device_map: Optional[dict] = None) -> None:
        super().__init__(config, max_batch_size, max_cache_len, device, dtype, layer_device_map)
        for dev in self._layer_device:
            # shaped lazily: head count / head_dim are learnt from the first write
            self.key_cache.append(torch.zeros((self._max_batch_size, self._max_cache_len, 0, 0), dtype=dtype, device=dev))
            self.value_cache.append(torch.zeros((self._max_batch_size, self._max_cache_len, 0, 0), dtype=dtype, device=dev))
        self._layer_heads = [0] * len(self._layer_device)
        self._layer_head_dim = [0] * len(self._layer_device)
        self._seqlens: dict[tuple[int, int], torch.Tensor] = {}

    # -- storage ---------------------------------------------------------------------------
    def _ensure_layer_spec(self, layer_idx: int, *, h: int, dh: int) -> None:
        layer_idx, h, dh = int(layer_idx), int(h), int(dh)
        cur = self.key_cache[layer_idx]
        if (cur.shape[2], cur.shape[3]) == (h, dh):
            return
        if self._layer_initialized[layer_idx]:
            raise RuntimeError(
                f"FlashSVDV15DenseKVCache shape changed after init for layer {layer_idx}: "
                f"old={(int(cur.shape[2]), int(cur.shape[3]))}, new={(h, dh)}")
        shape = (self._max_batch_size, self._max_cache_len, h, dh)
        self.key_cache[layer_idx] = torch.zeros(shape, dtype=self._dtype, device=self._layer_device[layer_idx])
        self.value_cache[layer_idx] = torch.zeros(shape, dtype=self._dtype, device=self._layer_device[layer_idx])
        self._layer_heads[layer_idx], self._layer_head_dim[layer_idx] = h, dh

    def _seqlens_buffer(self, layer_idx: int, batch_size: int) -> torch.Tensor:
        key = (int(layer_idx), int(batch_size))
        dev = self.key_cache[int(layer_idx)].device
        buf = self._seqlens.get(key)
        if buf is None or buf.device != dev:
            buf = torch.empty((int(batch_size),), device=dev, dtype=torch.int32)
            self._seqlens[key] = buf
        return buf

    @staticmethod
    def _fill_cache_seqlens_buffer(cache_seqlens: torch.Tensor, *, seen_tokens: int, cache_position=None) -> torch.Tensor:
        if cache_position is None:
            cache_seqlens.fill_(int(seen_tokens))
        elif torch.is_tensor(cache_position):
            pos = cache_position.to(device=cache_seqlens.device, dtype=torch.int32).reshape(-1)
            if pos.numel() == 0:
                cache_seqlens.zero_()
            elif pos.numel() == 1:
                cache_seqlens.copy_(pos.expand_as(cache_seqlens))
            else:
                cache_seqlens.copy_(pos[: cache_seqlens.shape[0]])
        else:
            cache_seqlens.fill_(int(cache_position))
        return cache_seqlens

    # -- HF-style update (prefill copy or positional scatter) -------------------------------
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict[str, Any]] = None):
        """key/value_states are [B, Hk, T, Dh]; returns the valid cache prefix as [B, Hk, L, Dh]."""
        layer_idx = int(layer_idx)
        cache_position = (cache_kwargs or {}).get("cache_position")
        self._ensure_layer_spec(layer_idx, h=key_states.shape[1], dh=key_states.shape[-1])
        kc, vc = self.key_cache[layer_idx], self.value_cache[layer_idx]
        k_bshd = key_states.to(device=kc.device, dtype=kc.dtype).transpose(1, 2)
        v_bshd = value_states.to(device=vc.device, dtype=vc.dtype).transpose(1, 2)
        b, t = k_bshd.shape[0], k_bshd.shape[1]
        if cache_position is None:
            kc[:b, :t].copy_(k_bshd)
            vc[:b, :t].copy_(v_bshd)
        else:
            idx = cache_position.to(device=kc.device)
            kc[:b].index_copy_(1, idx, k_bshd.contiguous())
            vc[:b].index_copy_(1, idx, v_bshd.contiguous())
        self._layer_initialized[layer_idx] = True
        self._note_seen(layer_idx, t, cache_position)
        n = t if cache_position is None else int(self.get_seq_length())
        return kc[:b, :n].transpose(1, 2).contiguous(), vc[:b, :n].transpose(1, 2).contiguous()

    # -- decode-step helpers ------------------------------------------------------------------
    def prepare_fa2_step(self, layer_idx: int, *, batch_size: int, cache_position=None):
        """(k_cache[:B], v_cache[:B], cache_seqlens int32 [B]) for an attend-with-append kernel."""
        layer_idx, batch_size = int(layer_idx), int(batch_size)
        lens = self._seqlens_buffer(layer_idx, batch_size)
        self._fill_cache_seqlens_buffer(lens, seen_tokens=self.get_seq_length(), cache_position=cache_position)
        return self.key_cache[layer_idx][:batch_size], self.value_cache[layer_idx][:batch_size], lens

    def get_fa2_kvcache(self, layer_idx: int, *, batch_size: int):
        return self.prepare_fa2_step(layer_idx, batch_size=batch_size, cache_position=None)

    def prepare_fa2_direct_write_step(self, layer_idx: int, *, batch_size: int, num_heads: int, head_dim: int,
                                      q_len: int, cache_position=None):
        """Views for writing the current token straight into the cache: (k_cache, v_cache,
        k_slot, v_slot, cache_seqlens = start + q_len).  None unless q_len == 1 and all
        positions are equal; IndexError if the slot is outside the cache."""
        layer_idx, batch_size, q_len = int(layer_idx), int(batch_size), int(q_len)
        if q_len != 1:
            return None
        self._ensure_layer_spec(layer_idx, h=num_heads, dh=head_dim)
        if cache_position is None:
            start = int(self.get_seq_length())
        elif torch.is_tensor(cache_position):
            pos = cache_position.reshape(-1)
            if pos.numel() == 0:
                return None
            vals = pos.tolist()  # one host read, like the reference
            if any(v != vals[0] for v in vals):
                return None
            start = int(vals[0])
        else:
            start = int(cache_position)
        if start < 0 or start + q_len > self._max_cache_len:
            raise IndexError(
                f"FlashSVDV15DenseKVCache write position out of range: start={start} q_len={q_len} max={self._max_cache_len}")
        kc, vc = self.key_cache[layer_idx][:batch_size], self.value_cache[layer_idx][:batch_size]
        lens = self._seqlens_buffer(layer_idx, batch_size)
        lens.fill_(start + q_len)
        self._layer_initialized[layer_idx] = True
        return kc, vc, kc[:, start:start + q_len], vc[:, start:start + q_len], lens

    def advance_after_fa2(self, layer_idx: int, *, q_len: int, cache_position) -> None:
        if int(layer_idx) != 0:
            return
        if cache_position is not None and torch.is_tensor(cache_position) and not cache_position.is_cuda \
                and cache_position.numel() > 0:
            self._seen_tokens = max(self._seen_tokens, int(cache_position.max()) + 1)
        else:
            self._seen_tokens = self._seen_tokens + int(q_len)

    def clone_for_autotune(self, *, layer_idx: int, batch_size: int) -> "FlashSVDV15DenseKVCache":
        """A scratch copy holding only ``layer_idx``'s first ``batch_size`` rows."""
        layer_idx, batch_size = int(layer_idx), int(batch_size)
        other = type(self)(self._config, max_batch_size=self._max_batch_size, max_cache_len=self._max_cache_len,
                           device=self._layer_device[0] if self._layer_device else None, dtype=self._dtype,
                           layer_device_map=dict(enumerate(self._layer_device)))
        other._seen_tokens = self._seen_tokens
        h, dh = self._layer_heads[layer_idx], self._layer_head_dim[layer_idx]
        if h > 0 and dh > 0:
            other._ensure_layer_spec(layer_idx, h=h, dh=dh)
            other.key_cache[layer_idx][:batch_size].copy_(self.key_cache[layer_idx][:batch_size])
            other.value_cache[layer_idx][:batch_size].copy_(self.value_cache[layer_idx][:batch_size])
            other._layer_initialized[layer_idx] = self._layer_initialized[layer_idx]
        return other


@dataclass
class _DecodeWorkspace:
    """Split-K scratch of the rank-space decode kernel: running max / sum [B,H,S] fp32, rank-space
    accumulator [B,H,S,R] fp32 and the two pre-rotated query halves [B,H,Dh/2]."""
    M: torch.Tensor
    L: torch.Tensor
    Acc: torch.Tensor
    Q0: torch.Tensor
    Q1: torch.Tensor


class FlashSVDLegacySparseKVCache(_CacheBase):
    """Rank-space KV cache: Pk = X @ k_v^T and Pv = X @ v_v^T (pre-RoPE), [B, S, R] per layer.
    K/V heads are rebuilt inside the decode kernel from the per-head bases."""

    def __init__(self, config, *, max_batch_size: int, max_cache_len: int, rank: Optional[int] = None,
                 rank_k: Optional[int] = None, rank_v: Optional[int] = None, device=None,
                 dtype: torch.dtype = torch.float16, layer_device_map: Optional[dict] = None) -> None:
        super().__init__(config, max_batch_size, max_cache_len, device, dtype, layer_device_map)
        if rank is not None:
            rank_k = rank_v = int(rank)
        rk, rv = int(rank_k or 0), int(rank_v or 0)
        self.rank = int(rk or rv or 0)  # hint only; per-layer ranks may differ
        for dev in self._layer_device:
            self.key_cache.append(torch.zeros((self._max_batch_size, self._max_cache_len, rk), dtype=dtype, device=dev))
            self.value_cache.append(torch.zeros((self._max_batch_size, self._max_cache_len, rv), dtype=dtype, device=dev))
        self._layer_key_rank = [rk] * len(self._layer_device)
        self._layer_value_rank = [rv] * len(self._layer_device)
        self._decode_workspaces: dict = {}

    def ensure_layer_ranks(self, layer_idx: int, k_rank: int, v_rank: int) -> None:
        layer_idx, k_rank, v_rank = int(layer_idx), int(k_rank), int(v_rank)
        kc, vc = self.key_cache[layer_idx], self.value_cache[layer_idx]
        if kc.shape[-1] == k_rank and vc.shape[-1] == v_rank:
            return
        if self._layer_initialized[layer_idx]:
            raise RuntimeError(
                "FlashSVDLegacySparseKVCache rank changed after initialization for layer "
                f"{layer_idx}: cache.key_rank={int(kc.shape[-1])} cache.value_rank={int(vc.shape[-1])} "
                f"but got key rank {k_rank}, value rank {v_rank}.")
        dev = self._layer_device[layer_idx]
        self.key_cache[layer_idx] = torch.zeros((self._max_batch_size, self._max_cache_len, k_rank), dtype=self._dtype, device=dev)
        self.value_cache[layer_idx] = torch.zeros((self._max_batch_size, self._max_cache_len, v_rank), dtype=self._dtype, device=dev)
        self._layer_key_rank[layer_idx], self._layer_value_rank[layer_idx] = k_rank, v_rank
        self.rank = int(self.rank or k_rank or v_rank)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[dict[str, Any]] = None):
        """key/value_states are rank coefficients [B, T, R]; returned unchanged (cast to the cache dtype)."""
        layer_idx = int(layer_idx)
        cache_position = (cache_kwargs or {}).get("cache_position")
        self.ensure_layer_ranks(layer_idx, key_states.shape[-1], value_states.shape[-1])
        kc, vc = self.key_cache[layer_idx], self.value_cache[layer_idx]
        key_states = key_states.to(dtype=kc.dtype, device=kc.device)
        value_states = value_states.to(dtype=vc.dtype, device=vc.device)
        self._layer_initialized[layer_idx] = True
        b, t = key_states.shape[0], key_states.shape[1]
        if cache_position is None:
            kc[:b, :t].copy_(key_states)
            vc[:b, :t].copy_(value_states)
        else:
            idx = cache_position.to(device=kc.device)
            kc[:b].index_copy_(1, idx, key_states)
            vc[:b].index_copy_(1, idx, value_states)
        self._note_seen(layer_idx, t, cache_position)
        return key_states, value_states

    def get_decode_workspace(self, *, batch_size: int, num_heads: int, rank: int, head_dim: int, max_splits: int,
                             device, dtype) -> _DecodeWorkspace:
        key = (int(batch_size), int(num_heads), int(rank), int(max_splits), dtype, torch.device(device))
        ws = self._decode_workspaces.get(key)
        if ws is None:
            if head_dim % 2:
                raise ValueError(f"head_dim must be even, got {head_dim}")
            b, h, r, s = key[:4]
            f32 = dict(device=device, dtype=torch.float32)
            ws = _DecodeWorkspace(M=torch.empty((b, h, s), **f32), L=torch.empty((b, h, s), **f32),
                                  Acc=torch.empty((b, h, s, r), **f32),
                                  Q0=torch.empty((b, h, head_dim // 2), device=device, dtype=dtype),
                                  Q1=torch.empty((b, h, head_dim // 2), device=device, dtype=dtype))
            self._decode_workspaces[key] = ws
        return ws


# names kept for older imports
FlashSVDDenseKVCache = FlashSVDV15DenseKVCache
LowRankKVCache = FlashSVDLegacySparseKVCache
