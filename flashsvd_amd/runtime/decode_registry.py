"""Decode dispatch: where the runtime finds its kernels.

Keeps the lookup functions of the reference's runtime/attn/decode_registry.py (:21-35 helpers,
:153-237 resolvers, :406-414 aliases) with the same names and return conventions, resolved to the
HIP-backed modules of this package instead of Triton files and the flash-attn wheel:

  get_flashsvd_v15_attn_densekv_decode_mod()  -> flashsvd_amd.kernels.densekv_reconstruct
  get_flash_attn_with_kvcache()               -> flash_attn_with_kvcache below (same keyword
                                                 contract as flash-attn 2.8.3 for q_len == 1)
  call_flash_attn_with_kvcache(fn, ...)       -> signature-filtered call, as in the reference

The legacy rank-space ("sparse KV") decode kernels are resolved to flashsvd_amd.kernels.rank_decode
when that module is present; variant names are canonicalised exactly like the reference.
"""
from __future__ import annotations

import importlib
import importlib.util
import inspect
import os
from pathlib import Path
from typing import Optional

import torch

_FLASHSVD_V15_ATTN_DENSEKV_DECODE_MOD = None
_LEGACY_SPARSEKV_ATTN_MODS = None
_WORKSPACES: dict = {}


def load_module_from_path(path: Path, module_name: str):
    spec = importlib.util.spec_from_file_location(module_name, str(path))
    if spec is None or spec.loader is None:
        raise ImportError(f"Failed to load module spec from: {path}")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def maybe_kwargs(fn, kwargs):
    """Drop the keyword arguments ``fn`` does not declare."""
    try:
        params = inspect.signature(fn).parameters
    except (TypeError, ValueError):
        return kwargs
    return {k: v for k, v in kwargs.items() if k in params}


def flash_attn_with_kvcache(q, k_cache, v_cache, k=None, v=None, rotary_cos=None, rotary_sin=None, cache_seqlens=None,
                            cache_batch_idx=None, softmax_scale=None, causal=False, window_size=(-1, -1),
                            rotary_interleaved=True, num_splits=0, dropout_p=0.0):
    """Decode attention with in-place cache append, q_len == 1.

    q [B,1,H,Dh]; k_cache/v_cache [B,S,Hk,Dh] (updated in place); k,v [B,1,Hk,Dh] are rotated with
    rotary_cos/sin [S', Dh/2] at position cache_seqlens[b] (non-interleaved only), written there,
    and attention covers cache_seqlens[b]+1 keys; without k/v it covers cache_seqlens[b] keys.
    Returns [B,1,H,Dh].  A query at the last position sees every key, so ``causal`` does not
    change the result."""
    from .. import hip_ops
    if q.dim() != 4 or q.shape[1] != 1:
        raise ValueError(f"flash_attn_with_kvcache here supports q_len == 1, got q {tuple(q.shape)}")
    if rotary_cos is not None and rotary_interleaved:
        raise NotImplementedError("interleaved rotary is not implemented; pass rotary_interleaved=False")
    if tuple(window_size) != (-1, -1) or cache_batch_idx is not None or dropout_p:
        raise NotImplementedError("window_size, cache_batch_idx and dropout are not implemented")
    B, _, H, Dh = q.shape
    if cache_seqlens is None:
        raise ValueError("cache_seqlens is required")
    if not torch.is_tensor(cache_seqlens):
        cache_seqlens = torch.full((B,), int(cache_seqlens), dtype=torch.int32, device=q.device)
    cache_seqlens = cache_seqlens.to(torch.int32).contiguous()
    nsplit = int(num_splits) if num_splits and num_splits > 0 else hip_ops.pick_nsplit(k_cache.shape[1], B, H, Dh)
    key = (q.device, B, H, Dh, nsplit)
    ws = _WORKSPACES.get(key)
    if ws is None:
        ws = hip_ops.attn_workspace(B, H, Dh, nsplit, q.device)
        _WORKSPACES[key] = ws
    out = hip_ops.attn_decode_densekv(
        q[:, 0], k_cache, v_cache, cache_seqlens,
        k_new=None if k is None else k[:, 0], v_new=None if v is None else v[:, 0],
        cos=rotary_cos, sin=rotary_sin, nsplit=nsplit, workspace=ws, softmax_scale=softmax_scale)
    return out.unsqueeze(1)


def get_flash_attn_with_kvcache():
    """The attend-with-append callable of this build (never None: it does not depend on flash-attn)."""
    return flash_attn_with_kvcache


def call_flash_attn_with_kvcache(flash_attn_with_kvcache_fn, q_bmhd, k_cache_bmhd, v_cache_bmhd, *, k_bmhd=None, v_bmhd=None,
                                 cache_seqlens=None, rotary_cos=None, rotary_sin=None, causal: bool):
    params = inspect.signature(flash_attn_with_kvcache_fn).parameters
    kwargs: dict = {}
    for name, val in (("k", k_bmhd), ("v", v_bmhd), ("cache_seqlens", cache_seqlens), ("rotary_cos", rotary_cos),
                      ("rotary_sin", rotary_sin)):
        if name in params and val is not None:
            kwargs[name] = val
    if "rotary_interleaved" in params:
        kwargs["rotary_interleaved"] = False
    if "causal" in params:
        kwargs["causal"] = causal
    if "dropout_p" in params:
        kwargs["dropout_p"] = 0.0
    if "window_size" in params:
        kwargs["window_size"] = (-1, -1)
    return flash_attn_with_kvcache_fn(q_bmhd, k_cache_bmhd, v_cache_bmhd, **kwargs)


def get_flashsvd_v15_attn_densekv_decode_mod():
    global _FLASHSVD_V15_ATTN_DENSEKV_DECODE_MOD
    if _FLASHSVD_V15_ATTN_DENSEKV_DECODE_MOD is None:
        _FLASHSVD_V15_ATTN_DENSEKV_DECODE_MOD = importlib.import_module("flashsvd_amd.kernels.densekv_reconstruct")
    return _FLASHSVD_V15_ATTN_DENSEKV_DECODE_MOD


# ---- rank-space ("legacy sparse KV") decode variants ---------------------------------------------
_V15 = "flashsvd_attn_legacy_v15_sparsekv"
_V16 = "flashsvd_attn_legacy_v16_sparsekv"


def get_flashsvd_attn_legacy_sparsekv_decode_mods():
    """{variant family -> module}.  Both families resolve to the one HIP rank-space decode module."""
    global _LEGACY_SPARSEKV_ATTN_MODS
    if _LEGACY_SPARSEKV_ATTN_MODS is None:
        try:
            mod = importlib.import_module("flashsvd_amd.kernels.rank_decode")
        except ImportError as exc:
            raise ImportError(f"Failed to load any decode attention module: {exc}") from exc
        _LEGACY_SPARSEKV_ATTN_MODS = {_V15: mod, _V16: mod}
    return _LEGACY_SPARSEKV_ATTN_MODS


def get_default_flashsvd_attn_legacy_sparsekv_decode_mod():
    mods = get_flashsvd_attn_legacy_sparsekv_decode_mods()
    return mods.get(_V16) or next(iter(mods.values()))


def canonical_legacy_sparsekv_decode_variant(name: str) -> str:
    raw = str(name or "").strip().lower().replace("-", "_")
    if raw in {"", "auto"}:
        return "auto"
    if raw in {_V15, "v15", "v1.5", "1.5"}:
        return _V15
    if raw in {_V16 + "_v1", "v16_v1", "v1", "legacy"}:
        return _V16 + "_v1"
    if raw in {_V16 + "_v2", _V16, "v16_v2", "v16", "v2"}:
        return _V16 + "_v2"
    return "auto"


def available_legacy_sparsekv_decode_variants(mods) -> list[str]:
    out: list[str] = []
    m15, m16 = mods.get(_V15), mods.get(_V16)
    if m15 is not None and hasattr(m15, "DecodePackedFactors") and hasattr(m15, "flashsvd_attn_decode_packed"):
        out.append(_V15)
    if m16 is not None and hasattr(m16, "DecodePackedFactors"):
        if hasattr(m16, "flashsvd_attn_decode_packed_v1"):
            out.append(_V16 + "_v1")
        if hasattr(m16, "flashsvd_attn_decode_packed"):
            out.append(_V16 + "_v2")
    return out


def resolve_legacy_sparsekv_decode_variant(mods, variant: str):
    variant = canonical_legacy_sparsekv_decode_variant(variant)
    if variant == _V15:
        mod = mods.get(_V15)
        return (mod, getattr(mod, "flashsvd_attn_decode_packed", None)) if mod is not None else (None, None)
    if variant == _V16 + "_v1":
        mod = mods.get(_V16)
        if mod is None:
            return None, None
        return mod, getattr(mod, "flashsvd_attn_decode_packed_v1", None) or getattr(mod, "flashsvd_attn_decode_packed", None)
    if variant == _V16 + "_v2":
        mod = mods.get(_V16)
        return (mod, getattr(mod, "flashsvd_attn_decode_packed", None)) if mod is not None else (None, None)
    return None, None


def parse_legacy_sparsekv_decode_variant_map(raw: str) -> dict[int, str]:
    """"1:v15,8:v16" -> {1: canonical, 8: canonical}; malformed items are skipped."""
    table: dict[int, str] = {}
    for item in str(raw or "").split(","):
        if ":" not in item:
            continue
        left, right = item.split(":", 1)
        try:
            bs = int(left.strip())
        except ValueError:
            continue
        if bs > 0:
            table[bs] = canonical_legacy_sparsekv_decode_variant(right.strip())
    return table


def select_legacy_sparsekv_decode_variant(*, mods, hidden_states=None, bsz: int = 1, H: int = 0, Hk: int = 0, R: int = 0,
                                          Dh: int = 0, seqlen_k: int = 0, Pq_q=None, Pk=None, Pv=None, Vq=None, Vk=None,
                                          Vv=None, rotary_cos=None, rotary_sin=None, call_kwargs=None) -> str:
    """Variant choice by FLASH_SVD_DECODE_KERNEL_VARIANT / FLASH_SVD_DECODE_KERNEL_MAP, else the
    reference's static default (v1.5 family for R >= 768, else v1.6 v1).  All variants share one HIP
    kernel here, so the timing-based autotune of the reference has nothing to choose between."""
    available = available_legacy_sparsekv_decode_variants(mods)
    if not available:
        return _V16 + "_v2"
    requested = canonical_legacy_sparsekv_decode_variant(os.getenv("FLASH_SVD_DECODE_KERNEL_VARIANT", "auto"))
    if requested != "auto" and requested in available:
        return requested
    table = parse_legacy_sparsekv_decode_variant_map(os.getenv("FLASH_SVD_DECODE_KERNEL_MAP", ""))
    if int(bsz) in table and table[int(bsz)] in available:
        return table[int(bsz)]
    candidates = [v for v in (_V15, _V16 + "_v1") if v in available]
    if os.getenv("FLASH_SVD_DECODE_AUTO_INCLUDE_V2", "0") != "0" and _V16 + "_v2" in available:
        candidates.append(_V16 + "_v2")
    if not candidates:
        candidates = list(available)
    if int(R) >= 768 and _V15 in candidates:
        return _V15
    if _V16 + "_v1" in candidates:
        return _V16 + "_v1"
    return candidates[0]


# names kept for older imports
get_flashsvd_decode_attn_mods = get_flashsvd_attn_legacy_sparsekv_decode_mods
get_default_flashsvd_decode_attn_mod = get_default_flashsvd_attn_legacy_sparsekv_decode_mod
canonical_decode_variant = canonical_legacy_sparsekv_decode_variant
available_decode_variants = available_legacy_sparsekv_decode_variants
resolve_decode_variant = resolve_legacy_sparsekv_decode_variant
get_dense_token_decode_mod = get_flashsvd_v15_attn_densekv_decode_mod
parse_decode_variant_map = parse_legacy_sparsekv_decode_variant_map
select_decode_variant = select_legacy_sparsekv_decode_variant
