"""Serving-side API: runtime configuration by environment flags, the manual decode step, greedy /
sampled generation and the decode benchmark.

Mirrors the public surface of the reference's scripts/demo_support/api.py (:21-143 flags,
:146-177 cast, :192-404 generation) and utils/evaluator.py (:30-82 manual decode step, :271-540
decode_kvcache_eval).  Flag semantics are identical: a flag is the string "1" or absent (never
"0"), values are stored verbatim, truthiness is membership in {1,true,yes,y,on}.
"""
from __future__ import annotations

import os
import time
from types import SimpleNamespace
from typing import Any, Optional

import torch
import torch.nn.functional as F

_RUNTIME_ENV_VARS = (
    "SVDLLM_FLASH_FALLBACK",
    "FLASH_SVD_DISABLE_FFN",
    "FLASH_SVD_BASELINE_LR_KVCACHE",
    "FLASH_SVD_ENABLE_DENSE_ATTN_DECODE",
    "FLASH_SVD_DENSE_DECODE_BACKEND",
    "FLASH_SVD_DENSE_DECODE_GRAPH",
    "FLASH_SVD_DENSE_DECODE_AUTOTUNE_SCOPE",
    "FLASH_SVD_USE_CUTLASS_ROPEATTN",
    "FLASH_SVD_BASELINE_DENSE_KVCACHE",
    "FLASH_SVD_REFERENCE_DENSE_ATTN",
    "FLASH_SVD_ENABLE_EXPERIMENTAL_FFN",
    "FLASH_SVD_MLP_CUDA_GRAPH",
    "FLASH_SVD_MLP_CUDA_GRAPH_ALIAS_OUTPUT",
    "FLASH_SVD_MLP_CUDA_GRAPH_SCOPE",
    "FLASH_SVD_FFN_BACKEND",
)

_EXPERIMENTAL_FFN_BACKENDS = frozenset({
    "flashsvd_mlp_dual_split_prod", "flashsvd_mlp_dual_split_cutlass", "flashsvd_mlp_dual_split_triton_v1",
    "flashsvd_mlp_dual_split_triton_v2", "flashsvd_mlp_dual_split_triton_v2_sm80", "flashsvd_mlp_dual_split_triton_v3",
    "dual_split_cublas", "dual_split_cutlass", "dual_split_kernel", "dual_split_kernel_v2", "dual_split_kernel_v2_sm80",
    "dual_split_kernel_v3",
})


def _put(name: str, value) -> None:
    """True -> "1", False/None -> unset, anything else -> str(value)."""
    if value is True:
        os.environ[name] = "1"
    elif value is False or value is None:
        os.environ.pop(name, None)
    else:
        os.environ[name] = str(value)


def _backend_needs_experimental_ffn(backend: str) -> bool:
    return str(backend).strip().lower().replace("-", "_") in _EXPERIMENTAL_FFN_BACKENDS


def runtime_env_snapshot() -> dict[str, Optional[str]]:
    return {name: os.getenv(name) for name in _RUNTIME_ENV_VARS}


def _env_truthy(name: str) -> bool:
    return os.getenv(name, "").strip().lower() in {"1", "true", "yes", "y", "on"}


def configure_runtime(mode: str = "flashsvd", *, ffn_backend: str = "auto", enable_mlp_graph: bool = True,
                      mlp_graph_scope: str = "layer_tail", graph_alias_output: bool = False,
                      enable_flash_dense_attn: bool = True, dense_decode_backend: str = "auto",
                      enable_dense_decode_graph: bool = True, dense_decode_autotune_scope: str = "attention",
                      enable_cutlass_rope_attn: bool = False) -> dict[str, Optional[str]]:
    """Set the runtime flags for ``mode`` and return the resulting snapshot.

    "flashsvd": dense-KV decode route + fused MLP (+ graph capture flags as requested).
    "hf" / "baseline": every override off, plain-path flags on."""
    raw = str(mode).strip().lower().replace("-", "_")
    if raw not in {"flashsvd", "hf", "baseline"}:
        raise ValueError(f"Unsupported runtime mode: {mode}")
    if raw == "flashsvd":
        dense = bool(enable_flash_dense_attn)
        plan = {
            "SVDLLM_FLASH_FALLBACK": False,
            "FLASH_SVD_DISABLE_FFN": False,
            "FLASH_SVD_BASELINE_LR_KVCACHE": False,
            "FLASH_SVD_ENABLE_DENSE_ATTN_DECODE": dense,
            "FLASH_SVD_DENSE_DECODE_BACKEND": str(dense_decode_backend) if dense else None,
            "FLASH_SVD_DENSE_DECODE_GRAPH": bool(enable_dense_decode_graph) and dense,
            "FLASH_SVD_DENSE_DECODE_AUTOTUNE_SCOPE": str(dense_decode_autotune_scope) if dense else None,
            "FLASH_SVD_USE_CUTLASS_ROPEATTN": bool(enable_cutlass_rope_attn),
            "FLASH_SVD_BASELINE_DENSE_KVCACHE": False,
            "FLASH_SVD_REFERENCE_DENSE_ATTN": False,
            "FLASH_SVD_ENABLE_EXPERIMENTAL_FFN": _backend_needs_experimental_ffn(ffn_backend),
            "FLASH_SVD_MLP_CUDA_GRAPH": bool(enable_mlp_graph),
            "FLASH_SVD_MLP_CUDA_GRAPH_ALIAS_OUTPUT": bool(graph_alias_output),
            "FLASH_SVD_MLP_CUDA_GRAPH_SCOPE": str(mlp_graph_scope),
            "FLASH_SVD_FFN_BACKEND": str(ffn_backend),
        }
    else:
        plan = {name: None for name in _RUNTIME_ENV_VARS}
        plan["SVDLLM_FLASH_FALLBACK"] = True
        plan["FLASH_SVD_DISABLE_FFN"] = True
    for name in _RUNTIME_ENV_VARS:
        _put(name, plan[name])
    return runtime_env_snapshot()


def cast_model_for_inference(model: Any, *, dtype: str = "auto", device=None):
    raw = str(dtype).strip().lower()
    if device is None:
        try:
            target = next(model.parameters()).device
        except StopIteration:
            target = torch.device("cpu")
    else:
        target = torch.device(device)
    table = {"fp16": torch.float16, "float16": torch.float16, "half": torch.float16, "bf16": torch.bfloat16,
             "bfloat16": torch.bfloat16, "fp32": torch.float32, "float32": torch.float32}
    if raw == "auto":
        tdtype = torch.bfloat16 if target.type == "cuda" else torch.float32
    elif raw in table:
        tdtype = table[raw]
    else:
        raise ValueError(f"Unsupported dtype: {dtype}")
    model = model.to(device=target, dtype=tdtype)
    model.eval()
    return model


def _sample_next_token(logits: torch.Tensor, *, do_sample: bool, temperature: float, top_p: float) -> torch.Tensor:
    """Greedy argmax unless sampling is on; nucleus filtering keeps the smallest prefix of the sorted
    distribution whose mass exceeds top_p (the first token is always kept)."""
    if not do_sample or temperature <= 0.0:
        return logits.argmax(dim=-1, keepdim=True)
    probs = F.softmax(logits.float() / float(max(temperature, 1e-5)), dim=-1)
    if float(top_p) >= 1.0:
        return torch.multinomial(probs, num_samples=1)
    sp, si = torch.sort(probs, dim=-1, descending=True)
    drop = torch.cumsum(sp, dim=-1) > float(top_p)
    drop = torch.cat([torch.zeros_like(drop[..., :1]), drop[..., :-1]], dim=-1)
    sp = sp.masked_fill(drop, 0.0)
    sp = sp / sp.sum(dim=-1, keepdim=True).clamp_min(1e-12)
    return torch.gather(si, -1, torch.multinomial(sp, num_samples=1))


def _can_use_manual_llama_decode_step(model) -> bool:
    inner = getattr(model, "model", None)
    return getattr(model, "lm_head", None) is not None and all(
        getattr(inner, a, None) is not None for a in ("embed_tokens", "layers", "norm", "rotary_emb"))


def _manual_llama_decode_step(model, input_ids: torch.Tensor, *, past_key_values, cache_position: torch.Tensor,
                              attention_mask: Optional[torch.Tensor] = None):
    """embed -> every decoder layer -> final norm -> lm_head on the last position.  A query at the
    newest position attends to the whole cache, so no mask tensor is built."""
    inner = model.model
    hidden = inner.embed_tokens(input_ids)
    position_ids = cache_position.unsqueeze(0)
    n_layers = int(getattr(model.config, "num_hidden_layers", len(inner.layers)))
    for layer in inner.layers[:n_layers]:
        out = layer(hidden, attention_mask=None, position_ids=position_ids, past_key_values=past_key_values,
                    cache_position=cache_position)
        while isinstance(out, (tuple, list)) and out:
            out = out[0]
        hidden = out
    norm = inner.norm
    head_w = getattr(model.lm_head, "weight", None)
    if head_w is not None and head_w.is_cuda and head_w.dtype in (torch.bfloat16, torch.float16) and hidden.dtype == head_w.dtype \
            and getattr(model.lm_head, "bias", None) is None and hasattr(norm, "variance_epsilon"):
        from . import hip_ops   # fused final norm + lm_head
        logits = hip_ops.linear(hidden[:, -1:, :], head_w, norm_weight=norm.weight, eps=norm.variance_epsilon)
    else:
        logits = model.lm_head(norm(hidden)[:, -1:, :])
    return SimpleNamespace(logits=logits, past_key_values=past_key_values)


def _build_generation_cache(model, *, prompt_len: int, max_new_tokens: int, batch_size: int, device):
    """(cache, use_manual_decode).  The dense FlashSVD cache is used when the dense-attention decode
    route or the dense-KV baseline is switched on; this build has no other cache for its modules."""
    from .runtime.cache import FlashSVDLegacySparseKVCache, FlashSVDV15DenseKVCache
    dtype = next(iter(model.parameters())).dtype
    use_flash = _env_truthy("FLASH_SVD_ENABLE_DENSE_ATTN_DECODE") and not _env_truthy("SVDLLM_FLASH_FALLBACK")
    # the rank-space cache when the checkpoint asks for it (config side channel written by the loader,
    # utils/model_utils.py:438-439) or the rank-space baseline switch is on (utils/evaluator.py:418-456)
    use_rank = (bool(getattr(model.config, "flash_svd_use_lowrank_cache", False)) or _env_truthy("FLASH_SVD_BASELINE_LR_KVCACHE")) \
        and not use_flash
    kind = FlashSVDLegacySparseKVCache if use_rank else FlashSVDV15DenseKVCache
    cache = kind(model.config, max_batch_size=int(batch_size), max_cache_len=int(prompt_len) + int(max_new_tokens) + 4,
                 device=device, dtype=dtype)
    return cache, bool(use_flash)


@torch.no_grad()
def generate_text(model, tokenizer, *, prompt: str, max_new_tokens: int = 64, device=None, do_sample: bool = False,
                  temperature: float = 0.8, top_p: float = 0.95, use_graph: Optional[bool] = None) -> dict[str, Any]:
    """Single-prompt generation; returns text and token ids like the reference's generate_text."""
    if device is None:
        try:
            device = next(model.parameters()).device
        except StopIteration:
            device = torch.device("cpu")
    device = torch.device(device)
    if getattr(tokenizer, "pad_token_id", None) is None and getattr(tokenizer, "eos_token_id", None) is not None:
        try:
            tokenizer.pad_token = tokenizer.eos_token
        except Exception:
            pass
    if not _can_use_manual_llama_decode_step(model):
        raise TypeError("generate_text needs a Llama-style model (model.embed_tokens/layers/norm/rotary_emb, lm_head)")
    enc = tokenizer(prompt, return_tensors="pt", add_special_tokens=False)
    input_ids = enc["input_ids"].to(device)
    if int(input_ids.shape[0]) != 1:
        raise ValueError("generate_text currently supports batch_size=1 only.")
    prompt_len = int(input_ids.shape[1])
    cache, _ = _build_generation_cache(model, prompt_len=prompt_len, max_new_tokens=int(max_new_tokens), batch_size=1,
                                       device=device)
    out = model(input_ids=input_ids, past_key_values=cache, cache_position=torch.arange(prompt_len), logits_to_keep=1)
    output_ids = input_ids[0].tolist()
    eos = getattr(tokenizer, "eos_token_id", None)
    sample = dict(do_sample=bool(do_sample), temperature=float(temperature), top_p=float(top_p))
    next_token = _sample_next_token(out.logits[:, -1, :], **sample)
    if use_graph is None:
        use_graph = _env_truthy("FLASH_SVD_DENSE_DECODE_GRAPH") or _env_truthy("FLASH_SVD_MLP_CUDA_GRAPH")
    dec = None
    pdec = None
    if use_graph and not do_sample and hasattr(model, "decode_step"):
        from .graphs import GraphedDecoder
        from .step import make_persistent_decoder
        pdec = make_persistent_decoder(model, cache, 1, max_new_tokens=int(max_new_tokens) + 1)
        if pdec is not None:
            pdec.set_state(next_token, prompt_len)
        else:
            dec = GraphedDecoder(model, cache, 1)
            dec.set_state(next_token, prompt_len)
            dec.capture()
    for step in range(int(max_new_tokens)):
        tid = int(next_token.item())
        output_ids.append(tid)
        if (eos is not None and tid == int(eos)) or step + 1 >= int(max_new_tokens):
            break
        if pdec is not None:
            next_token = pdec.step_token()
        elif dec is not None:
            next_token = dec.step()
        else:
            out = _manual_llama_decode_step(model, next_token, past_key_values=cache,
                                            cache_position=torch.tensor([prompt_len + step]))
            next_token = _sample_next_token(out.logits[:, -1, :], **sample)
    if pdec is not None:
        pdec.check()      # a step that gave up waiting leaves stale token ids behind: raise instead of returning them
    completion = output_ids[prompt_len:]
    return {"prompt_token_count": prompt_len, "generated_token_count": len(completion), "output_ids": output_ids,
            "completion_ids": completion, "text": tokenizer.decode(output_ids, skip_special_tokens=False),
            "completion_text": tokenizer.decode(completion, skip_special_tokens=False)}


@torch.no_grad()
def decode_kvcache_eval(model, *, prompt_len: int = 2048, new_tokens: int = 128, batch_size: int = 1, device: str = "cuda",
                        warmup: int = 5, max_cache_len: Optional[int] = None, lowrank_cache: bool = False,
                        flashsvd_dense_cache: Optional[bool] = None, baseline_dense_kvcache: bool = False, use_graph: bool = True,
                        profile_decode: bool = False, profile_decode_steps: int = 20) -> dict:
    """Prefill a random prompt, run `warmup` untimed decode tokens, then time `new_tokens` tokens
    between two device synchronisations.  Result keys follow the reference's dict.

    Cache choice as in utils/evaluator.py:352-388: ``lowrank_cache`` decodes over the rank-space cache
    (FlashSVDLegacySparseKVCache: per-layer, possibly unequal q/k/v ranks, shaped at the first write), otherwise the
    dense cache (this build has no third, HF-static one, so ``flashsvd_dense_cache`` left unset means "dense unless
    lowrank_cache").  Two modes switched on together raise, as there."""
    from .graphs import GraphedDecoder
    from .runtime.cache import FlashSVDLegacySparseKVCache, FlashSVDV15DenseKVCache
    if flashsvd_dense_cache is None:
        flashsvd_dense_cache = not (lowrank_cache or baseline_dense_kvcache)
    if lowrank_cache and flashsvd_dense_cache:
        raise ValueError("lowrank_cache and flashsvd_dense_cache are mutually exclusive.")
    if lowrank_cache and baseline_dense_kvcache:
        raise ValueError("lowrank_cache and baseline_dense_kvcache are mutually exclusive.")
    if flashsvd_dense_cache and baseline_dense_kvcache:
        raise ValueError("flashsvd_dense_cache and baseline_dense_kvcache are mutually exclusive.")
    model.eval()
    dev = torch.device(device)
    if max_cache_len is None:
        max_cache_len = int(prompt_len) + max(0, int(warmup)) + int(new_tokens) + (int(profile_decode_steps) if profile_decode else 0) + 1
    dtype = next(iter(model.parameters())).dtype
    vocab = int(getattr(model.config, "vocab_size", 32000))
    input_ids = torch.randint(0, vocab, (int(batch_size), int(prompt_len)), device=dev, dtype=torch.long)
    kind = FlashSVDLegacySparseKVCache if lowrank_cache else FlashSVDV15DenseKVCache
    cache = kind(model.config, max_batch_size=int(batch_size), max_cache_len=int(max_cache_len), device=dev, dtype=dtype)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = model(input_ids=input_ids, past_key_values=cache, cache_position=torch.arange(int(prompt_len)), logits_to_keep=1)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    next_token = out.logits[:, -1, :].argmax(dim=-1, keepdim=True)
    from .step import make_persistent_decoder
    pdec = make_persistent_decoder(model, cache, int(batch_size), max_new_tokens=int(max_cache_len)) if use_graph else None
    if pdec is not None:
        pdec.set_state(next_token, int(prompt_len))
        step = pdec.step_token
    else:
        dec = GraphedDecoder(model, cache, int(batch_size))
        dec.set_state(next_token, int(prompt_len))
        if use_graph:
            dec.capture()
        step = dec.step if use_graph else dec.eager_step
    for _ in range(max(0, int(warmup))):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(int(new_tokens)):
        step()
    torch.cuda.synchronize()
    t_decode = time.perf_counter() - t1
    if pdec is not None:
        pdec.check()
    result = {
        "decode_engine": "persistent" if pdec is not None else ("graph" if use_graph else "eager"),
        "prompt_len": int(prompt_len), "new_tokens": int(new_tokens), "batch_size": int(batch_size),
        "prefill_time_s": float(t_prefill), "decode_time_s": float(t_decode),
        "prefill_tok_s": float(batch_size * prompt_len / t_prefill) if t_prefill > 0 else float("inf"),
        "decode_tok_s": float(batch_size * new_tokens / t_decode) if t_decode > 0 else float("inf"),
        "decode_ms_per_token": float(t_decode * 1000.0 / max(1, int(new_tokens))),
        "lowrank_cache": bool(lowrank_cache), "flashsvd_dense_cache": bool(flashsvd_dense_cache),
        "baseline_dense_kvcache": bool(baseline_dense_kvcache),
    }
    profile = None
    if profile_decode and pdec is not None:
        # one traced token: where the time of a step goes, phase by phase (events around modules, as in
        # utils/evaluator.py:553-689, cannot look inside a single launch), folded into the same categories
        result["decode_profile_us"] = pdec.phase_profile()
        profile = decode_profile_from_phases(result["decode_profile_us"], len(model.model.layers),
                                             float(result["decode_ms_per_token"]))
    elif profile_decode:
        profile = profile_decode_modules(dec, int(profile_decode_steps))
    if profile is not None:
        result["decode_profile"] = profile
    print("=== KV-Cache Prefill/Decode Benchmark ===")
    print(f"Prefill: prompt_len={prompt_len} | time {t_prefill:.3f}s | {result['prefill_tok_s']:,.0f} tok/s")
    print(f"Decode : new_tokens={new_tokens} | time {t_decode:.3f}s | {result['decode_ms_per_token']:.3f} ms/token | "
          f"{result['decode_tok_s']:,.0f} tok/s")
    if profile is not None:
        print("\n".join(format_decode_profile(profile)))
    return result


_PROFILE_CATEGORIES = ("attn_total", "mlp_total", "ln1_total", "ln2_total", "embed_tokens", "final_norm", "lm_head")


def _finish_profile(per_mod: dict, total_ms_per_tok: float, steps: int, seq: int, source: str) -> dict:
    """Fold per-module milliseconds into the reference's categories (utils/evaluator.py:646-660).  Both
    RMSNorms of a layer and the final norm run inside the projection that consumes them, so their own rows
    read zero and their time sits in attn / mlp / lm_head."""
    def suffix(sfx):
        return sum(v for k, v in per_mod.items() if k.endswith(sfx))
    breakdown = {"attn_total": suffix(".attn"), "mlp_total": suffix(".mlp"), "ln1_total": suffix(".ln1"),
                 "ln2_total": suffix(".ln2"), "embed_tokens": per_mod.get("embed_tokens", 0.0),
                 "final_norm": per_mod.get("final_norm", 0.0), "lm_head": per_mod.get("lm_head", 0.0)}
    other = max(0.0, float(total_ms_per_tok) - float(sum(breakdown.values())))
    return {"source": source, "steps": int(steps), "seq": int(seq), "total_forward_ms_per_token": float(total_ms_per_tok),
            "breakdown_ms": breakdown, "other_ms": other, "per_module_ms": dict(per_mod)}


def decode_profile_from_phases(phases_us: dict, n_layers: int, total_ms_per_tok: float) -> dict:
    """The persistent step's per-phase microseconds (averages over layers) as a per-token module profile."""
    def ms(*names):
        return sum(float(phases_us.get(n, {}).get("total", 0.0)) for n in names) / 1000.0
    # the composed form of the step takes a layer's rank projections inside other phases: the product with the hidden
    # state behind the q / k / v expansion or the SwiGLU pair (mlp_rank_x, attn_rank_x), the rest with o_u / down_u
    attn = ms("attn_rank_proj", "qkv_u", "attn", "attn_merge", "o_v", "o_u", "attn_rank_x", "down_u+attn_rank")
    mlp = ms("mlp_rank_proj", "swiglu", "down_v", "down_u", "mlp_rank_x", "o_u+mlp_rank")
    per_mod = {"embed_tokens": ms("embed"), "lm_head": ms("lm_head", "argmax")}
    for i in range(int(n_layers)):
        per_mod[f"layer{i}.attn"] = attn
        per_mod[f"layer{i}.mlp"] = mlp
    return _finish_profile(per_mod, total_ms_per_tok, 1, 0, "persistent step, one traced token")


def profile_decode_modules(dec, steps: int) -> dict:
    """Per-module device time of ``steps`` un-captured per-kernel decode tokens, measured with events recorded
    around each module's kernels on the current stream (the reference does this with forward hooks)."""
    from . import hip_ops
    model, cache = dec.model, dec.cache
    inner = model.model
    pairs: dict = {}

    def timed(name, fn):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        out = fn()
        b.record()
        pairs.setdefault(name, []).append((a, b))
        return out

    totals = []
    start_pos = int(getattr(dec, "_host_pos", 0))
    for _ in range(int(steps)):
        if getattr(dec, "_host_pos", 0) + 1 > cache.max_cache_len:
            raise IndexError(f"decode position {dec._host_pos} outside the cache (max {cache.max_cache_len})")
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        x = timed("embed_tokens", lambda: inner.embed_tokens(dec.tokens)[:, 0])
        for i, layer in enumerate(inner.layers):
            n1 = layer.input_layernorm
            x2 = timed(f"layer{i}.attn", lambda: layer.self_attn.decode_token(
                x, cache, dec.positions, norm_weight=n1.weight, eps=n1.variance_epsilon, residual=x, rope=dec.rope,
                attn_ws=dec.attn_ws, nsplit=dec.nsplit))
            x = timed(f"layer{i}.mlp", lambda: layer._layer_tail(x2))
        logits = timed("lm_head", lambda: hip_ops.linear(x, model.lm_head.weight, norm_weight=inner.norm.weight,
                                                          eps=inner.norm.variance_epsilon))
        dec.tokens.copy_(logits.argmax(dim=-1, keepdim=True))
        dec.positions.add_(1)
        t1.record()
        totals.append((t0, t1))
        dec._host_pos = getattr(dec, "_host_pos", 0) + 1
        cache._seen_tokens += 1
    torch.cuda.synchronize()
    n = float(max(1, int(steps)))
    per_mod = {k: sum(float(a.elapsed_time(b)) for a, b in v) / n for k, v in pairs.items()}
    total = sum(float(a.elapsed_time(b)) for a, b in totals) / n
    return _finish_profile(per_mod, total, int(steps), start_pos, "per-kernel path, events around modules")


def format_decode_profile(profile: dict, topk: int = 10) -> list[str]:
    total = float(profile["total_forward_ms_per_token"])
    pct = (lambda v: 100.0 * v / total if total > 0 else 0.0)
    lines = ["", "=== Decode Profile (module device time) ===",
             f"Avg over {profile['steps']} steps @ seq≈{profile['seq']} | total_forward {total:.3f} ms/token ({profile['source']})"]
    for k, v in sorted(profile["breakdown_ms"].items(), key=lambda kv: kv[1], reverse=True):
        lines.append(f"  {k:12s}: {v:8.3f} ms ({pct(v):5.1f}%)")
    lines.append(f"  {'other':12s}: {profile['other_ms']:8.3f} ms ({pct(profile['other_ms']):5.1f}%)")
    top = sorted(((k, v) for k, v in profile["per_module_ms"].items() if v > 0), key=lambda kv: kv[1], reverse=True)[:topk]
    if top:
        lines.append(f"Top {len(top)}/{topk} modules:")
        lines += [f"  {name:16s}: {ms:8.3f} ms ({pct(ms):5.1f}%)" for name, ms in top]
    lines.append("")
    return lines


def enable_flashsvd_llama_layer_tail_cuda_graph() -> None:
    """Process-global and idempotent, like the patch of the same name in the reference (called from
    utils/model_utils.py:768-786 and benchmark/mlp/bench_svd_llama_decode_graph.py:227): transformers'
    LlamaDecoderLayer, used unmodified with SVD_LlamaMLP (and SVD_LlamaAttention) swapped in, and this package's own
    decoder layer run "residual + post-attention norm + MLP + residual" as one captured graph when
    FLASH_SVD_MLP_CUDA_GRAPH is on with scope layer_tail (or auto)."""
    from . import llama
    llama.LAYER_TAIL_GRAPH_ENABLED = True
    llama.patch_hf_llama_decoder_layer()


__all__ = ["cast_model_for_inference", "configure_runtime", "decode_kvcache_eval", "generate_text", "runtime_env_snapshot",
           "enable_flashsvd_llama_layer_tail_cuda_graph"]
