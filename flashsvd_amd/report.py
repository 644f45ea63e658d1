"""Acceptance tooling for the decode path: the three-mode correctness report and the main speed table.

``check``  follows the reference's benchmark/decode/check_flashsvd_decode_correctness.py (:121-157 mode flags,
           :225-322 the three runs, :400-478 the report): a model is run as *baseline* (module by module: six
           attention factor linears, chain-of-linears MLP rounding, no graph), *flash_legacy* (packed attention,
           exact-legacy MLP backend) and *flash_test* (packed attention, the MLP backend under test), each through a
           full-sequence pass, a teacher-forced decode and a greedy decode; with one sequence the persistent decode
           step is reported as a fourth row, *flash_step*.  Every mode runs on the HIP kernels.
``table``  follows benchmark/decode/collect_lowrankarena_main_table.py (:99-144 the pair of runs, :157-205 repeat
           statistics, :208-295 the markdown): baseline against production decode per checkpoint.  Checkpoints are
           local directories (nothing is downloaded).
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import statistics
import time
import traceback
from pathlib import Path
from typing import Optional, Sequence

import torch
import torch.nn.functional as F

from . import api

_MODE_ENV = ("SVDLLM_FLASH_FALLBACK", "FLASH_SVD_DISABLE_FFN", "FLASH_SVD_BASELINE_LR_KVCACHE",
             "FLASH_SVD_ENABLE_DENSE_ATTN_DECODE", "FLASH_SVD_USE_CUTLASS_ROPEATTN", "FLASH_SVD_BASELINE_DENSE_KVCACHE",
             "FLASH_SVD_REFERENCE_DENSE_ATTN", "FLASH_SVD_ENABLE_EXPERIMENTAL_FFN", "FLASH_SVD_MLP_CUDA_GRAPH",
             "FLASH_SVD_MLP_CUDA_GRAPH_SCOPE", "FLASH_SVD_FFN_BACKEND", "FLASH_SVD_DENSE_DECODE_BACKEND")


# ---------------------------------------------------------------------------------------------
# metrics
# ---------------------------------------------------------------------------------------------
def max_abs(x: torch.Tensor, y: torch.Tensor) -> float:
    return float((x.float() - y.float()).abs().max().item())


def mean_abs(x: torch.Tensor, y: torch.Tensor) -> float:
    return float((x.float() - y.float()).abs().mean().item())


def rel_linf(x: torch.Tensor, y: torch.Tensor) -> float:
    denom = float(x.float().abs().max().item())
    return 0.0 if denom == 0.0 else float((x.float() - y.float()).abs().max().item()) / denom


def cross_entropy_from_logits(logits: torch.Tensor, targets: torch.Tensor) -> float:
    return float(F.cross_entropy(logits.float().reshape(-1, logits.shape[-1]), targets.reshape(-1), reduction="mean").item())


def token_match(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a == b).to(torch.float32).mean().item())


def compare_mode(base: dict, cur: dict, full_targets: torch.Tensor, decode_targets: torch.Tensor) -> dict:
    bf, cf = base["full_logits"][:, :-1, :], cur["full_logits"][:, :-1, :]
    bd, cd = base["decode_logits"], cur["decode_logits"]
    return {"full_max_abs": max_abs(bf, cf), "full_mean_abs": mean_abs(bf, cf), "full_rel_linf": rel_linf(bf, cf),
            "full_ce": cross_entropy_from_logits(cf, full_targets),
            "decode_max_abs": max_abs(bd, cd), "decode_mean_abs": mean_abs(bd, cd), "decode_rel_linf": rel_linf(bd, cd),
            "decode_ce": cross_entropy_from_logits(cd, decode_targets),
            "greedy_token_match": token_match(cur["greedy_tokens"], base["greedy_tokens"])}


def format_mode_line(label: str, m: dict) -> str:
    return (f"- {label}: full_max_abs={m['full_max_abs']:.6g} full_mean_abs={m['full_mean_abs']:.6g} "
            f"full_rel_linf={m['full_rel_linf']:.6g} full_ce={m['full_ce']:.6f} "
            f"| decode_max_abs={m['decode_max_abs']:.6g} decode_mean_abs={m['decode_mean_abs']:.6g} "
            f"decode_rel_linf={m['decode_rel_linf']:.6g} decode_ce={m['decode_ce']:.6f} "
            f"| greedy_token_match={m['greedy_token_match']:.6f}")


# ---------------------------------------------------------------------------------------------
# modes
# ---------------------------------------------------------------------------------------------
def _set_env(name: str, value: Optional[str]) -> None:
    if value is None:
        os.environ.pop(name, None)
    else:
        os.environ[name] = value


def configure_mode(mode: str, *, backend: str, use_graph: bool = False, graph_scope: str = "mlp",
                   enable_flash_dense_attn: bool = True, enable_baseline_dense_kvcache: bool = False) -> None:
    """Environment of one report mode (values "1"/"0" like the reference's checker)."""
    mode = str(mode).strip().lower()
    if mode == "baseline":
        plan = {"SVDLLM_FLASH_FALLBACK": "1", "FLASH_SVD_DISABLE_FFN": "1", "FLASH_SVD_ENABLE_DENSE_ATTN_DECODE": "0",
                "FLASH_SVD_BASELINE_DENSE_KVCACHE": "1" if enable_baseline_dense_kvcache else "0",
                "FLASH_SVD_ENABLE_EXPERIMENTAL_FFN": "0", "FLASH_SVD_MLP_CUDA_GRAPH": "0", "FLASH_SVD_MLP_CUDA_GRAPH_SCOPE": "mlp",
                "FLASH_SVD_FFN_BACKEND": "flashsvd_mlp_dual_split_exact_legacy", "FLASH_SVD_DENSE_DECODE_BACKEND": "exact"}
    elif mode == "flash":
        plan = {"SVDLLM_FLASH_FALLBACK": "0", "FLASH_SVD_DISABLE_FFN": "0",
                "FLASH_SVD_ENABLE_DENSE_ATTN_DECODE": "1" if enable_flash_dense_attn else "0",
                "FLASH_SVD_BASELINE_DENSE_KVCACHE": "0",
                "FLASH_SVD_ENABLE_EXPERIMENTAL_FFN": "1" if api._backend_needs_experimental_ffn(backend) else "0",
                "FLASH_SVD_MLP_CUDA_GRAPH": "1" if use_graph else "0", "FLASH_SVD_MLP_CUDA_GRAPH_SCOPE": str(graph_scope),
                "FLASH_SVD_FFN_BACKEND": str(backend), "FLASH_SVD_DENSE_DECODE_BACKEND": "packed"}
    else:
        raise ValueError(f"Unsupported mode: {mode}")
    for name in ("FLASH_SVD_BASELINE_LR_KVCACHE", "FLASH_SVD_USE_CUTLASS_ROPEATTN", "FLASH_SVD_REFERENCE_DENSE_ATTN"):
        plan[name] = "0"
    for name, value in plan.items():
        _set_env(name, value)


def clear_runtime_caches(model) -> None:
    for layer in getattr(getattr(model, "model", None), "layers", None) or ():
        mlp = getattr(layer, "mlp", None)
        for name in ("_flashsvd_graph_cache", "_flashsvd_layer_graph_cache"):
            cache = getattr(mlp, name, None)
            if isinstance(cache, dict):
                cache.clear()


def _new_cache(model, batch: int, max_len: int, device, dtype):
    from .runtime.cache import FlashSVDV15DenseKVCache
    return FlashSVDV15DenseKVCache(model.config, max_batch_size=int(batch), max_cache_len=int(max_len), device=device, dtype=dtype)


@torch.inference_mode()
def run_fullseq(model, input_ids: torch.Tensor) -> torch.Tensor:
    return model(input_ids=input_ids, attention_mask=torch.ones_like(input_ids), use_cache=False).logits.detach().clone()


@torch.inference_mode()
def run_decode_teacher_forced(model, input_ids: torch.Tensor, *, prompt_len: int, decode_steps: int) -> torch.Tensor:
    """Logits [B, decode_steps, V]: prefill, then feed the GIVEN next tokens one by one."""
    dev, dtype = input_ids.device, next(iter(model.parameters())).dtype
    cache = _new_cache(model, input_ids.shape[0], input_ids.shape[1] + 4, dev, dtype)
    out = model(input_ids=input_ids[:, :prompt_len], past_key_values=cache, use_cache=True,
                cache_position=torch.arange(int(prompt_len), device=dev))
    logits = [out.logits[:, -1, :].detach().clone()]
    for step in range(int(decode_steps) - 1):
        tok = input_ids[:, prompt_len + step: prompt_len + step + 1]
        pos = torch.tensor([int(prompt_len) + step], device=dev, dtype=torch.long)
        out = model(input_ids=tok, use_cache=True, past_key_values=cache, cache_position=pos)
        logits.append(out.logits[:, -1, :].detach().clone())
    return torch.stack(logits, dim=1)


@torch.inference_mode()
def run_decode_greedy(model, input_ids: torch.Tensor, *, prompt_len: int, decode_steps: int) -> torch.Tensor:
    dev, dtype = input_ids.device, next(iter(model.parameters())).dtype
    cache = _new_cache(model, input_ids.shape[0], int(prompt_len) + int(decode_steps) + 4, dev, dtype)
    out = model(input_ids=input_ids[:, :prompt_len], past_key_values=cache, use_cache=True,
                cache_position=torch.arange(int(prompt_len), device=dev))
    nxt = out.logits[:, -1, :].argmax(dim=-1, keepdim=True)
    tokens = [nxt.detach().clone()]
    for step in range(int(decode_steps) - 1):
        pos = torch.tensor([int(prompt_len) + step], device=dev, dtype=torch.long)
        out = model(input_ids=nxt, use_cache=True, past_key_values=cache, cache_position=pos)
        nxt = out.logits[:, -1, :].argmax(dim=-1, keepdim=True)
        tokens.append(nxt.detach().clone())
    return torch.cat(tokens, dim=1)


@torch.inference_mode()
def run_step_engine(model, input_ids: torch.Tensor, *, prompt_len: int, decode_steps: int) -> dict:
    """Teacher-forced logits and greedy tokens of the persistent decode step (one sequence)."""
    from .step import PersistentDecoder
    dev, dtype = input_ids.device, next(iter(model.parameters())).dtype
    outs = {}
    for forced in (True, False):
        cache = _new_cache(model, 1, int(prompt_len) + int(decode_steps) + 4, dev, dtype)
        out = model(input_ids=input_ids[:, :prompt_len], past_key_values=cache, use_cache=True,
                    cache_position=torch.arange(int(prompt_len), device=dev))
        first = out.logits[:, -1, :]
        dec = PersistentDecoder(model, cache, max_new_tokens=int(decode_steps) + 1)
        if forced:
            logits = [first.detach().clone()]
            for step in range(int(decode_steps) - 1):
                dec.set_state(input_ids[0, prompt_len + step], int(prompt_len) + step)
                dec.step(1)
                dec.check()
                logits.append(dec.logits[None].clone())
            outs["decode_logits"] = torch.stack(logits, dim=1)
        else:
            tok0 = first.argmax(dim=-1, keepdim=True)
            dec.set_state(tok0, int(prompt_len))
            if decode_steps > 1:
                dec.step(int(decode_steps) - 1)
            outs["greedy_tokens"] = torch.cat([tok0, dec.tokens()[None, :]], dim=1) if decode_steps > 1 else tok0
    return outs


def check_decode_correctness(model, *, input_ids: torch.Tensor, prompt_len: int, decode_steps: int,
                             legacy_backend: str = "flashsvd_mlp_dual_split_exact_legacy",
                             test_backend: str = "flashsvd_mlp_dual_split_triton_v2_sm80", graph: bool = False,
                             graph_scope: str = "mlp", flash_dense_attn: bool = True, baseline_dense_kvcache: bool = False,
                             step_engine: bool = True) -> dict:
    """Run every mode and compare with the baseline.  Returns {"baseline": {...ce}, "modes": {label: metrics},
    "tokens": {label: [...]}}; the environment is restored afterwards."""
    prev = {name: os.getenv(name) for name in _MODE_ENV}
    outputs = {}
    try:
        for label, backend in (("baseline", "baseline"), ("flash_legacy", legacy_backend), ("flash_test", test_backend)):
            configure_mode("baseline" if label == "baseline" else "flash", backend=backend, use_graph=graph, graph_scope=graph_scope,
                           enable_flash_dense_attn=flash_dense_attn, enable_baseline_dense_kvcache=baseline_dense_kvcache)
            clear_runtime_caches(model)
            torch.cuda.synchronize()
            outputs[label] = {
                "full_logits": run_fullseq(model, input_ids[:, :prompt_len]),
                "decode_logits": run_decode_teacher_forced(model, input_ids, prompt_len=prompt_len, decode_steps=decode_steps),
                "greedy_tokens": run_decode_greedy(model, input_ids, prompt_len=prompt_len, decode_steps=decode_steps)}
        if step_engine and input_ids.shape[0] == 1:
            try:
                outputs["flash_step"] = dict(run_step_engine(model, input_ids, prompt_len=prompt_len, decode_steps=decode_steps),
                                             full_logits=outputs["flash_test"]["full_logits"])
            except (ValueError, TypeError) as exc:          # a model shape the persistent step does not take
                outputs["flash_step_skipped"] = f"{type(exc).__name__}: {exc}"
    finally:
        for name, value in prev.items():
            _set_env(name, value)
    full_targets = input_ids[:, 1:prompt_len]
    decode_targets = input_ids[:, prompt_len: prompt_len + int(decode_steps)]
    base = outputs["baseline"]
    report = {"baseline": {"full_seq_ce": cross_entropy_from_logits(base["full_logits"][:, :-1, :], full_targets),
                           "decode_ce": cross_entropy_from_logits(base["decode_logits"], decode_targets)},
              "modes": {}, "tokens": {"baseline": base["greedy_tokens"][0].tolist()}}
    for label in ("flash_legacy", "flash_test", "flash_step"):
        if label in outputs:
            report["modes"][label] = compare_mode(base, outputs[label], full_targets, decode_targets)
            report["tokens"][label] = outputs[label]["greedy_tokens"][0].tolist()
    if "flash_step_skipped" in outputs:
        report["flash_step_skipped"] = outputs["flash_step_skipped"]
    return report


def format_correctness_report(report: dict, *, header: str = "", print_tokens: bool = True) -> list[str]:
    lines = ["==== FlashSVD Decode Correctness ===="]
    if header:
        lines.append(header)
    lines.append(f"baseline full_seq_ce={report['baseline']['full_seq_ce']:.6f} decode_ce={report['baseline']['decode_ce']:.6f}")
    lines += [format_mode_line(label, m) for label, m in report["modes"].items()]
    if "flash_step_skipped" in report:
        lines.append(f"- flash_step: skipped ({report['flash_step_skipped']})")
    if print_tokens:
        lines.append("Greedy token ids:")
        lines += [f"- {label:<12}: {toks}" for label, toks in report["tokens"].items()]
    return lines


def build_input_ids(model, tokenizer, *, prompt_text: Optional[str], prompt_len: int, decode_steps: int, batch_size: int,
                    add_special_tokens: bool, device) -> tuple:
    """(ids [B, prompt+steps], prompt_len, from_text): the prompt is the given text or random ids; the teacher-forced
    continuation is random ids (check_flashsvd_decode_correctness.py:46-91)."""
    vocab = int(getattr(model.config, "vocab_size", 32000))
    if prompt_text is None:
        total = int(prompt_len) + int(decode_steps)
        return torch.randint(0, vocab, (int(batch_size), total), device=device, dtype=torch.long), int(prompt_len), False
    if tokenizer is None:
        raise ValueError("a text prompt needs a tokenizer")
    prompt_ids = tokenizer(prompt_text, return_tensors="pt", add_special_tokens=bool(add_special_tokens))["input_ids"]
    if prompt_ids.numel() == 0:
        raise ValueError("Tokenized prompt is empty.")
    prompt_ids = prompt_ids.to(device=device, dtype=torch.long)
    n = int(prompt_ids.shape[1])
    ids = torch.randint(0, vocab, (int(batch_size), n + int(decode_steps)), device=device, dtype=torch.long)
    ids[:, :n] = prompt_ids.repeat(int(batch_size), 1)
    return ids, n, True


# ---------------------------------------------------------------------------------------------
# main table
# ---------------------------------------------------------------------------------------------
METRIC_KEYS = ("baseline_prefill_time_s", "baseline_decode_time_s", "flash_prefill_time_s", "flash_decode_time_s",
               "baseline_prefill_tok_s", "flash_prefill_tok_s", "baseline_decode_ms", "flash_decode_ms",
               "baseline_decode_tok_s", "flash_decode_tok_s", "prefill_speedup_x", "decode_speedup_x",
               "baseline_e2e_time_s", "flash_e2e_time_s", "e2e_speedup_x")


def pair_row(baseline: dict, flashsvd: dict) -> dict:
    """One repeat: the two benchmark dicts folded into the table's columns."""
    row = {"status": "ok",
           "baseline_prefill_time_s": float(baseline["prefill_time_s"]), "baseline_decode_time_s": float(baseline["decode_time_s"]),
           "flash_prefill_time_s": float(flashsvd["prefill_time_s"]), "flash_decode_time_s": float(flashsvd["decode_time_s"]),
           "baseline_prefill_tok_s": float(baseline["prefill_tok_s"]), "flash_prefill_tok_s": float(flashsvd["prefill_tok_s"]),
           "baseline_decode_ms": float(baseline["decode_ms_per_token"]), "flash_decode_ms": float(flashsvd["decode_ms_per_token"]),
           "baseline_decode_tok_s": float(baseline["decode_tok_s"]), "flash_decode_tok_s": float(flashsvd["decode_tok_s"])}
    row["prefill_speedup_x"] = row["flash_prefill_tok_s"] / max(1e-12, row["baseline_prefill_tok_s"])
    row["decode_speedup_x"] = row["baseline_decode_ms"] / max(1e-12, row["flash_decode_ms"])
    row["baseline_e2e_time_s"] = row["baseline_prefill_time_s"] + row["baseline_decode_time_s"]
    row["flash_e2e_time_s"] = row["flash_prefill_time_s"] + row["flash_decode_time_s"]
    row["e2e_speedup_x"] = row["baseline_e2e_time_s"] / max(1e-12, row["flash_e2e_time_s"])
    return row


def aggregate_repeat_rows(repeats: list) -> dict:
    ok_rows = [row for row in repeats if row.get("status") == "ok"]
    if not ok_rows:
        first = repeats[0] if repeats else {}
        return {"status": "error", "ok_repeats": 0, "requested_repeats": len(repeats),
                "error": first.get("error", "all repeats failed"), "traceback": first.get("traceback")}
    summary = {"status": "ok" if len(ok_rows) == len(repeats) else "partial", "ok_repeats": len(ok_rows),
               "requested_repeats": len(repeats)}
    for key in METRIC_KEYS:
        values = [float(row[key]) for row in ok_rows]
        summary[key] = float(statistics.fmean(values))
        summary[f"{key}_std"] = float(statistics.stdev(values)) if len(values) > 1 else 0.0
        summary[f"{key}_min"] = float(min(values))
        summary[f"{key}_max"] = float(max(values))
    return summary


def _ff(value, digits: int = 3) -> str:
    return f"{float(value):.{digits}f}"


def build_markdown(*, results: list, config: dict, md_path) -> str:
    L = ["# LowRankArena Main Table Results", "", f"Generated: {time.strftime('%Y-%m-%d %H:%M:%S')}", "", "## Benchmark Config", ""]
    for label, key in (("GPU", "gpu"), ("Device", "device"), ("Dtype", "dtype"), ("Prompt length", "prompt_len"),
                       ("New tokens", "new_tokens"), ("Warmup", "warmup"), ("Batch size", "batch_size"), ("Repeats", "repeats"),
                       ("FlashSVD MLP backend", "ffn_backend"), ("Decode engine", "decode_engine")):
        L.append(f"- {label}: `{config.get(key)}`")
    L += ["- Compare mode: baseline dense-KV (module by module, no graph) vs FlashSVD production packed path", "", "## Main Table", "",
          "| Family | Ratio | n | Baseline Prefill (s) | FlashSVD Prefill (s) | Prefill Speedup | Baseline Decode (ms/token) | "
          "FlashSVD Decode (ms/token) | Decode Speedup | Baseline E2E (s) | FlashSVD E2E (s) | E2E Speedup |",
          "| --- | ---: | ---: | ---: | ---: | ---: | ---: | ---: | ---: | ---: | ---: | ---: |"]
    for row in results:
        if row["status"] == "error":
            L.append(f"| {row['family_name']} | {row['ratio']} | 0/{row.get('requested_repeats', 0)} |" + " fail |" * 9)
            continue
        L.append(f"| {row['family_name']} | {row['ratio']} | {row['ok_repeats']}/{row['requested_repeats']} | "
                 f"{_ff(row['baseline_prefill_time_s'])} | {_ff(row['flash_prefill_time_s'])} | "
                 f"{_ff(row['prefill_speedup_x'], 2)}x ± {_ff(row['prefill_speedup_x_std'], 2)} | "
                 f"{_ff(row['baseline_decode_ms'])} | {_ff(row['flash_decode_ms'])} | "
                 f"{_ff(row['decode_speedup_x'], 2)}x ± {_ff(row['decode_speedup_x_std'], 2)} | "
                 f"{_ff(row['baseline_e2e_time_s'])} | {_ff(row['flash_e2e_time_s'])} | "
                 f"{_ff(row['e2e_speedup_x'], 2)}x ± {_ff(row['e2e_speedup_x_std'], 2)} |")
    L += ["", "## Detailed Throughput", "",
          "| Family | Ratio | n | Baseline Prefill Tok/s | FlashSVD Prefill Tok/s | Baseline Decode Tok/s | FlashSVD Decode Tok/s | Checkpoint |",
          "| --- | ---: | ---: | ---: | ---: | ---: | ---: | --- |"]
    for row in results:
        if row["status"] == "error":
            L.append(f"| {row['family_name']} | {row['ratio']} | 0/{row.get('requested_repeats', 0)} |" + " fail |" * 4
                     + f" `{row.get('checkpoint', '')}` |")
            continue
        L.append(f"| {row['family_name']} | {row['ratio']} | {row['ok_repeats']}/{row['requested_repeats']} | "
                 f"{_ff(row['baseline_prefill_tok_s'], 0)} | {_ff(row['flash_prefill_tok_s'], 0)} | "
                 f"{_ff(row['baseline_decode_tok_s'], 0)} | {_ff(row['flash_decode_tok_s'], 0)} | `{row['checkpoint']}` |")
    L += ["", "## Per-repeat Results", "",
          "| Family | Ratio | Repeat | Prefill Speedup | Decode Speedup | E2E Speedup | Baseline Decode (ms/token) | "
          "FlashSVD Decode (ms/token) | Status |", "| --- | ---: | ---: | ---: | ---: | ---: | ---: | ---: | --- |"]
    for row in results:
        for rep in row.get("repeats", []):
            if rep.get("status") != "ok":
                L.append(f"| {row['family_name']} | {row['ratio']} | {rep.get('repeat_index', '?')} |" + " fail |" * 5
                         + f" {rep.get('error', 'error')} |")
                continue
            L.append(f"| {row['family_name']} | {row['ratio']} | {rep['repeat_index']} | {_ff(rep['prefill_speedup_x'], 2)}x | "
                     f"{_ff(rep['decode_speedup_x'], 2)}x | {_ff(rep['e2e_speedup_x'], 2)}x | {_ff(rep['baseline_decode_ms'])} | "
                     f"{_ff(rep['flash_decode_ms'])} | ok |")
    failed = [row for row in results if row["status"] != "ok"]
    if failed:
        L += ["", "## Failures", ""] + [f"- `{row['family_name']} {row['ratio']}`: `{row.get('error')}`" for row in failed]
    L += ["", f"_Saved to `{md_path}`._"]
    return "\n".join(L)


def run_pair(model, *, prompt_len: int, new_tokens: int, warmup: int, batch_size: int, ffn_backend: str, device="cuda"):
    """(baseline, flashsvd) benchmark dicts of one model: module-by-module eager decode against the production path."""
    prev = {name: os.getenv(name) for name in _MODE_ENV + ("FLASHSVD_AMD_DECODE_ENGINE",)}
    try:
        configure_mode("baseline", backend="baseline", enable_baseline_dense_kvcache=True)
        clear_runtime_caches(model)
        baseline = api.decode_kvcache_eval(model, prompt_len=prompt_len, new_tokens=new_tokens, warmup=warmup, batch_size=batch_size,
                                           device=device, flashsvd_dense_cache=False, baseline_dense_kvcache=True, use_graph=False)
        configure_mode("flash", backend=ffn_backend, use_graph=True)
        clear_runtime_caches(model)
        flashsvd = api.decode_kvcache_eval(model, prompt_len=prompt_len, new_tokens=new_tokens, warmup=warmup, batch_size=batch_size,
                                           device=device, use_graph=True)
    finally:
        for name, value in prev.items():
            _set_env(name, value)
    return baseline, flashsvd


def parse_checkpoint_specs(raw: str) -> list:
    """"Family name:ratio=/path,Family:ratio=/path" -> [(family_name, ratio, path)]."""
    out = []
    for part in str(raw).split(","):
        part = part.strip()
        if not part:
            continue
        if "=" not in part:
            raise ValueError(f"checkpoint spec {part!r}: expected 'Family:ratio=/path'")
        left, path = part.split("=", 1)
        family, _, ratio = left.partition(":")
        out.append((family.strip() or "model", ratio.strip() or "-", path.strip()))
    if not out:
        raise ValueError("no checkpoints given")
    return out


def collect_main_table(specs: Sequence[tuple], *, load, repeats: int = 1, prompt_len: int = 512, new_tokens: int = 32, warmup: int = 3,
                       batch_size: int = 1, ffn_backend: str = "flashsvd_mlp_dual_split_prod", device="cuda") -> list:
    """Rows for ``build_markdown``; ``load(path)`` returns the model.  A failing checkpoint or repeat becomes an
    error row and the run goes on."""
    results = []
    for family, ratio, path in specs:
        row = {"family_id": family.lower().replace(" ", "_"), "family_name": family, "ratio": ratio, "checkpoint": str(path)}
        try:
            model = load(path)
            reps = []
            for idx in range(1, int(repeats) + 1):
                rep = {"repeat_index": idx, "checkpoint": str(path)}
                try:
                    rep.update(pair_row(*run_pair(model, prompt_len=prompt_len, new_tokens=new_tokens, warmup=warmup,
                                                  batch_size=batch_size, ffn_backend=ffn_backend, device=device)))
                except Exception as exc:
                    rep.update(status="error", error=f"{type(exc).__name__}: {exc}", traceback=traceback.format_exc())
                reps.append(rep)
            row["repeats"] = reps
            row.update(aggregate_repeat_rows(reps))
            del model
            gc.collect()
            if torch.cuda.is_available():
                torch.cuda.empty_cache()
        except Exception as exc:
            row.update(status="error", error=f"{type(exc).__name__}: {exc}", traceback=traceback.format_exc())
        results.append(row)
    return results


# ---------------------------------------------------------------------------------------------
# command line
# ---------------------------------------------------------------------------------------------
def main(argv=None) -> int:
    ap = argparse.ArgumentParser("flashsvd_amd.report")
    sub = ap.add_subparsers(dest="cmd", required=True)
    c = sub.add_parser("check", help="three-mode decode correctness report")
    c.add_argument("--checkpoint", type=str, required=True)
    c.add_argument("--device", type=str, default="cuda")
    c.add_argument("--batch_size", type=int, default=1)
    c.add_argument("--prompt_len", type=int, default=512)
    c.add_argument("--decode_steps", type=int, default=32)
    c.add_argument("--prompt_text", type=str, default=None)
    c.add_argument("--prompt_file", type=str, default=None)
    c.add_argument("--add_special_tokens", action=argparse.BooleanOptionalAction, default=False)
    c.add_argument("--seed", type=int, default=0)
    c.add_argument("--legacy_backend", type=str, default="flashsvd_mlp_dual_split_exact_legacy")
    c.add_argument("--test_backend", type=str, default="flashsvd_mlp_dual_split_triton_v2_sm80")
    c.add_argument("--graph", action=argparse.BooleanOptionalAction, default=False)
    c.add_argument("--graph_scope", type=str, default="mlp", choices=["auto", "mlp", "layer_tail"])
    c.add_argument("--flash_dense_attn", action=argparse.BooleanOptionalAction, default=True)
    c.add_argument("--baseline_dense_kvcache", action=argparse.BooleanOptionalAction, default=False)
    c.add_argument("--print_tokens", action=argparse.BooleanOptionalAction, default=True)
    t = sub.add_parser("table", help="baseline against production decode per checkpoint")
    t.add_argument("--checkpoints", type=str, required=True, help="'Family:ratio=/path,...' (local directories)")
    t.add_argument("--device", type=str, default="cuda:0")
    t.add_argument("--prompt_len", type=int, default=512)
    t.add_argument("--new_tokens", type=int, default=32)
    t.add_argument("--warmup", type=int, default=3)
    t.add_argument("--batch_size", type=int, default=1)
    t.add_argument("--repeats", type=int, default=1)
    t.add_argument("--ffn_backend", type=str, default="flashsvd_mlp_dual_split_prod")
    t.add_argument("--md_out", type=str, required=True)
    t.add_argument("--json_out", type=str, required=True)
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise RuntimeError("a GPU is required.")
    from .checkpoint import get_model_from_local
    if args.cmd == "check":
        torch.manual_seed(int(args.seed))
        model = get_model_from_local(args.checkpoint, device=args.device, dtype=torch.bfloat16)
        text = args.prompt_text if args.prompt_text else (Path(args.prompt_file).read_text(encoding="utf-8") if args.prompt_file else None)
        tokenizer = None
        if text is not None:
            from transformers import AutoTokenizer
            tokenizer = AutoTokenizer.from_pretrained(args.checkpoint, local_files_only=True)
        ids, n, from_text = build_input_ids(model, tokenizer, prompt_text=text, prompt_len=args.prompt_len, decode_steps=args.decode_steps,
                                            batch_size=args.batch_size, add_special_tokens=args.add_special_tokens,
                                            device=torch.device(args.device))
        report = check_decode_correctness(model, input_ids=ids, prompt_len=n, decode_steps=args.decode_steps,
                                          legacy_backend=args.legacy_backend, test_backend=args.test_backend, graph=args.graph,
                                          graph_scope=args.graph_scope, flash_dense_attn=args.flash_dense_attn,
                                          baseline_dense_kvcache=args.baseline_dense_kvcache)
        header = (f"Config: B={args.batch_size} prompt_len={n} decode_steps={args.decode_steps} dtype=bf16 graph={int(args.graph)} "
                  f"flash_dense_attn={int(args.flash_dense_attn)} baseline_dense_kvcache={int(args.baseline_dense_kvcache)} "
                  f"test_backend={args.test_backend} prompt_source={'text' if from_text else 'random'}")
        print("\n".join(format_correctness_report(report, header=header, print_tokens=args.print_tokens)))
        return 0
    specs = parse_checkpoint_specs(args.checkpoints)
    results = collect_main_table(specs, load=lambda p: get_model_from_local(p, device=args.device, dtype=torch.bfloat16),
                                 repeats=args.repeats, prompt_len=args.prompt_len, new_tokens=args.new_tokens, warmup=args.warmup,
                                 batch_size=args.batch_size, ffn_backend=args.ffn_backend, device=args.device)
    json_path, md_path = Path(args.json_out), Path(args.md_out)
    json_path.parent.mkdir(parents=True, exist_ok=True)
    json_path.write_text(json.dumps(results, indent=2), encoding="utf-8")
    md_path.parent.mkdir(parents=True, exist_ok=True)
    config = {"gpu": torch.cuda.get_device_name(0), "device": args.device, "dtype": "bf16", "prompt_len": args.prompt_len,
              "new_tokens": args.new_tokens, "warmup": args.warmup, "batch_size": args.batch_size, "repeats": args.repeats,
              "ffn_backend": args.ffn_backend, "decode_engine": os.getenv("FLASHSVD_AMD_DECODE_ENGINE", "auto")}
    text = build_markdown(results=results, config=config, md_path=md_path)
    md_path.write_text(text, encoding="utf-8")
    print(text)
    print(f"\nJSON saved to {json_path}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
