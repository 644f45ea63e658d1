"""Per-layer dense-decode plan: rank padding, backend candidates, measurement and the plan file.

Follows the reference's benchmark/attn/generate_dense_decode_plan.py (candidate rules :59-150, selection and
file layout :312-462) and the per-layer reconstruct benchmark it builds on
(benchmark/attn/bench_real_checkpoint_decode_reconstruct.py:92-257, environment knobs :283-285).

Why padding matters on this hardware: the weight-streaming kernels read rows in 16-byte pieces, so a rank that
is not a multiple of 8 falls back to element-wise loads, the matrix-core paths need multiples of 32 and the
persistent decode step multiples of 128.  Real checkpoints carry ranks such as 1492.  Padding appends ZERO rows
to ``v_proj`` and ZERO columns to ``u_proj``: the extra coefficients are exactly 0 and contribute exactly 0 to
every fp32 sum, so the only numerical effect is a different split of the sums over lanes (fp32 reassociation).

Two backends exist for the current-token attention block, like the reference's:
  exact   six separate factor linears, then attend-with-append (rotary and cache write inside attention);
  packed  one row-packed rank projection, fused head expansion + RoPE + cache append, then attention.
"""
from __future__ import annotations

import argparse
import copy
import json
import os
from collections import Counter
from pathlib import Path
from typing import Iterable, Optional, Sequence

import torch
import torch.nn as nn

PLAN_FORMAT_RECONSTRUCT = "flashsvd_dense_decode_plan_v1"
PLAN_FORMAT_ATTENTION = "flashsvd_dense_decode_plan_v2"
PAD_MODES = ("independent", "uniform_layer")
BACKENDS = ("exact", "packed")


# ---------------------------------------------------------------------------------------------
# parsing helpers (generate_dense_decode_plan.py:28-58)
# ---------------------------------------------------------------------------------------------
def parse_pad_multiples(raw) -> list[int]:
    out: list[int] = []
    for part in str(raw).split(","):
        part = part.strip()
        if not part:
            continue
        value = max(1, int(part))
        if value not in out:
            out.append(value)
    return out or [1, 8, 16, 32, 64]


def parse_int_list(raw, *, default: Sequence[int]) -> list[int]:
    out: list[int] = []
    for part in str(raw).split(","):
        part = part.strip()
        if not part:
            continue
        value = int(part)
        if value not in out:
            out.append(value)
    return out or list(default)


def is_finite_number(value) -> bool:
    try:
        value = float(value)
    except Exception:
        return False
    return value == value and value not in (float("inf"), float("-inf"))


# ---------------------------------------------------------------------------------------------
# rank padding
# ---------------------------------------------------------------------------------------------
def padded_ranks(ranks: Iterable[int], multiple: int, mode: str = "independent") -> tuple:
    """Each rank rounded up to ``multiple``; "uniform_layer" then lifts all of them to the largest."""
    mode = str(mode).strip().lower()
    if mode not in PAD_MODES:
        raise ValueError(f"pad mode {mode!r}: expected one of {PAD_MODES}")
    mult = max(1, int(multiple))
    out = [(int(r) + mult - 1) // mult * mult for r in ranks]
    if mode == "uniform_layer":
        out = [max(out)] * len(out)
    return tuple(out)


def _padded_weight(w: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    if tuple(w.shape) == (rows, cols):
        return w
    out = w.new_zeros(rows, cols)
    out[: w.shape[0], : w.shape[1]] = w
    return out


def pad_factor_pair(v_lin: nn.Linear, u_lin: nn.Linear, new_rank: int, _shared: Optional[dict] = None) -> bool:
    """Grow the rank of ``u_lin(v_lin(x))`` to ``new_rank`` with zero rows of v and zero columns of u, in place.
    ``_shared`` maps id(old weight) -> padded Parameter so that weights shared between layers stay shared."""
    r = int(v_lin.weight.shape[0])
    if int(u_lin.weight.shape[1]) != r:
        raise ValueError(f"factor pair does not chain: v {tuple(v_lin.weight.shape)}, u {tuple(u_lin.weight.shape)}")
    if new_rank < r:
        raise ValueError(f"cannot pad rank {r} down to {new_rank}")
    if new_rank == r:
        return False
    shared = {} if _shared is None else _shared
    for lin, shape in ((v_lin, (new_rank, v_lin.weight.shape[1])), (u_lin, (u_lin.weight.shape[0], new_rank))):
        key = id(lin.weight)
        if key not in shared:
            shared[key] = nn.Parameter(_padded_weight(lin.weight.data, *shape), requires_grad=False)
        elif tuple(shared[key].shape) != tuple(shape):
            raise ValueError("a weight shared between layers would need two different paddings")
        lin.weight = shared[key]
        lin.in_features, lin.out_features = int(shape[1]), int(shape[0])
    if getattr(v_lin, "bias", None) is not None:
        v_lin.bias = nn.Parameter(torch.cat([v_lin.bias.data, v_lin.bias.data.new_zeros(new_rank - r)]), requires_grad=False)
    return True


def pad_attention_ranks(attn, multiple: int = 1, mode: str = "independent", *, split_sizes=None, pad_o: bool = True,
                        _shared: Optional[dict] = None) -> dict:
    """Pad q/k/v (and o) of one attention module; ``split_sizes`` overrides the q/k/v targets."""
    actual = tuple(int(getattr(attn, f"{p}_v_proj").weight.shape[0]) for p in ("q", "k", "v"))
    if not hasattr(attn, "_unpadded_qkv_ranks"):
        attn._unpadded_qkv_ranks = actual
    target = tuple(int(s) for s in split_sizes) if split_sizes is not None else padded_ranks(actual, multiple, mode)
    report = {}
    for p, r, t in zip(("q", "k", "v"), actual, target):
        pad_factor_pair(getattr(attn, f"{p}_v_proj"), getattr(attn, f"{p}_u_proj"), t, _shared)
        report[p] = (r, t)
    if pad_o:
        ro = int(attn.o_v_proj.weight.shape[0])
        to = padded_ranks((ro,), multiple)[0]
        pad_factor_pair(attn.o_v_proj, attn.o_u_proj, to, _shared)
        report["o"] = (ro, to)
    attn.low_rank = int(attn.k_v_proj.weight.shape[0])
    attn._reset_runtime_state()
    return report


def pad_mlp_ranks(mlp, multiple: int = 1, *, _shared: Optional[dict] = None) -> dict:
    """gate and up keep one common rank (the SwiGLU phase streams them as a pair); down is padded on its own."""
    rg, ru, rd = (int(getattr(mlp, f"{p}_v_proj").weight.shape[0]) for p in ("gate", "up", "down"))
    tg = tu = padded_ranks((rg, ru), multiple, "uniform_layer")[0]
    td = padded_ranks((rd,), multiple)[0]
    for p, t in (("gate", tg), ("up", tu), ("down", td)):
        pad_factor_pair(getattr(mlp, f"{p}_v_proj"), getattr(mlp, f"{p}_u_proj"), t, _shared)
    mlp._packed_gu_v = None
    mlp._packed_key = None
    for name in ("_flashsvd_graph_cache", "_flashsvd_layer_graph_cache"):     # captured graphs point at the old weights
        if isinstance(getattr(mlp, name, None), dict):
            getattr(mlp, name).clear()
    return {"gate": (rg, tg), "up": (ru, tu), "down": (rd, td)}


def pad_model_ranks(model, multiple: int = 128, mode: str = "uniform_layer", *, include_mlp: bool = True) -> dict:
    """Pad every factor pair of the model in place (no second copy of the weights stays alive).
    Returns {"layers": {idx: {proj: (rank, padded)}}, "added_bytes": n}."""
    shared: dict = {}
    layers = {}
    before = _factor_bytes(model)
    for idx, layer in enumerate(model.model.layers):
        rep = pad_attention_ranks(layer.self_attn, multiple, mode, _shared=shared)
        if include_mlp:
            rep.update(pad_mlp_ranks(layer.mlp, multiple, _shared=shared))
        layers[idx] = rep
    return {"layers": layers, "added_bytes": _factor_bytes(model) - before, "multiple": int(multiple), "mode": str(mode)}


def _factor_bytes(model) -> int:
    seen, total = set(), 0
    for layer in model.model.layers:
        for blk, projs in ((layer.self_attn, ("q", "k", "v", "o")), (layer.mlp, ("gate", "up", "down"))):
            for p in projs:
                for f in ("u", "v"):
                    w = getattr(blk, f"{p}_{f}_proj").weight
                    if id(w) not in seen:
                        seen.add(id(w))
                        total += w.numel() * w.element_size()
    return total


# ---------------------------------------------------------------------------------------------
# candidates and selection (pure functions)
# ---------------------------------------------------------------------------------------------
def build_candidates(*, layer_idx: int, actual_ranks, result: dict, pad_multiple: int, include_exact: bool) -> list[dict]:
    """Reconstruct-mode candidates of one (layer, pad multiple) measurement: ``exact`` once, ``packed_linear``
    while the split sizes equal the real ranks, ``packed_flat`` once padding changed them."""
    actual_ranks = tuple(int(v) for v in actual_ranks)
    candidates = []
    exact_ms = float(result["exact_ms"])
    if include_exact:
        candidates.append(dict(layer=int(layer_idx), backend="exact", impl="exact", split_sizes=list(actual_ranks),
                               pad_multiple=1, ms=exact_ms, speedup_vs_exact=1.0))
    split_sizes = (int(result["rq"]), int(result["rk"]), int(result["rv"]))
    packed_linear_ms = float(result["packed_linear_ms"])
    packed_flat_ms = float(result["packed_torch_ms"])
    if split_sizes == actual_ranks and is_finite_number(packed_linear_ms):
        candidates.append(dict(layer=int(layer_idx), backend="packed", impl="packed_linear", split_sizes=list(split_sizes),
                               pad_multiple=int(pad_multiple), ms=packed_linear_ms,
                               speedup_vs_exact=exact_ms / max(packed_linear_ms, 1e-9)))
    if (split_sizes != actual_ranks or not is_finite_number(packed_linear_ms)) and is_finite_number(packed_flat_ms):
        candidates.append(dict(layer=int(layer_idx), backend="packed", impl="packed_flat", split_sizes=list(split_sizes),
                               pad_multiple=int(pad_multiple), ms=packed_flat_ms,
                               speedup_vs_exact=exact_ms / max(packed_flat_ms, 1e-9)))
    return candidates


def build_attention_candidates(*, layer_idx: int, actual_ranks, split_sizes, exact_ms: float, packed_ms: float,
                               pad_multiple: int) -> list[dict]:
    return [
        dict(layer=int(layer_idx), backend="exact", impl="exact_attention", split_sizes=[int(v) for v in actual_ranks],
             pad_multiple=1, ms=float(exact_ms), speedup_vs_exact=1.0),
        dict(layer=int(layer_idx), backend="packed", impl="packed_attention", split_sizes=[int(v) for v in split_sizes],
             pad_multiple=int(pad_multiple), ms=float(packed_ms), speedup_vs_exact=float(exact_ms) / max(float(packed_ms), 1e-9)),
    ]


def select_best(candidates: list[dict]) -> dict:
    """Fastest candidate; at equal time the packed backend wins."""
    return min(candidates, key=lambda c: (float(c["ms"]), 0 if str(c["backend"]) == "packed" else 1))


def _candidate_row(c: dict) -> dict:
    return dict(backend=str(c["backend"]), impl=str(c["impl"]), pad_multiple=int(c["pad_multiple"]),
                split_sizes=[int(v) for v in c["split_sizes"]], ms=float(c["ms"]), speedup_vs_exact=float(c["speedup_vs_exact"]))


def assemble_plan(measurements: dict, *, mode: str, source: dict) -> dict:
    """measurements: {layer_idx: {"actual_ranks": (rq, rk, rv), "buckets": {past_bucket: [candidates]}}}
    (reconstruct mode uses the single bucket -1).  Returns the plan in the reference's file layout."""
    attention = mode == "attention"
    layer_plan = {}
    backend_n, pad_n, bucket_n, past_n = Counter(), Counter(), Counter(), Counter()
    for layer_idx in sorted(measurements, key=int):
        m = measurements[layer_idx]
        actual = tuple(int(v) for v in m["actual_ranks"])
        bucket_plan, layer_best = {}, []
        for past_bucket, candidates in m["buckets"].items():
            best = select_best(candidates)
            bucket = "_".join(str(int(v)) for v in best["split_sizes"])
            backend_n[str(best["backend"])] += 1
            pad_n[int(best["pad_multiple"])] += 1
            bucket_n[bucket] += 1
            if attention:
                past_n[int(past_bucket)] += 1
            bucket_plan[str(int(past_bucket))] = dict(
                backend=str(best["backend"]), impl=str(best["impl"]), pad_multiple=int(best["pad_multiple"]),
                split_sizes=[int(v) for v in best["split_sizes"]], bucket=bucket, best_ms=float(best["ms"]),
                best_speedup_vs_exact=float(best["speedup_vs_exact"]),
                candidates=[_candidate_row(c) for c in sorted(candidates, key=lambda c: float(c["ms"]))])
            layer_best.append((int(past_bucket), best))
        default_bucket, default = min(layer_best, key=lambda item: float(item[1]["ms"]))
        entry = dict(layer_idx=int(layer_idx), backend=str(default["backend"]), impl=str(default["impl"]),
                     pad_multiple=int(default["pad_multiple"]), qkv_ranks=[int(v) for v in actual],
                     split_sizes=[int(v) for v in default["split_sizes"]],
                     bucket="_".join(str(int(v)) for v in default["split_sizes"]), best_ms=float(default["ms"]),
                     best_speedup_vs_exact=float(default["speedup_vs_exact"]))
        if attention:
            entry["buckets"] = bucket_plan
            entry["default_past_bucket"] = int(default_bucket)
        else:
            entry["candidates"] = bucket_plan[str(-1)]["candidates"]
        layer_plan[str(int(layer_idx))] = entry
    return {
        "format": PLAN_FORMAT_ATTENTION if attention else PLAN_FORMAT_RECONSTRUCT,
        "source": dict(source),
        "defaults": {"backend": backend_n.most_common(1)[0][0] if backend_n else "packed",
                     "pad_multiple": int(pad_n.most_common(1)[0][0]) if pad_n else 16},
        "summary": {"backend_counts": dict(backend_n), "pad_counts": {str(k): int(v) for k, v in pad_n.items()},
                    "bucket_counts": dict(bucket_n), "past_bucket_counts": {str(k): int(v) for k, v in past_n.items()}},
        "layers": layer_plan,
    }


def save_plan(plan: dict, path) -> Path:
    path = Path(path).resolve()
    path.parent.mkdir(parents=True, exist_ok=True)
    path.write_text(json.dumps(plan, indent=2, sort_keys=True) + "\n")
    return path


def load_plan(path) -> dict:
    plan = json.loads(Path(path).read_text())
    if not isinstance(plan, dict) or plan.get("format") not in (PLAN_FORMAT_RECONSTRUCT, PLAN_FORMAT_ATTENTION):
        raise ValueError(f"{path} is not a dense-decode plan (format {plan.get('format') if isinstance(plan, dict) else None!r})")
    if not isinstance(plan.get("layers"), dict):
        raise ValueError(f"{path}: plan has no layer table")
    return plan


def plan_choice(entry: Optional[dict], past_len: Optional[int] = None) -> str:
    """Backend of a layer entry for the given number of cached keys: the bucket with the largest past length
    not above ``past_len`` (the smallest bucket before that), else the layer default."""
    if not entry:
        return "packed"
    buckets = entry.get("buckets")
    if isinstance(buckets, dict) and buckets and past_len is not None:
        keys = sorted(int(k) for k in buckets)
        below = [k for k in keys if k <= int(past_len)]
        return _backend_name(buckets[str(below[-1] if below else keys[0])].get("backend"))
    return _backend_name(entry.get("backend"))


def _backend_name(raw) -> str:
    name = str(raw or "packed").strip().lower()
    if name == "auto":
        return "packed"
    if name not in BACKENDS:
        raise ValueError(f"dense-decode backend {raw!r}: expected auto, exact or packed")
    return name


def apply_dense_decode_plan(model, plan: dict, *, pad: bool = True) -> dict:
    """Install a plan: every planned attention layer gets its backend table and (``pad``) its q/k/v factors are
    padded in place to the plan's split sizes.  Layers the plan does not name follow its defaults.
    Returns {layer: (backend, split_sizes)}."""
    layers = model.model.layers
    out = {}
    shared: dict = {}
    defaults = plan.get("defaults") or {}
    for idx, layer in enumerate(layers):
        attn = layer.self_attn
        entry = plan["layers"].get(str(idx))
        if entry is None:
            entry = {"backend": defaults.get("backend", "packed"), "pad_multiple": int(defaults.get("pad_multiple", 1))}
            split = padded_ranks(attn._qkv_rank_tuple(), entry["pad_multiple"]) if pad else attn._qkv_rank_tuple()
        else:
            actual = tuple(int(v) for v in entry.get("qkv_ranks", attn._qkv_rank_tuple()))
            have = tuple(getattr(attn, "_unpadded_qkv_ranks", attn._qkv_rank_tuple()))
            if actual != have:
                raise ValueError(f"plan layer {idx} was measured for ranks {actual}, the model has {have}")
            split = tuple(int(v) for v in entry["split_sizes"]) if pad else attn._qkv_rank_tuple()
        _backend_name(entry.get("backend"))
        if pad and tuple(split) != tuple(attn._qkv_rank_tuple()):
            pad_attention_ranks(attn, split_sizes=split, pad_o=False, _shared=shared)
        attn._dense_decode_plan = entry
        attn._dense_decode_backend_cache.clear()
        out[idx] = (plan_choice(entry), tuple(attn._qkv_rank_tuple()))
    return out


# ---------------------------------------------------------------------------------------------
# measurement (GPU)
# ---------------------------------------------------------------------------------------------
def bench_ms(fn, *, warmup: int, iters: int) -> float:
    """Median of ``iters`` event-timed calls after ``warmup`` untimed ones, milliseconds."""
    for _ in range(int(warmup)):
        fn()
    torch.cuda.synchronize()
    samples = []
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(int(iters)):
        start.record()
        fn()
        end.record()
        torch.cuda.synchronize()
        samples.append(float(start.elapsed_time(end)))
    samples.sort()
    return float(samples[len(samples) // 2]) if samples else float("inf")


def clear_attn_runtime_caches(attn) -> None:
    for name in ("_decode_Vq", "_decode_Vk", "_decode_Vv"):
        setattr(attn, name, None)
    cache = getattr(attn, "_dense_decode_prepacked_cache", None)
    if isinstance(cache, dict):
        cache.clear()


def _padded_clone(attn, multiple: int, mode: str):
    """A copy of the attention module whose q/k/v ranks are padded (the original is left alone)."""
    clone = copy.copy(attn)
    clone._modules = dict(attn._modules)
    for p in ("q", "k", "v"):
        for f in ("u", "v"):
            name = f"{p}_{f}_proj"
            lin = copy.copy(getattr(attn, name))
            lin._parameters = dict(lin._parameters)
            clone._modules[name] = lin
    clone._reset_runtime_state()
    if multiple > 1 or mode != "independent":
        pad_attention_ranks(clone, multiple, mode, pad_o=False)
    return clone


def benchmark_attn_layer(attn, x: torch.Tensor, *, warmup: int, iters: int, pad_multiple: int = 1,
                         pad_mode: str = "independent") -> dict:
    """Current-token q/k/v of one layer three ways (bench_real_checkpoint_decode_reconstruct.py:92-257):
    exact = six factor linears; packed_linear = one packed rank projection + three u linears (unpadded ranks
    only); packed_flat = ``x @ packed_qkv_rank`` + prepacked reconstruct on the padded tensors.  Times in ms and
    the largest deviation of each packed form from the exact one."""
    from . import hip_ops
    from .runtime.decode_registry import get_flashsvd_v15_attn_densekv_decode_mod
    attn.eval()
    clear_attn_runtime_caches(attn)
    attn._ensure_runtime_state()
    os.environ["FLASH_SVD_DENSE_DECODE_RANK_PAD_MULTIPLE"] = str(max(1, int(pad_multiple)))
    os.environ["FLASH_SVD_DENSE_DECODE_PAD_MODE"] = str(pad_mode)
    packed_qkv_rank, vq_flat, vk_flat, vv_flat, split_sizes = attn._get_dense_decode_tensors(device=x.device, dtype=x.dtype)
    actual = attn._qkv_rank_tuple()
    rq, rk, rv = (int(v) for v in split_sizes)
    can_use_linear = (rq, rk, rv) == tuple(actual)
    hidden_flat = x[:, 0, :].contiguous()
    H, Hk, Dh = attn.num_heads, attn.num_key_value_heads, attn.head_dim
    mod = get_flashsvd_v15_attn_densekv_decode_mod()
    B = hidden_flat.shape[0]

    def exact_fn():
        q = hip_ops.linear(hip_ops.linear(hidden_flat, attn.q_v_proj.weight), attn.q_u_proj.weight).view(B, H, Dh)
        k = hip_ops.linear(hip_ops.linear(hidden_flat, attn.k_v_proj.weight), attn.k_u_proj.weight).view(B, Hk, Dh)
        v = hip_ops.linear(hip_ops.linear(hidden_flat, attn.v_v_proj.weight), attn.v_u_proj.weight).view(B, Hk, Dh)
        return q, k, v

    def packed_flat_fn():
        packed_rank = mod.xw_linear(hidden_flat, packed_qkv_rank)
        p_q, p_k, p_v = torch.split(packed_rank, (rq, rk, rv), dim=1)
        return mod.reconstruct_qkv_token_shared_prepacked(p_q, p_k, p_v, vq_flat, vk_flat, vv_flat, H=H, Hk=Hk, Dh=Dh)

    def packed_linear_fn():
        p = hip_ops.linear(hidden_flat, attn._packed_qkv_v)
        a0, a1, a2 = actual
        q = hip_ops.linear(p[:, :a0], attn.q_u_proj.weight).view(B, H, Dh)
        k = hip_ops.linear(p[:, a0:a0 + a1], attn.k_u_proj.weight).view(B, Hk, Dh)
        v = hip_ops.linear(p[:, a0 + a1:], attn.v_u_proj.weight).view(B, Hk, Dh)
        return q, k, v

    def diff(a, b):
        return max(float((s.float() - t.float()).abs().max()) for s, t in zip(a, b))

    ref = exact_fn()
    flat_diff = diff(packed_flat_fn(), ref)
    linear_diff = diff(packed_linear_fn(), ref) if can_use_linear else 0.0
    exact_ms = bench_ms(exact_fn, warmup=warmup, iters=iters)
    packed_flat_ms = bench_ms(packed_flat_fn, warmup=warmup, iters=iters)
    packed_linear_ms = bench_ms(packed_linear_fn, warmup=warmup, iters=iters) if can_use_linear else float("nan")
    return {
        "rq": rq, "rk": rk, "rv": rv, "hidden": int(attn.hidden_size), "heads": int(H), "kv_heads": int(Hk), "head_dim": int(Dh),
        "exact_ms": float(exact_ms),
        "packed_torch_ms": float(packed_flat_ms), "packed_torch_speedup": float(exact_ms / max(packed_flat_ms, 1e-9)),
        "packed_torch_max_diff": float(flat_diff),
        "packed_linear_ms": float(packed_linear_ms),
        "packed_linear_speedup": float(exact_ms / max(packed_linear_ms, 1e-9)) if can_use_linear else float("nan"),
        "packed_linear_max_diff": float(linear_diff),
    }


def make_dense_cache(model, attn, *, batch_size: int, past_len: int, device, dtype):
    """A cache whose first ``past_len`` rows of this layer hold random keys and values."""
    from .runtime.cache import FlashSVDV15DenseKVCache
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=int(batch_size), max_cache_len=max(int(past_len) + 16, 16),
                                    device=device, dtype=dtype)
    cache._ensure_layer_spec(int(attn.layer_idx), h=int(attn.num_key_value_heads), dh=int(attn.head_dim))
    if int(past_len) > 0:
        cache.key_cache[int(attn.layer_idx)][: int(batch_size), : int(past_len)].normal_()
        cache.value_cache[int(attn.layer_idx)][: int(batch_size), : int(past_len)].normal_()
    cache._seen_tokens = int(past_len)
    return cache


def benchmark_attn_layer_attention(model, attn, x: torch.Tensor, *, past_len: int, warmup: int, iters: int,
                                   pad_multiple: int = 1, pad_mode: str = "independent") -> dict:
    """The whole current-token attention block of one layer with each backend over ``past_len`` cached keys;
    the packed backend runs on factors padded to ``pad_multiple`` (a temporary copy of this layer's q/k/v)."""
    attn.eval()
    actual = tuple(int(v) for v in attn._qkv_rank_tuple())
    pos = torch.tensor([int(past_len)], dtype=torch.long)
    base = make_dense_cache(model, attn, batch_size=int(x.shape[0]), past_len=int(past_len), device=x.device, dtype=x.dtype)

    def runner(module, backend):
        cache = base.clone_for_autotune(layer_idx=int(attn.layer_idx), batch_size=int(x.shape[0]))
        if cache is None:
            raise RuntimeError("Failed to clone dense cache for attention benchmark.")
        module._dense_decode_plan = {"backend": backend}
        module._ensure_runtime_state()

        def call():
            return module._flashsvd_dense_decode_token_from_hidden(x, cache, cache_position=pos, cache_bindings=None,
                                                                   advance_cache=False)
        return call

    saved = getattr(attn, "_dense_decode_plan", None)
    try:
        exact_ms = bench_ms(runner(attn, "exact"), warmup=warmup, iters=iters)
        padded = _padded_clone(attn, int(pad_multiple), pad_mode)
        split = tuple(int(v) for v in padded._qkv_rank_tuple())
        packed_ms = bench_ms(runner(padded, "packed"), warmup=warmup, iters=iters)
        del padded
    finally:
        attn._dense_decode_plan = saved
    return {"exact_ms": float(exact_ms), "packed_ms": float(packed_ms), "rq": split[0], "rk": split[1], "rv": split[2],
            "actual_rq": actual[0], "actual_rk": actual[1], "actual_rv": actual[2]}


def generate_dense_decode_plan(model, *, mode: str = "attention", batch_size: int = 1, layers: Optional[Sequence[int]] = None,
                               warmup: int = 5, iters: int = 20, past_buckets: Sequence[int] = (0, 512),
                               pad_multiples: Sequence[int] = (1, 8, 16, 32, 64), pad_mode: str = "independent",
                               device="cuda", dtype=torch.bfloat16, checkpoint: str = "", log=print) -> dict:
    """Measure every candidate of every layer and return the plan (generate_dense_decode_plan.py:259-462)."""
    if mode not in ("reconstruct", "attention"):
        raise ValueError(f"mode {mode!r}: expected reconstruct or attention")
    if not torch.cuda.is_available():
        raise RuntimeError("a GPU is required for plan generation.")
    padded_ranks((1,), 1, pad_mode)
    attn_layers = [layer.self_attn for layer in model.model.layers]
    layer_indices = list(range(len(attn_layers))) if layers is None else [int(i) for i in layers]
    saved_env = {k: os.environ.get(k) for k in ("FLASH_SVD_DENSE_DECODE_RANK_PAD_MULTIPLE", "FLASH_SVD_DENSE_DECODE_PAD_MODE")}
    measurements = {}
    try:
        for layer_idx in layer_indices:
            attn = attn_layers[layer_idx]
            actual = tuple(int(v) for v in attn._qkv_rank_tuple())
            buckets = {}
            for past_bucket in (past_buckets if mode == "attention" else [-1]):
                candidates = []
                for pad_multiple in pad_multiples:
                    x = torch.randn(int(batch_size), 1, int(attn.hidden_size), device=device, dtype=dtype)
                    if mode == "attention":
                        r = benchmark_attn_layer_attention(model, attn, x, past_len=int(past_bucket), warmup=warmup, iters=iters,
                                                           pad_multiple=int(pad_multiple), pad_mode=pad_mode)
                        candidates.extend(build_attention_candidates(
                            layer_idx=layer_idx, actual_ranks=actual, split_sizes=(r["rq"], r["rk"], r["rv"]),
                            exact_ms=r["exact_ms"], packed_ms=r["packed_ms"], pad_multiple=int(pad_multiple)))
                    else:
                        r = benchmark_attn_layer(attn, x, warmup=warmup, iters=iters, pad_multiple=int(pad_multiple),
                                                 pad_mode=pad_mode)
                        candidates.extend(build_candidates(layer_idx=layer_idx, actual_ranks=actual, result=r,
                                                           pad_multiple=int(pad_multiple),
                                                           include_exact=int(pad_multiple) == int(pad_multiples[0])))
                    clear_attn_runtime_caches(attn)
                buckets[int(past_bucket)] = candidates
                best = select_best(candidates)
                tag = f"L{layer_idx:02d}" if mode != "attention" else f"L{layer_idx:02d} P{int(past_bucket):04d}"
                log(f"{tag} actual={actual[0]}/{actual[1]}/{actual[2]} best={best['backend']}:{best['impl']} "
                    f"split={tuple(best['split_sizes'])} pad={int(best['pad_multiple'])} ms={float(best['ms']):.4f} "
                    f"speedup={float(best['speedup_vs_exact']):.3f}x")
            measurements[layer_idx] = {"actual_ranks": actual, "buckets": buckets}
    finally:
        for k, v in saved_env.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    source = dict(checkpoint=str(checkpoint), dtype=str(dtype).replace("torch.", ""), device=str(device), batch_size=int(batch_size),
                  warmup=int(warmup), iters=int(iters), mode=str(mode), pad_mode=str(pad_mode),
                  pad_multiples=[int(v) for v in pad_multiples], past_buckets=[int(v) for v in past_buckets],
                  rank_map_path=None, rank_map_loaded=False)
    return assemble_plan(measurements, mode=mode, source=source)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser("Generate a per-layer dense-decode plan from checkpoint measurements")
    ap.add_argument("--checkpoint", type=str, required=True, help="local checkpoint directory")
    ap.add_argument("--output", type=str, required=True)
    ap.add_argument("--device", type=str, default="cuda")
    ap.add_argument("--dtype", type=str, default="bf16", choices=["bf16"])
    ap.add_argument("--batch_size", type=int, default=1)
    ap.add_argument("--layer", type=int, default=-1, help="Single layer index. -1 generates the full plan.")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--mode", type=str, default="attention", choices=["reconstruct", "attention"])
    ap.add_argument("--past_buckets", type=str, default="0,512")
    ap.add_argument("--pad_multiples", type=str, default="1,8,16,32,64")
    ap.add_argument("--pad_mode", type=str, default=os.getenv("FLASH_SVD_DENSE_DECODE_PAD_MODE", "independent"))
    args = ap.parse_args(argv)
    from .checkpoint import get_model_from_local
    model = get_model_from_local(args.checkpoint, device=args.device, dtype=torch.bfloat16)
    pad_multiples = parse_pad_multiples(args.pad_multiples)
    past_buckets = parse_int_list(args.past_buckets, default=[0, 512])
    print("==== FlashSVD Dense Decode Plan Generation ====")
    print(f"checkpoint={args.checkpoint} dtype={args.dtype} device={args.device} batch={args.batch_size} warmup={args.warmup} "
          f"iters={args.iters} mode={args.mode} pad_multiples={pad_multiples} pad_mode={args.pad_mode} past_buckets={past_buckets}")
    plan = generate_dense_decode_plan(model, mode=args.mode, batch_size=args.batch_size,
                                      layers=None if args.layer < 0 else [args.layer], warmup=args.warmup, iters=args.iters,
                                      past_buckets=past_buckets, pad_multiples=pad_multiples, pad_mode=args.pad_mode,
                                      device=args.device, checkpoint=args.checkpoint)
    print(f"Saved plan to: {save_plan(plan, args.output)}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
