"""Loading factorised Llama checkpoints into the drop-in modules (CPU-side logic, no kernel involved).

Mirrors the loaders of the reference's utils/model_utils.py for the formats the decode path meets:

* a Hugging Face directory whose linears are wrapped factor pairs — ``<proj>.u_proj / <proj>.v_proj``
  (SVD-LLM / ASVD exports) or ``<proj>.BLinear / <proj>.ALinear`` (Dobi) — converted to native modules
  like ``_maybe_convert_uv_wrapped_llama_to_flashsvd`` (model_utils.py:573-671);
* a Basis-Sharing directory (``architectures`` contains "ShareLlama"): ``*_proj`` holds the u factor and
  ``*_basis`` the v factor (key map model_utils.py:321-363), bases shared across layer groups are tied to
  one tensor (``_tie_basis_sharing_layer_groups`` :366-412) and the model is finalised like
  ``_finalize_basis_sharing_flashsvd_model`` (:415-464);
* native keys (``self_attn.q_u_proj.weight`` ...), which is what ``state_dict()`` of this package writes;
* a single torch file: tensors only by default; pickled ``{'model', 'tokenizer'}`` objects only behind the
  trust gate ``FLASH_SVD_TRUST_PICKLE=1`` (``_torch_load_local_checkpoint`` :1043-1091 — unlike the
  reference there is no "looks like one of ours" heuristic: without the flag a pickle is refused).

Weights are read with loaders that execute nothing from the file: safetensors, or
``torch.load(weights_only=True)``.  Shard discovery follows ``_iter_pytorch_bin_shards`` (:229-268) and
also accepts the safetensors equivalents.
"""
from __future__ import annotations

import json
import os
from pathlib import Path
from types import SimpleNamespace
from typing import Dict, Iterable, Iterator, Optional

import torch
import torch.nn as nn

ATTN_BASIS_MAP = {"q_proj": "q_u_proj", "q_basis": "q_v_proj", "k_proj": "k_u_proj", "k_basis": "k_v_proj",
                  "v_proj": "v_u_proj", "v_basis": "v_v_proj", "o_proj": "o_u_proj", "o_basis": "o_v_proj"}
MLP_BASIS_MAP = {"gate_proj": "gate_u_proj", "gate_basis": "gate_v_proj", "up_proj": "up_u_proj", "up_basis": "up_v_proj",
                 "down_proj": "down_u_proj", "down_basis": "down_v_proj"}
_ATTN_PROJ = ("q", "k", "v", "o")
_MLP_PROJ = ("gate", "up", "down")
# wrapper factor names -> which factor they are (applied first = "v", applied second = "u")
_WRAPPED = {"u_proj": "u", "v_proj": "v", "BLinear": "u", "ALinear": "v"}


def _env_truthy(name: str) -> bool:
    return os.getenv(name, "").strip().lower() in ("1", "true", "yes", "on")


def read_local_config(path) -> Dict[str, object]:
    f = Path(path) / "config.json"
    if not f.is_file():
        raise FileNotFoundError(f"no config.json under {path}")
    with f.open("r", encoding="utf-8") as fh:
        cfg = json.load(fh)
    if not isinstance(cfg, dict):
        raise ValueError(f"config.json under {path} is not an object")
    return cfg


def is_basis_sharing_config(cfg: Dict[str, object]) -> bool:
    archs = cfg.get("architectures")
    return isinstance(archs, list) and any("sharellama" in str(a).lower() for a in archs)


def torch_dtype_from_raw(value) -> Optional[torch.dtype]:
    if value is None:
        return None
    if isinstance(value, torch.dtype):
        return value
    return {"torch.float16": torch.float16, "float16": torch.float16, "fp16": torch.float16, "half": torch.float16,
            "torch.bfloat16": torch.bfloat16, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
            "torch.float32": torch.float32, "float32": torch.float32, "fp32": torch.float32}.get(str(value).strip().lower())


# ---------------------------------------------------------------------------------------------
# shards
# ---------------------------------------------------------------------------------------------
def iter_weight_shards(path) -> Iterator[Path]:
    """Weight files of a checkpoint directory: an index file wins, then a single file, then numbered
    shards; safetensors before torch files.  Missing shards named by an index are an error."""
    path = Path(path)
    for index_name, single, pattern in (("model.safetensors.index.json", "model.safetensors", "model-*.safetensors"),
                                        ("pytorch_model.bin.index.json", "pytorch_model.bin", "pytorch_model-*.bin")):
        index_path = path / index_name
        if index_path.is_file():
            with index_path.open("r", encoding="utf-8") as fh:
                weight_map = json.load(fh).get("weight_map")
            if not isinstance(weight_map, dict) or not weight_map:
                raise ValueError(f"Invalid HF shard index at: {index_path}")
            for name in dict.fromkeys(str(n) for n in weight_map.values()):
                shard = path / name
                if not shard.is_file():
                    raise FileNotFoundError(f"Missing shard referenced by index: {shard}")
                yield shard
            return
        if (path / single).is_file():
            yield path / single
            return
        shards = sorted(path.glob(pattern))
        if shards:
            yield from shards
            return
    raise FileNotFoundError(f"Could not find checkpoint shards under: {path}")


def load_shard(shard) -> Dict[str, torch.Tensor]:
    """Tensors of one shard, read without executing anything from the file."""
    shard = Path(shard)
    if shard.suffix == ".safetensors":
        from safetensors.torch import load_file
        return load_file(str(shard), device="cpu")
    obj = torch.load(str(shard), map_location="cpu", weights_only=True)
    if not isinstance(obj, dict):
        raise TypeError(f"Unexpected shard type for {shard}: {type(obj)!r}")
    return obj


def torch_load_local_checkpoint(path):
    """A single torch file: tensors-only load first; a pickled object only when FLASH_SVD_TRUST_PICKLE=1."""
    try:
        return torch.load(str(path), map_location="cpu", weights_only=True)
    except Exception as e:
        msg = str(e)
        if "Weights only load failed" not in msg and "weights_only" not in msg:
            raise
        if not _env_truthy("FLASH_SVD_TRUST_PICKLE"):
            raise RuntimeError(
                f"Refusing to load pickled checkpoint with weights_only=False: {path}\n"
                "The file holds pickled objects (the {'model': model, 'tokenizer': tok} format), which can run "
                "code while loading.\nIf you trust this checkpoint, re-run with: FLASH_SVD_TRUST_PICKLE=1") from e
        return torch.load(str(path), map_location="cpu", weights_only=False)


# ---------------------------------------------------------------------------------------------
# key maps
# ---------------------------------------------------------------------------------------------
def sync_linear_meta(linear: nn.Linear) -> None:
    if isinstance(linear, nn.Linear):
        linear.in_features = int(linear.weight.shape[1])
        linear.out_features = int(linear.weight.shape[0])


def replace_module_weight(module: nn.Module, tensor: torch.Tensor) -> None:
    if not isinstance(tensor, torch.Tensor):
        raise TypeError(f"Expected a tensor weight, got: {type(tensor)!r}")
    module.weight = nn.Parameter(tensor, requires_grad=False)
    if isinstance(module, nn.Linear):
        sync_linear_meta(module)
    elif isinstance(module, nn.Embedding):
        module.num_embeddings, module.embedding_dim = int(tensor.shape[0]), int(tensor.shape[1])


def destination_of(key: str) -> Optional[tuple]:
    """('top', name) | ('layer', idx, block, attr) for a checkpoint key in any of the three namings
    (Basis-Sharing, wrapped factor pairs, native), or None for a key this path does not use."""
    if key in ("model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"):
        return ("top", key[: -len(".weight")])
    parts = key.split(".")
    if len(parts) < 5 or parts[0] != "model" or parts[1] != "layers" or parts[-1] != "weight" or not parts[2].isdigit():
        return None
    idx, block = int(parts[2]), parts[3]
    if block in ("input_layernorm", "post_attention_layernorm") and len(parts) == 5:
        return ("layer", idx, block, None)
    if block not in ("self_attn", "mlp"):
        return None
    projs = _ATTN_PROJ if block == "self_attn" else _MLP_PROJ
    if len(parts) == 6:
        name = parts[4]
        basis = (ATTN_BASIS_MAP if block == "self_attn" else MLP_BASIS_MAP).get(name)
        if basis is not None:                                   # Basis-Sharing: q_proj / q_basis
            return ("layer", idx, block, basis)
        for p in projs:                                         # native: q_u_proj / q_v_proj
            if name in (f"{p}_u_proj", f"{p}_v_proj"):
                return ("layer", idx, block, name)
        return None
    if len(parts) == 7:                                         # wrapped: q_proj.u_proj / q_proj.BLinear
        proj, factor = parts[4], _WRAPPED.get(parts[5])
        if factor is not None and proj.endswith("_proj") and proj[: -len("_proj")] in projs:
            return ("layer", idx, block, f"{proj[: -len('_proj')]}_{factor}_proj")
    return None


def assign_tensor(model: nn.Module, key: str, tensor: torch.Tensor) -> bool:
    """Install one checkpoint tensor; False when the key is not part of the low-rank decode path."""
    dst = destination_of(key)
    if dst is None:
        return False
    if dst[0] == "top":
        mod = model
        for name in dst[1].split("."):
            mod = getattr(mod, name)
        replace_module_weight(mod, tensor)
        return True
    _, idx, block, attr = dst
    layer = model.model.layers[idx]
    target = getattr(layer, block) if attr is None else getattr(getattr(layer, block), attr)
    replace_module_weight(target, tensor)
    return True


def expected_keys(num_hidden_layers: int, style: str = "native") -> set:
    """Keys a complete checkpoint holds in the given naming: "native", "basis_sharing", "wrapped" or "dobi"."""
    keys = {"model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"}
    for i in range(int(num_hidden_layers)):
        pre = f"model.layers.{i}"
        keys |= {f"{pre}.input_layernorm.weight", f"{pre}.post_attention_layernorm.weight"}
        for block, projs in (("self_attn", _ATTN_PROJ), ("mlp", _MLP_PROJ)):
            for p in projs:
                if style == "native":
                    keys |= {f"{pre}.{block}.{p}_u_proj.weight", f"{pre}.{block}.{p}_v_proj.weight"}
                elif style == "basis_sharing":
                    keys |= {f"{pre}.{block}.{p}_proj.weight", f"{pre}.{block}.{p}_basis.weight"}
                elif style == "wrapped":
                    keys |= {f"{pre}.{block}.{p}_proj.u_proj.weight", f"{pre}.{block}.{p}_proj.v_proj.weight"}
                elif style == "dobi":
                    keys |= {f"{pre}.{block}.{p}_proj.BLinear.weight", f"{pre}.{block}.{p}_proj.ALinear.weight"}
                else:
                    raise ValueError(f"unknown key style {style!r}")
    return keys


def detect_style(keys: Iterable[str]) -> str:
    for k in keys:
        if k.endswith("_basis.weight"):
            return "basis_sharing"
        if k.endswith(".BLinear.weight") or k.endswith(".ALinear.weight"):
            return "dobi"
        if k.endswith("_proj.u_proj.weight") or k.endswith("_proj.v_proj.weight"):
            return "wrapped"
        if k.endswith("_u_proj.weight") or k.endswith("_v_proj.weight"):
            return "native"
    raise ValueError("no low-rank factor keys found in the checkpoint")


# ---------------------------------------------------------------------------------------------
# Basis-Sharing: shared bases and finalisation
# ---------------------------------------------------------------------------------------------
_GROUP_GETTERS = {
    "q_groups": lambda layer: layer.self_attn.q_v_proj, "k_groups": lambda layer: layer.self_attn.k_v_proj,
    "v_groups": lambda layer: layer.self_attn.v_v_proj, "o_groups": lambda layer: layer.self_attn.o_v_proj,
    "gate_groups": lambda layer: layer.mlp.gate_v_proj, "up_groups": lambda layer: layer.mlp.up_v_proj,
    "down_groups": lambda layer: layer.mlp.down_v_proj,
}


def tie_basis_sharing_layer_groups(model: nn.Module, cfg: Dict[str, object]) -> int:
    """Layers listed together in ``<proj>_groups`` share one basis: check that they really are equal and make
    them one tensor.  Returns the number of tensors freed."""
    layers = getattr(getattr(model, "model", None), "layers", None)
    if layers is None:
        return 0
    tied = 0
    for group_name, getter in _GROUP_GETTERS.items():
        raw_groups = cfg.get(group_name)
        if not isinstance(raw_groups, list):
            continue
        for gi, raw in enumerate(raw_groups):
            if not isinstance(raw, list) or len(raw) <= 1:
                continue
            group = [int(i) for i in raw]
            ref = getter(layers[group[0]]).weight
            for li in group[1:]:
                cur = getter(layers[li])
                if tuple(cur.weight.shape) != tuple(ref.shape):
                    raise ValueError(f"Basis_Sharing group {group_name}[{gi}] has mismatched shapes: "
                                     f"{tuple(ref.shape)} vs {tuple(cur.weight.shape)}")
                if not torch.equal(cur.weight, ref):
                    diff = float((cur.weight.float() - ref.float()).abs().max())
                    raise ValueError(f"Basis_Sharing group {group_name}[{gi}] is not actually shared "
                                     f"(layers {group[0]} and {li}, max diff {diff:.6f}).")
                cur.weight = ref
                sync_linear_meta(cur)
                tied += 1
    return tied


def finalize_lowrank_model(model: nn.Module, *, require_shared_qkv_rank: bool = False) -> None:
    """Bring the module bookkeeping in line with the loaded factors: ranks, ratios, kv-head count, derived
    decode tensors dropped so that they are rebuilt from the new weights."""
    for idx, layer in enumerate(model.model.layers):
        attn, mlp = layer.self_attn, layer.mlp
        rq, rk, rv = (int(getattr(attn, f"{p}_v_proj").weight.shape[0]) for p in ("q", "k", "v"))
        if require_shared_qkv_rank and len({rq, rk, rv}) != 1:
            raise ValueError(f"Basis_Sharing attention layer {idx} must have shared q/k/v rank; got {rq}/{rk}/{rv}.")
        for p in _ATTN_PROJ:
            u, v = getattr(attn, f"{p}_u_proj"), getattr(attn, f"{p}_v_proj")
            if u.weight.shape[1] != v.weight.shape[0]:
                raise ValueError(f"layer {idx} {p}: u factor {tuple(u.weight.shape)} does not chain with v factor "
                                 f"{tuple(v.weight.shape)}")
        attn.layer_idx = idx
        attn.low_rank = rk
        attn.ratio = float(2.0 * rq / max(1, attn.hidden_size))
        attn.num_key_value_heads = int(attn.k_u_proj.weight.shape[0] // max(1, attn.head_dim))
        attn.num_key_value_groups = int(attn.num_heads // max(1, attn.num_key_value_heads))
        attn._reset_runtime_state()
        gr, ur = int(mlp.gate_v_proj.weight.shape[0]), int(mlp.up_v_proj.weight.shape[0])
        if gr != ur:
            raise ValueError(f"MLP layer {idx} must have shared gate/up rank; got {gr}/{ur}.")
        for p in _MLP_PROJ:
            u, v = getattr(mlp, f"{p}_u_proj"), getattr(mlp, f"{p}_v_proj")
            if u.weight.shape[1] != v.weight.shape[0]:
                raise ValueError(f"layer {idx} {p}: u factor {tuple(u.weight.shape)} does not chain with v factor "
                                 f"{tuple(v.weight.shape)}")
        hs, inter = int(mlp.up_v_proj.weight.shape[1]), int(mlp.gate_u_proj.weight.shape[0])
        mlp.hidden_size, mlp.intermediate_size = hs, inter
        mlp.ratio = float(gr * (float(hs) + float(inter)) / max(1.0, float(hs) * float(inter)))
        mlp._packed_gu_v = None
        mlp._packed_key = None


# ---------------------------------------------------------------------------------------------
# loaders
# ---------------------------------------------------------------------------------------------
def config_namespace(cfg: Dict[str, object]) -> SimpleNamespace:
    """The fields of config.json the modules read, with Llama defaults."""
    hidden, heads = int(cfg["hidden_size"]), int(cfg["num_attention_heads"])
    return SimpleNamespace(
        hidden_size=hidden, num_attention_heads=heads,
        num_key_value_heads=int(cfg.get("num_key_value_heads") or heads),
        head_dim=int(cfg.get("head_dim") or hidden // heads),
        intermediate_size=int(cfg["intermediate_size"]), num_hidden_layers=int(cfg["num_hidden_layers"]),
        vocab_size=int(cfg["vocab_size"]), rope_theta=float(cfg.get("rope_theta", 10000.0)),
        rms_norm_eps=float(cfg.get("rms_norm_eps", 1e-6)), hidden_act=str(cfg.get("hidden_act", "silu")),
        max_position_embeddings=int(cfg.get("max_position_embeddings", 4096)),
        architectures=["LlamaForCausalLM"], torch_dtype=torch_dtype_from_raw(cfg.get("torch_dtype") or cfg.get("dtype")))


def load_lowrank_model_from_dir(path, *, device=None, dtype: Optional[torch.dtype] = None):
    """Build an SVDLlamaForCausalLM for the config under ``path`` and fill it from the weight shards, whatever
    naming they use.  Returns the model (eval mode, weights on ``device`` in ``dtype`` if given)."""
    from . import llama
    path = Path(path)
    cfg = read_local_config(path)
    config = config_namespace(cfg)
    with torch.device("meta"):
        model = llama.SVDLlamaForCausalLM(config, attn_ratio=0.5, mlp_ratio=0.5)
    seen: set = set()
    style = None
    for shard_path in iter_weight_shards(path):
        shard = load_shard(shard_path)
        if style is None:
            try:
                style = detect_style(shard.keys())
            except ValueError:
                style = None
        for key, tensor in shard.items():
            if assign_tensor(model, str(key), tensor):
                seen.add(str(key))
        del shard
    if style is None:
        raise ValueError(f"no low-rank factor keys found under {path}")
    missing = sorted(expected_keys(config.num_hidden_layers, style) - seen)
    if missing:
        raise KeyError(f"checkpoint load is missing {len(missing)} required tensors from {path}. "
                       f"First missing keys: {', '.join(missing[:8])}")
    basis = is_basis_sharing_config(cfg) or style == "basis_sharing"
    if basis:
        tie_basis_sharing_layer_groups(model, cfg)
    finalize_lowrank_model(model, require_shared_qkv_rank=basis)
    model.config.num_key_value_heads = model.model.layers[0].self_attn.num_key_value_heads if config.num_hidden_layers else \
        config.num_key_value_heads
    want = dtype or config.torch_dtype
    for mod in model.modules():
        if isinstance(mod, llama.LlamaRotaryEmbedding):
            half = mod.dim // 2
            mod.inv_freq = 1.0 / (mod.base ** (torch.arange(0, half, dtype=torch.float32) / half))
    if want is not None or device is not None:
        # tied bases must stay tied: move each distinct tensor once
        moved: Dict[int, torch.Tensor] = {}
        for mod in model.modules():
            w = getattr(mod, "weight", None)
            if isinstance(w, nn.Parameter):
                key = id(w)
                if key not in moved:
                    moved[key] = nn.Parameter(w.data.to(device=device, dtype=want if w.is_floating_point() else None),
                                              requires_grad=False)
                mod.weight = moved[key]
            if isinstance(mod, llama.LlamaRotaryEmbedding) and device is not None:
                mod.inv_freq = mod.inv_freq.to(device)
    model.seqlen = int(config.max_position_embeddings)
    return model.eval()


def convert_uv_wrapped_llama(model: nn.Module) -> nn.Module:
    """Replace wrapped factor pairs (``q_proj.u_proj/v_proj`` or ``BLinear/ALinear``) of a module tree with
    native low-rank modules that share the same weight tensors.  Layers that are native already, or whose
    projections are not all factorised, are left alone."""
    from . import llama
    layers = getattr(getattr(model, "model", None), "layers", None)
    if layers is None:
        return model

    def factors(mod):
        u, v = getattr(mod, "u_proj", None), getattr(mod, "v_proj", None)
        if not (isinstance(u, nn.Linear) and isinstance(v, nn.Linear)):
            u, v = getattr(mod, "BLinear", None), getattr(mod, "ALinear", None)
        return (u, v) if isinstance(u, nn.Linear) and isinstance(v, nn.Linear) else None

    for idx, layer in enumerate(layers):
        attn, mlp = getattr(layer, "self_attn", None), getattr(layer, "mlp", None)
        if attn is None or mlp is None or (hasattr(attn, "q_u_proj") and hasattr(mlp, "gate_u_proj")):
            continue
        src = {p: factors(getattr(attn, f"{p}_proj", None)) for p in _ATTN_PROJ}
        src.update({p: factors(getattr(mlp, f"{p}_proj", None)) for p in _MLP_PROJ})
        if any(v is None for v in src.values()):
            continue
        if min(int(v.out_features) for _, v in src.values()) <= 0:
            raise ValueError(f"FlashSVD native conversion found an invalid low-rank projection in layer {idx}.")
        new_attn = llama.SVD_LlamaAttention(config=model.config, ratio=0.5, layer_idx=int(getattr(attn, "layer_idx", idx)),
                                            ranks={p: int(src[p][1].out_features) for p in _ATTN_PROJ})
        new_mlp = llama.SVD_LlamaMLP(int(model.config.hidden_size), int(model.config.intermediate_size),
                                     str(getattr(model.config, "hidden_act", "silu")), ratio=0.5,
                                     rank=int(src["gate"][1].out_features))
        for p in _ATTN_PROJ:
            replace_module_weight(getattr(new_attn, f"{p}_u_proj"), src[p][0].weight.data)
            replace_module_weight(getattr(new_attn, f"{p}_v_proj"), src[p][1].weight.data)
        for p in _MLP_PROJ:
            replace_module_weight(getattr(new_mlp, f"{p}_u_proj"), src[p][0].weight.data)
            replace_module_weight(getattr(new_mlp, f"{p}_v_proj"), src[p][1].weight.data)
        layer.self_attn, layer.mlp = new_attn, new_mlp
    if all(hasattr(l.self_attn, "q_u_proj") and hasattr(l.mlp, "gate_u_proj") for l in layers):
        finalize_lowrank_model(model)
    return model


def get_model_from_local(path, *, device=None, dtype: Optional[torch.dtype] = None):
    """Directory -> model built from its shards; single torch file -> the object it holds (tensors only unless
    the trust gate is open), converted to native modules when it is a wrapped model."""
    p = Path(path)
    if p.is_dir():
        return load_lowrank_model_from_dir(p, device=device, dtype=dtype)
    obj = torch_load_local_checkpoint(p)
    if isinstance(obj, dict) and "model" in obj and hasattr(obj["model"], "forward"):
        return convert_uv_wrapped_llama(obj["model"])
    if hasattr(obj, "forward"):
        return convert_uv_wrapped_llama(obj)
    raise ValueError(f"Unrecognized checkpoint format at: {path}")
