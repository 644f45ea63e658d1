"""Checkpoint loading into the drop-in modules (host logic, runs without a GPU).

Behaviour follows the reference's utils/model_utils.py: key maps (:321-363), shared bases (:366-412),
finalisation (:415-464), shard discovery (:229-268), wrapped-pair conversion (:573-671), pickle trust gate
(:1043-1091).  The checkpoints are synthetic and written by the tests themselves.
"""
import json

import pytest
import torch
import torch.nn as nn
from safetensors.torch import save_file

from flashsvd_amd import checkpoint as ck

CFG = dict(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=96,
           num_hidden_layers=2, vocab_size=50, rope_theta=10000.0, rms_norm_eps=1e-5, hidden_act="silu",
           max_position_embeddings=128, torch_dtype="bfloat16", architectures=["LlamaForCausalLM"])
RA, RM = 24, 32


def native_state(seed=0, layers=2, ra=RA, rm=RM, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    d, qd, kvd, D, V = 64, 64, 32, 96, 50
    rnd = lambda *s: (torch.randn(*s, generator=g) * 0.05).to(dtype)
    sd = {"model.embed_tokens.weight": rnd(V, d), "model.norm.weight": rnd(d), "lm_head.weight": rnd(V, d)}
    for i in range(layers):
        p = f"model.layers.{i}"
        sd[f"{p}.input_layernorm.weight"] = rnd(d)
        sd[f"{p}.post_attention_layernorm.weight"] = rnd(d)
        for name, out, inp in (("q", qd, d), ("k", kvd, d), ("v", kvd, d), ("o", d, qd)):
            sd[f"{p}.self_attn.{name}_v_proj.weight"] = rnd(ra, inp)
            sd[f"{p}.self_attn.{name}_u_proj.weight"] = rnd(out, ra)
        for name, out, inp in (("gate", D, d), ("up", D, d), ("down", d, D)):
            sd[f"{p}.mlp.{name}_v_proj.weight"] = rnd(rm, inp)
            sd[f"{p}.mlp.{name}_u_proj.weight"] = rnd(out, rm)
    return sd


def rename(sd, style):
    out = {}
    for k, v in sd.items():
        parts = k.split(".")
        if len(parts) == 6 and parts[3] in ("self_attn", "mlp"):
            proj, factor = parts[4].split("_")[0], parts[4].split("_")[1]
            if style == "basis_sharing":
                parts[4] = f"{proj}_proj" if factor == "u" else f"{proj}_basis"
            elif style == "wrapped":
                parts[4:5] = [f"{proj}_proj", f"{factor}_proj"]
            elif style == "dobi":
                parts[4:5] = [f"{proj}_proj", "BLinear" if factor == "u" else "ALinear"]
        out[".".join(parts)] = v
    return out


def write_dir(tmp_path, sd, cfg=CFG, *, fmt="safetensors", shards=1, index=True):
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    keys = sorted(sd)
    ext = "safetensors" if fmt == "safetensors" else "bin"
    stem = "model" if fmt == "safetensors" else "pytorch_model"
    save = (lambda d, f: save_file({k: v.contiguous() for k, v in d.items()}, str(f))) if fmt == "safetensors" else \
        (lambda d, f: torch.save(d, str(f)))
    if shards == 1:
        save(sd, tmp_path / f"{stem}.{ext}")
        return tmp_path
    weight_map = {}
    for s in range(shards):
        name = f"{stem}-{s + 1:05d}-of-{shards:05d}.{ext}"
        part = {k: sd[k] for k in keys[s::shards]}
        save(part, tmp_path / name)
        weight_map.update({k: name for k in part})
    if index:
        (tmp_path / f"{stem}.{ext}.index.json").write_text(json.dumps({"weight_map": weight_map}))
    return tmp_path


def assert_matches(model, sd):
    got = model.state_dict()
    for k, v in sd.items():
        assert torch.equal(got[k].cpu(), v), k


@pytest.mark.parametrize("style", ["native", "basis_sharing", "wrapped", "dobi"])
@pytest.mark.parametrize("fmt,shards,index", [("safetensors", 1, True), ("bin", 1, True), ("bin", 3, True),
                                              ("bin", 3, False), ("safetensors", 2, True)])
def test_load_dir_every_naming_and_container(tmp_path, style, fmt, shards, index):
    sd = native_state()
    cfg = dict(CFG, architectures=["ShareLlamaForCausalLM"]) if style == "basis_sharing" else CFG
    write_dir(tmp_path, rename(sd, style), cfg, fmt=fmt, shards=shards, index=index)
    model = ck.load_lowrank_model_from_dir(tmp_path)
    assert_matches(model, sd)
    attn, mlp = model.model.layers[1].self_attn, model.model.layers[1].mlp
    assert attn.low_rank == RA and attn.q_v_proj.out_features == RA and attn.q_u_proj.in_features == RA
    assert attn.num_key_value_heads == 2 and attn.num_key_value_groups == 2 and attn.layer_idx == 1
    assert mlp.gate_v_proj.out_features == RM and mlp.down_u_proj.in_features == RM
    assert attn.ratio == pytest.approx(2.0 * RA / 64) and mlp.ratio == pytest.approx(RM * (64 + 96) / (64 * 96))
    assert not any(p.is_meta for p in model.parameters()) and not model.training
    assert model.model.rotary_emb.inv_freq.device.type == "cpu" and model.model.rotary_emb.inv_freq.shape == (8,)
    assert next(model.parameters()).dtype == torch.bfloat16


def test_dtype_override_and_fp32_checkpoint(tmp_path):
    sd = native_state(dtype=torch.float32)
    write_dir(tmp_path, sd, dict(CFG, torch_dtype="float32"))
    assert next(ck.load_lowrank_model_from_dir(tmp_path).parameters()).dtype == torch.float32
    model = ck.load_lowrank_model_from_dir(tmp_path, dtype=torch.bfloat16)
    assert torch.equal(model.lm_head.weight, sd["lm_head.weight"].to(torch.bfloat16))


def test_missing_keys_are_named(tmp_path):
    sd = rename(native_state(), "basis_sharing")
    del sd["model.layers.1.mlp.down_basis.weight"], sd["model.layers.0.self_attn.k_proj.weight"]
    write_dir(tmp_path, sd)
    with pytest.raises(KeyError) as e:
        ck.load_lowrank_model_from_dir(tmp_path)
    assert "missing 2 required tensors" in str(e.value) and "model.layers.0.self_attn.k_proj.weight" in str(e.value)


def test_unused_keys_are_ignored(tmp_path):
    sd = native_state()
    extra = dict(sd, **{"model.layers.0.self_attn.rotary_emb.inv_freq": torch.zeros(8), "unrelated.weight": torch.zeros(3)})
    write_dir(tmp_path, extra)
    assert_matches(ck.load_lowrank_model_from_dir(tmp_path), sd)


def test_no_factor_keys(tmp_path):
    sd = {k: v for k, v in native_state().items() if "_proj" not in k}
    write_dir(tmp_path, sd)
    with pytest.raises(ValueError, match="no low-rank factor keys"):
        ck.load_lowrank_model_from_dir(tmp_path)


def test_shared_bases_are_tied(tmp_path):
    sd = native_state()
    for p in ("q", "k", "v"):
        sd[f"model.layers.1.self_attn.{p}_v_proj.weight"] = sd[f"model.layers.0.self_attn.{p}_v_proj.weight"].clone()
    sd["model.layers.1.mlp.up_v_proj.weight"] = sd["model.layers.0.mlp.up_v_proj.weight"].clone()
    cfg = dict(CFG, architectures=["ShareLlamaForCausalLM"], q_groups=[[0, 1]], k_groups=[[0, 1]], v_groups=[[0, 1]],
               o_groups=[[0], [1]], up_groups=[[0, 1]])
    write_dir(tmp_path, rename(sd, "basis_sharing"), cfg)
    model = ck.load_lowrank_model_from_dir(tmp_path)
    l0, l1 = model.model.layers
    for p in ("q", "k", "v"):
        assert getattr(l1.self_attn, f"{p}_v_proj").weight is getattr(l0.self_attn, f"{p}_v_proj").weight
    assert l1.mlp.up_v_proj.weight is l0.mlp.up_v_proj.weight
    assert l1.self_attn.o_v_proj.weight is not l0.self_attn.o_v_proj.weight
    assert l1.mlp.gate_v_proj.weight is not l0.mlp.gate_v_proj.weight
    assert_matches(model, sd)
    # tying survives the dtype / device pass
    model = ck.load_lowrank_model_from_dir(tmp_path, dtype=torch.float32)
    assert model.model.layers[1].self_attn.q_v_proj.weight is model.model.layers[0].self_attn.q_v_proj.weight


def test_group_that_is_not_shared_is_refused(tmp_path):
    cfg = dict(CFG, architectures=["ShareLlamaForCausalLM"], q_groups=[[0, 1]])
    write_dir(tmp_path, rename(native_state(), "basis_sharing"), cfg)
    with pytest.raises(ValueError, match=r"q_groups\[0\] is not actually shared"):
        ck.load_lowrank_model_from_dir(tmp_path)


def test_group_shape_mismatch(tmp_path):
    sd = native_state()
    sd["model.layers.1.mlp.down_v_proj.weight"] = torch.zeros(RM + 8, 96, dtype=torch.bfloat16)
    sd["model.layers.1.mlp.down_u_proj.weight"] = torch.zeros(64, RM + 8, dtype=torch.bfloat16)
    cfg = dict(CFG, architectures=["ShareLlamaForCausalLM"], down_groups=[[0, 1]])
    write_dir(tmp_path, rename(sd, "basis_sharing"), cfg)
    with pytest.raises(ValueError, match="mismatched shapes"):
        ck.load_lowrank_model_from_dir(tmp_path)


def test_rank_rules(tmp_path):
    sd = native_state()
    sd["model.layers.0.self_attn.k_v_proj.weight"] = torch.zeros(RA - 8, 64, dtype=torch.bfloat16)
    sd["model.layers.0.self_attn.k_u_proj.weight"] = torch.zeros(32, RA - 8, dtype=torch.bfloat16)
    (tmp_path / "a").mkdir(), (tmp_path / "b").mkdir(), (tmp_path / "c").mkdir(), (tmp_path / "d").mkdir()
    # unequal q/k/v ranks: fine for plain factor pairs, refused for Basis-Sharing
    write_dir(tmp_path / "a", sd)
    assert ck.load_lowrank_model_from_dir(tmp_path / "a").model.layers[0].self_attn.low_rank == RA - 8
    write_dir(tmp_path / "b", rename(sd, "basis_sharing"), dict(CFG, architectures=["ShareLlamaForCausalLM"]))
    with pytest.raises(ValueError, match="shared q/k/v rank"):
        ck.load_lowrank_model_from_dir(tmp_path / "b")
    # gate/up ranks must agree everywhere (the SwiGLU phase streams them as one pair)
    sd = native_state()
    sd["model.layers.1.mlp.up_v_proj.weight"] = torch.zeros(RM + 8, 64, dtype=torch.bfloat16)
    sd["model.layers.1.mlp.up_u_proj.weight"] = torch.zeros(96, RM + 8, dtype=torch.bfloat16)
    write_dir(tmp_path / "c", sd)
    with pytest.raises(ValueError, match="shared gate/up rank"):
        ck.load_lowrank_model_from_dir(tmp_path / "c")
    # factors that do not chain
    sd = native_state()
    sd["model.layers.0.self_attn.o_u_proj.weight"] = torch.zeros(64, RA + 8, dtype=torch.bfloat16)
    write_dir(tmp_path / "d", sd)
    with pytest.raises(ValueError, match="does not chain"):
        ck.load_lowrank_model_from_dir(tmp_path / "d")


def test_shard_discovery_errors(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(CFG))
    with pytest.raises(FileNotFoundError, match="Could not find checkpoint shards"):
        list(ck.iter_weight_shards(tmp_path))
    (tmp_path / "pytorch_model.bin.index.json").write_text(json.dumps({"weight_map": {"a": "pytorch_model-00001-of-00002.bin"}}))
    with pytest.raises(FileNotFoundError, match="Missing shard referenced by index"):
        list(ck.iter_weight_shards(tmp_path))
    (tmp_path / "pytorch_model.bin.index.json").write_text(json.dumps({"weight_map": {}}))
    with pytest.raises(ValueError, match="Invalid HF shard index"):
        list(ck.iter_weight_shards(tmp_path))
    with pytest.raises(FileNotFoundError, match="config.json"):
        ck.read_local_config(tmp_path / "nowhere")


def test_index_order_and_dedup(tmp_path):
    for n in ("pytorch_model-00001-of-00002.bin", "pytorch_model-00002-of-00002.bin"):
        torch.save({}, tmp_path / n)
    wm = {"x": "pytorch_model-00002-of-00002.bin", "y": "pytorch_model-00001-of-00002.bin", "z": "pytorch_model-00002-of-00002.bin"}
    (tmp_path / "pytorch_model.bin.index.json").write_text(json.dumps({"weight_map": wm}))
    assert [p.name for p in ck.iter_weight_shards(tmp_path)] == ["pytorch_model-00002-of-00002.bin",
                                                                  "pytorch_model-00001-of-00002.bin"]


def test_config_helpers():
    assert ck.is_basis_sharing_config({"architectures": ["ShareLlamaForCausalLM"]})
    assert not ck.is_basis_sharing_config({"architectures": ["LlamaForCausalLM"]}) and not ck.is_basis_sharing_config({})
    assert ck.torch_dtype_from_raw("torch.bfloat16") is torch.bfloat16 and ck.torch_dtype_from_raw("FP16") is torch.float16
    assert ck.torch_dtype_from_raw(None) is None and ck.torch_dtype_from_raw("int7") is None
    assert ck.torch_dtype_from_raw(torch.float32) is torch.float32
    assert ck.destination_of("model.layers.3.self_attn.q_basis.weight") == ("layer", 3, "self_attn", "q_v_proj")
    assert ck.destination_of("model.layers.3.mlp.down_proj.BLinear.weight") == ("layer", 3, "mlp", "down_u_proj")
    assert ck.destination_of("model.layers.3.mlp.down_proj.ALinear.weight") == ("layer", 3, "mlp", "down_v_proj")
    assert ck.destination_of("model.layers.3.mlp.q_proj.u_proj.weight") is None
    assert ck.destination_of("model.layers.x.mlp.up_proj.weight") is None
    assert ck.destination_of("model.layers.0.self_attn.q_proj.bias") is None
    assert len(ck.expected_keys(2, "basis_sharing")) == 3 + 2 * (2 + 14)


class _Pair(nn.Module):
    def __init__(self, inp, out, r, names):
        super().__init__()
        setattr(self, names[0], nn.Linear(r, out, bias=False))
        setattr(self, names[1], nn.Linear(inp, r, bias=False))


class _Holder(nn.Module):
    pass


def wrapped_model(names, *, dense_proj=None):
    cfg = ck.config_namespace(CFG)
    model, inner = _Holder(), _Holder()
    model.config, model.model = cfg, inner
    inner.layers = nn.ModuleList()
    for i in range(2):
        layer, attn, mlp = _Holder(), _Holder(), _Holder()
        attn.layer_idx = i
        for p, out, inp in (("q", 64, 64), ("k", 32, 64), ("v", 32, 64), ("o", 64, 64)):
            setattr(attn, f"{p}_proj", _Pair(inp, out, RA + (8 if p == "o" else 0), names))
        for p, out, inp in (("gate", 96, 64), ("up", 96, 64), ("down", 64, 96)):
            setattr(mlp, f"{p}_proj", _Pair(inp, out, RM, names))
        if dense_proj is not None and i == 1:
            setattr(mlp, dense_proj, nn.Linear(96, 64, bias=False))
        layer.self_attn, layer.mlp = attn, mlp
        inner.layers.append(layer)
    return model


@pytest.mark.parametrize("names", [("u_proj", "v_proj"), ("BLinear", "ALinear")])
def test_convert_wrapped_module_tree(names):
    from flashsvd_amd import llama
    model = wrapped_model(names)
    src = {(i, p): (getattr(getattr(l.self_attn if p in "qkvo" else l.mlp, f"{p}_proj"), names[0]).weight,
                    getattr(getattr(l.self_attn if p in "qkvo" else l.mlp, f"{p}_proj"), names[1]).weight)
           for i, l in enumerate(model.model.layers) for p in ("q", "k", "v", "o", "gate", "up", "down")}
    ck.convert_uv_wrapped_llama(model)
    for i, l in enumerate(model.model.layers):
        assert isinstance(l.self_attn, llama.SVD_LlamaAttention) and isinstance(l.mlp, llama.SVD_LlamaMLP)
        for p in ("q", "k", "v", "o", "gate", "up", "down"):
            blk = l.self_attn if p in "qkvo" else l.mlp
            u, v = src[(i, p)]
            assert getattr(blk, f"{p}_u_proj").weight.data_ptr() == u.data_ptr()      # shared, not copied
            assert getattr(blk, f"{p}_v_proj").weight.data_ptr() == v.data_ptr()
        assert l.self_attn.o_v_proj.out_features == RA + 8 and l.self_attn.low_rank == RA and l.self_attn.layer_idx == i
    # a second pass leaves native layers alone
    before = model.model.layers[0].self_attn
    ck.convert_uv_wrapped_llama(model)
    assert model.model.layers[0].self_attn is before


def test_convert_skips_partially_factorised_layers():
    from flashsvd_amd import llama
    model = wrapped_model(("u_proj", "v_proj"), dense_proj="down_proj")
    ck.convert_uv_wrapped_llama(model)
    assert isinstance(model.model.layers[0].self_attn, llama.SVD_LlamaAttention)
    assert not isinstance(model.model.layers[1].self_attn, llama.SVD_LlamaAttention)


def test_single_file_trust_gate(tmp_path, monkeypatch):
    tensors = tmp_path / "t.pt"
    torch.save({"a": torch.arange(4)}, tensors)
    assert torch.equal(ck.torch_load_local_checkpoint(tensors)["a"], torch.arange(4))
    with pytest.raises(ValueError, match="Unrecognized checkpoint format"):
        ck.get_model_from_local(tensors)
    pickled = tmp_path / "m.pt"
    torch.save({"model": wrapped_model(("u_proj", "v_proj")), "tokenizer": None}, pickled)
    monkeypatch.delenv("FLASH_SVD_TRUST_PICKLE", raising=False)
    with pytest.raises(RuntimeError, match="FLASH_SVD_TRUST_PICKLE=1"):
        ck.get_model_from_local(pickled)
    monkeypatch.setenv("FLASH_SVD_TRUST_PICKLE", "1")          # a file this test wrote itself
    from flashsvd_amd import llama
    model = ck.get_model_from_local(pickled)
    assert isinstance(model.model.layers[1].mlp, llama.SVD_LlamaMLP)
