"""CPU-only tests: runtime flags, caches, registry, module bookkeeping, and that the C-ABI library
loads and exports every symbol the header declares (no kernel is launched here)."""
import ctypes
import os
import re
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]


# ------------------------------------------------------------------ C ABI
def test_library_exports_every_declared_symbol():
    from flashsvd_amd import _lib
    header = (ROOT / "include" / "flashsvd_hip.h").read_text()
    declared = set(re.findall(r"\b(fsvd_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 10
    lib = _lib.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(_lib.SIGNATURES), "ctypes signature table and header disagree"
    assert lib.fsvd_version() >= 102
    assert isinstance(lib.fsvd_last_error(), bytes)
    # pure host-side size queries
    assert lib.fsvd_attn_decode_workspace_bytes(1, 32, 128, 8) == 256 * 1024 + 32 * 8 * 130 * 4
    assert lib.fsvd_attn_decode_workspace_bytes(0, 32, 128, 8) == 0
    assert lib.fsvd_mlp_dual_split_workspace_bytes(1, 1536, 11008, 4096, 0, 128) > 64 * 1024 + 11008 * 2 + 1536 * 4


def test_null_pointer_and_shape_errors_come_back_as_status_codes():
    from flashsvd_amd import _lib
    lib = _lib.load()
    rc = lib.fsvd_linear(None, 8, None, 8, None, None, 1e-6, None, 0, None, 8, 1, 8, 8, 0, 0, None)
    assert rc == -4 and b"NULL" in lib.fsvd_last_error()
    buf = ctypes.create_string_buffer(64)  # never dereferenced: shape check fails first
    p = ctypes.addressof(buf)
    rc = lib.fsvd_linear(p, 4, p, 8, None, None, 1e-6, None, 0, p, 8, 1, 8, 8, 0, 0, None)
    assert rc == -1 and b"leading dimension" in lib.fsvd_last_error()
    rc = lib.fsvd_swiglu_linear(p, 16, 8, p, p, 8, p, 8, 1, 8, 8, 7, 0, 0, None)
    assert rc == -1
    with pytest.raises(_lib.FlashSVDHipError):
        _lib.check("fsvd_linear", -1)


# ------------------------------------------------------------------ runtime flags
def test_configure_runtime_flashsvd_snapshot():
    from flashsvd_amd import api
    cfg = api.configure_runtime(mode="flashsvd", ffn_backend="auto", enable_mlp_graph=True, mlp_graph_scope="layer_tail",
                                enable_flash_dense_attn=True)
    # the values the reference's smoke test pins (scripts/smoke_tests/test_public_api.py:42-56)
    assert cfg["SVDLLM_FLASH_FALLBACK"] is None
    assert cfg["FLASH_SVD_MLP_CUDA_GRAPH"] == "1"
    assert cfg["FLASH_SVD_MLP_CUDA_GRAPH_SCOPE"] == "layer_tail"
    assert cfg["FLASH_SVD_ENABLE_DENSE_ATTN_DECODE"] == "1"
    assert cfg["FLASH_SVD_DENSE_DECODE_BACKEND"] == "auto"
    assert cfg["FLASH_SVD_DENSE_DECODE_GRAPH"] == "1"
    assert cfg["FLASH_SVD_DENSE_DECODE_AUTOTUNE_SCOPE"] == "attention"
    assert cfg["FLASH_SVD_FFN_BACKEND"] == "auto" and cfg["FLASH_SVD_ENABLE_EXPERIMENTAL_FFN"] is None
    assert set(cfg) == set(api._RUNTIME_ENV_VARS) and len(cfg) == 15
    assert os.environ.get("FLASH_SVD_DISABLE_FFN") is None  # false flags are unset, never "0"


def test_configure_runtime_modes_and_flag_semantics():
    from flashsvd_amd import api
    cfg = api.configure_runtime("flashsvd", ffn_backend="flashsvd_mlp_dual_split_prod", enable_flash_dense_attn=False,
                                enable_mlp_graph=False, graph_alias_output=True, enable_cutlass_rope_attn=True)
    assert cfg["FLASH_SVD_ENABLE_EXPERIMENTAL_FFN"] == "1"
    assert cfg["FLASH_SVD_ENABLE_DENSE_ATTN_DECODE"] is None and cfg["FLASH_SVD_DENSE_DECODE_BACKEND"] is None
    assert cfg["FLASH_SVD_DENSE_DECODE_GRAPH"] is None and cfg["FLASH_SVD_DENSE_DECODE_AUTOTUNE_SCOPE"] is None
    assert cfg["FLASH_SVD_MLP_CUDA_GRAPH"] is None and cfg["FLASH_SVD_MLP_CUDA_GRAPH_ALIAS_OUTPUT"] == "1"
    assert cfg["FLASH_SVD_USE_CUTLASS_ROPEATTN"] == "1"
    for mode in ("hf", "baseline", "HF", " Baseline "):
        cfg = api.configure_runtime(mode)
        assert cfg["SVDLLM_FLASH_FALLBACK"] == "1" and cfg["FLASH_SVD_DISABLE_FFN"] == "1"
        assert all(v is None for k, v in cfg.items() if k not in ("SVDLLM_FLASH_FALLBACK", "FLASH_SVD_DISABLE_FFN"))
    with pytest.raises(ValueError, match="Unsupported runtime mode"):
        api.configure_runtime("turbo")
    assert api._backend_needs_experimental_ffn("Dual-Split-Kernel-V2") and not api._backend_needs_experimental_ffn("auto")
    assert not api._backend_needs_experimental_ffn("flashsvd_mlp_dual_split_exact_legacy")
    os.environ["FLASH_SVD_DISABLE_FFN"] = " Yes "
    assert api._env_truthy("FLASH_SVD_DISABLE_FFN")
    os.environ["FLASH_SVD_DISABLE_FFN"] = "0"
    assert not api._env_truthy("FLASH_SVD_DISABLE_FFN")
    api.configure_runtime("flashsvd")


def test_mlp_rounding_mode_follows_backend_flags():
    from flashsvd_amd import api, llama
    api.configure_runtime("flashsvd", ffn_backend="auto")
    assert llama.mlp_rounding_mode() == 0
    api.configure_runtime("flashsvd", ffn_backend="flashsvd_mlp_dual_split_prod")
    assert llama.mlp_rounding_mode() == 1
    api.configure_runtime("flashsvd", ffn_backend="flashsvd_mlp_dual_split_exact_legacy")
    assert llama.mlp_rounding_mode() == 0
    api.configure_runtime("hf")
    assert llama.mlp_rounding_mode() == 0
    api.configure_runtime("flashsvd")


def test_sample_next_token_greedy_and_nucleus():
    from flashsvd_amd import api
    logits = torch.tensor([[0.1, 3.0, 0.2, 2.9]])
    assert api._sample_next_token(logits, do_sample=False, temperature=1.0, top_p=1.0).tolist() == [[1]]
    assert api._sample_next_token(logits, do_sample=True, temperature=0.0, top_p=1.0).tolist() == [[1]]
    torch.manual_seed(0)
    seen = {int(api._sample_next_token(logits, do_sample=True, temperature=1.0, top_p=0.6)) for _ in range(50)}
    assert seen <= {1, 3}  # the nucleus holds the two dominant tokens only


# ------------------------------------------------------------------ caches
CFG = SimpleNamespace(num_hidden_layers=2, rope_theta=10000.0)


def test_dense_cache_update_prefill_then_positions():
    from flashsvd_amd.runtime.cache import FlashSVDDenseKVCache, FlashSVDV15DenseKVCache
    assert FlashSVDDenseKVCache is FlashSVDV15DenseKVCache
    c = FlashSVDV15DenseKVCache(CFG, max_batch_size=2, max_cache_len=8, device="cpu", dtype=torch.float32)
    assert c.key_cache[0].shape == (2, 8, 0, 0) and c.max_cache_len == 8 and c.get_max_cache_shape() == 8
    k, v = torch.randn(2, 3, 5, 4), torch.randn(2, 3, 5, 4)   # [B,Hk,T,Dh]
    ko, vo = c.update(k, v, 0)
    assert c.key_cache[0].shape == (2, 8, 3, 4) and torch.equal(ko, k) and torch.equal(vo, v)
    assert torch.equal(c.key_cache[0][:, :5], k.transpose(1, 2)) and c.get_seq_length() == 5
    c.update(k, v, 1)
    assert c.get_seq_length() == 5                                  # only layer 0 counts tokens
    k1, v1 = torch.randn(2, 3, 1, 4), torch.randn(2, 3, 1, 4)
    ko, vo = c.update(k1, v1, 0, {"cache_position": torch.tensor([5])})
    assert c.get_seq_length() == 6 and ko.shape == (2, 3, 6, 4) and torch.equal(ko[:, :, 5], k1[:, :, 0])
    assert c.get_mask_sizes(torch.tensor([6]), 0) == (7, 0)
    with pytest.raises(RuntimeError, match="shape changed after init"):
        c.update(torch.randn(2, 2, 1, 4), torch.randn(2, 2, 1, 4), 0)


def test_dense_cache_fa2_helpers():
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    c = FlashSVDV15DenseKVCache(CFG, max_batch_size=3, max_cache_len=8, device="cpu", dtype=torch.float32)
    c._ensure_layer_spec(0, h=2, dh=4)
    c._seen_tokens = 4
    kc, vc, lens = c.prepare_fa2_step(0, batch_size=2)
    assert kc.shape == (2, 8, 2, 4) and lens.dtype == torch.int32 and lens.tolist() == [4, 4]
    assert c.prepare_fa2_step(0, batch_size=2, cache_position=torch.tensor([6]))[2].tolist() == [6, 6]
    assert c.prepare_fa2_step(0, batch_size=2, cache_position=torch.tensor([1, 2, 3]))[2].tolist() == [1, 2]
    assert c.prepare_fa2_step(0, batch_size=2, cache_position=torch.tensor([], dtype=torch.long))[2].tolist() == [0, 0]
    assert c.prepare_fa2_step(0, batch_size=2, cache_position=7)[2].tolist() == [7, 7]
    assert c.get_fa2_kvcache(0, batch_size=3)[2].tolist() == [4, 4, 4]
    assert c.prepare_fa2_step(0, batch_size=2)[2].data_ptr() == lens.data_ptr()     # per (layer, batch) buffer is reused
    got = c.prepare_fa2_direct_write_step(0, batch_size=2, num_heads=2, head_dim=4, q_len=1, cache_position=torch.tensor([5]))
    kc, vc, kslot, vslot, lens = got
    assert kslot.shape == (2, 1, 2, 4) and kslot.data_ptr() == kc[:, 5:6].data_ptr() and lens.tolist() == [6, 6]
    assert c.prepare_fa2_direct_write_step(0, batch_size=2, num_heads=2, head_dim=4, q_len=2) is None
    assert c.prepare_fa2_direct_write_step(0, batch_size=2, num_heads=2, head_dim=4, q_len=1, cache_position=torch.tensor([3, 4])) is None
    assert c.prepare_fa2_direct_write_step(0, batch_size=2, num_heads=2, head_dim=4, q_len=1)[4].tolist() == [5, 5]
    with pytest.raises(IndexError, match="out of range"):
        c.prepare_fa2_direct_write_step(0, batch_size=2, num_heads=2, head_dim=4, q_len=1, cache_position=8)
    c.advance_after_fa2(1, q_len=1, cache_position=None)
    assert c.get_seq_length() == 4
    c.advance_after_fa2(0, q_len=1, cache_position=torch.tensor([9]))
    assert c.get_seq_length() == 10
    c.advance_after_fa2(0, q_len=1, cache_position=None)
    assert c.get_seq_length() == 11


def test_rope_tables_and_clone():
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from oracle import flashsvd_oracle as O
    c = FlashSVDV15DenseKVCache(CFG, max_batch_size=1, max_cache_len=8, device="cpu", dtype=torch.bfloat16)
    cos, sin = c.get_rope_tables(seqlen=8, head_dim=16, device=torch.device("cpu"), dtype=torch.bfloat16)
    ocos, osin = O.rope_tables(8, 16, 10000.0, torch.bfloat16)
    assert torch.equal(cos, ocos) and torch.equal(sin, osin) and cos.shape == (8, 8)
    assert c.get_rope_tables(seqlen=8, head_dim=16, device=torch.device("cpu"), dtype=torch.bfloat16)[0] is cos
    with pytest.raises(ValueError):
        c.get_rope_tables(seqlen=8, head_dim=15, device=torch.device("cpu"), dtype=torch.bfloat16)
    c.update(torch.ones(1, 2, 3, 4), torch.ones(1, 2, 3, 4), 1)
    d = c.clone_for_autotune(layer_idx=1, batch_size=1)
    assert torch.equal(d.key_cache[1], c.key_cache[1].to(d.key_cache[1].dtype)) and d.key_cache[0].shape[2] == 0
    d.key_cache[1].zero_()
    assert c.key_cache[1].abs().sum() > 0


def test_rank_cache():
    from flashsvd_amd.runtime.cache import FlashSVDLegacySparseKVCache, LowRankKVCache
    assert LowRankKVCache is FlashSVDLegacySparseKVCache
    c = FlashSVDLegacySparseKVCache(CFG, max_batch_size=2, max_cache_len=6, device="cpu", dtype=torch.float32)
    assert c.key_cache[0].shape == (2, 6, 0) and c.rank == 0
    pk, pv = torch.randn(2, 4, 5), torch.randn(2, 4, 3)             # [B,T,Rk], [B,T,Rv]: ranks may differ
    ko, vo = c.update(pk, pv, 0)
    assert c.key_cache[0].shape == (2, 6, 5) and c.value_cache[0].shape == (2, 6, 3) and c.rank == 5
    assert torch.equal(ko, pk) and torch.equal(c.key_cache[0][:, :4], pk) and c.get_seq_length() == 4
    c.update(torch.ones(2, 1, 5), torch.ones(2, 1, 3), 0, {"cache_position": torch.tensor([4])})
    assert c.get_seq_length() == 5 and torch.all(c.key_cache[0][:, 4] == 1)
    with pytest.raises(RuntimeError, match="rank changed after initialization"):
        c.update(torch.ones(2, 1, 7), torch.ones(2, 1, 3), 0)
    c2 = FlashSVDLegacySparseKVCache(CFG, max_batch_size=1, max_cache_len=4, rank=8, device="cpu")
    assert c2.key_cache[1].shape == (1, 4, 8) and c2.rank == 8
    ws = c2.get_decode_workspace(batch_size=1, num_heads=4, rank=8, head_dim=16, max_splits=3, device=torch.device("cpu"), dtype=torch.float32)
    assert ws.M.shape == (1, 4, 3) and ws.Acc.shape == (1, 4, 3, 8) and ws.Q0.shape == (1, 4, 8) and ws.L.dtype == torch.float32
    assert c2.get_decode_workspace(batch_size=1, num_heads=4, rank=8, head_dim=16, max_splits=3, device=torch.device("cpu"), dtype=torch.float32) is ws


# ------------------------------------------------------------------ registry
def test_registry_helpers():
    from flashsvd_amd import runtime
    from flashsvd_amd.runtime import decode_registry as R

    def fn(q, kc, vc, k=None, cache_seqlens=None, causal=False, rotary_interleaved=True):
        return dict(k=k, cache_seqlens=cache_seqlens, causal=causal, rotary_interleaved=rotary_interleaved)
    out = R.call_flash_attn_with_kvcache(fn, 1, 2, 3, k_bmhd="K", v_bmhd="V", cache_seqlens="L", rotary_cos="C", rotary_sin="S", causal=True)
    assert out == dict(k="K", cache_seqlens="L", causal=True, rotary_interleaved=False)   # v/rotary dropped: fn lacks them
    assert R.maybe_kwargs(fn, dict(k=1, zzz=2)) == dict(k=1)
    assert R.get_flash_attn_with_kvcache() is R.flash_attn_with_kvcache
    mod = R.get_flashsvd_v15_attn_densekv_decode_mod()
    assert hasattr(mod, "reconstruct_qkv_token_shared_prepacked") and R.get_dense_token_decode_mod() is mod
    c = R.canonical_legacy_sparsekv_decode_variant
    assert c("") == "auto" and c("V1.5") == "flashsvd_attn_legacy_v15_sparsekv" and c("legacy").endswith("v16_sparsekv_v1")
    assert c("v16") .endswith("_v2") and c("nonsense") == "auto" and R.canonical_decode_variant is c
    assert R.parse_legacy_sparsekv_decode_variant_map("1:v15, 8:v2,bad,0:v1,x:v1") == {
        1: "flashsvd_attn_legacy_v15_sparsekv", 8: "flashsvd_attn_legacy_v16_sparsekv_v2"}
    for name in runtime.__all__:
        assert hasattr(runtime, name)
    with pytest.raises(ImportError):
        R.load_module_from_path(ROOT / "does_not_exist.txt", "nope")


# ------------------------------------------------------------------ modules (host side only)
def test_rank_rule_and_module_layout():
    from flashsvd_amd import llama
    assert llama.lowrank_rank(4096, 4096, 0.5) == 1024 and llama.lowrank_rank(11008, 4096, 0.5) == 1492
    cfg = SimpleNamespace(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=96,
                          num_hidden_layers=1, vocab_size=50, rope_theta=10000.0, rms_norm_eps=1e-6, hidden_act="silu",
                          max_position_embeddings=128)
    attn = llama.SVD_LlamaAttention(cfg, ratio=0.5, layer_idx=0)
    assert attn.q_v_proj.weight.shape == (16, 64) and attn.q_u_proj.weight.shape == (64, 16)
    assert attn.k_u_proj.weight.shape == (32, attn.k_v_proj.out_features) and attn.num_key_value_groups == 2
    for name in ("_decode_Vq", "_decode_Vk", "_decode_Vv", "_decode_ptrs", "_dense_decode_prepacked_cache", "_dense_decode_backend_cache"):
        assert hasattr(attn, name)
    before = [m.weight.detach().clone() for m in (attn.q_v_proj, attn.k_v_proj, attn.v_v_proj)]
    attn._ensure_runtime_state()
    packed = attn._packed_qkv_v
    rq, rk, rv = attn._qkv_rank_tuple()
    assert packed.shape == (rq + rk + rv, 64) and torch.equal(packed, torch.cat(before))
    assert attn.k_v_proj.weight.data_ptr() == packed[rq:].data_ptr()      # module weights are views of the packed buffer
    attn._ensure_runtime_state()
    assert attn._packed_qkv_v is packed                                    # idempotent
    Vq, Vk, Vv = attn._get_decode_factors()
    assert Vq.shape == (4, rq, 16) and Vk.shape == (2, rk, 16)
    assert torch.equal(Vq[1, :, 3], attn.q_u_proj.weight[16 + 3])          # Vq[h,r,d] = q_u[h*Dh+d, r]
    t = attn._get_dense_decode_tensors()
    assert t[0].shape == (64, rq + rk + rv) and t[1].shape == (rq, 64) and t[2].shape == (rk, 32) and t[-1] == (rq, rk, rv)
    x = torch.randn(3, 64)
    assert torch.allclose(x @ t[0], torch.cat([x @ m.weight.t() for m in (attn.q_v_proj, attn.k_v_proj, attn.v_v_proj)], 1), atol=1e-5)
    os.environ["FLASH_SVD_DENSE_DECODE_RANK_PAD_MULTIPLE"] = "32"
    try:
        tp = attn._get_dense_decode_tensors()
        assert tp[-1] == (32, 32, 32) and tp[0].shape == (64, 96) and tp[1].shape == (32, 64)
        assert torch.allclose((x @ tp[0])[:, :rq] @ tp[1][:rq], (x @ t[0])[:, :rq] @ t[1], atol=1e-5)
        assert torch.all(tp[0][:, rq:32] == 0)
    finally:
        del os.environ["FLASH_SVD_DENSE_DECODE_RANK_PAD_MULTIPLE"]
    mlp = llama.SVD_LlamaMLP(64, 96, "silu", ratio=0.5)
    assert mlp.gate_v_proj.weight.shape == (llama.lowrank_rank(96, 64, 0.5), 64) and isinstance(mlp._flashsvd_graph_cache, dict)
    with pytest.raises(ValueError):
        llama.SVD_LlamaMLP(64, 96, "gelu")
    with pytest.raises(RuntimeError, match="no CPU path"):
        mlp(torch.zeros(1, 1, 64, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="no CPU path"):
        attn(torch.zeros(1, 1, 64, dtype=torch.bfloat16))
    model = llama.SVDLlamaForCausalLM(cfg, attn_ratio=0.5, mlp_ratio=0.5)
    keys = set(model.state_dict())
    assert "model.layers.0.self_attn.k_u_proj.weight" in keys and "model.layers.0.mlp.down_v_proj.weight" in keys
    assert "lm_head.weight" in keys and "model.norm.weight" in keys


def test_dual_split_config_pickers_honour_env():
    from flashsvd_amd.kernels import dual_split as ds
    assert ds._pick_dual_split_token_v2_config(1536, 11008) == {"BR": 128, "BD": 128, "BR2": 128, "warps": 8, "stages": 2}
    assert ds._pick_dual_split_token_config(256, 1376)["BR2"] == 256 and ds._pick_dual_split_token_config(600, 1376)["BR2"] == 128
    assert ds._pick_dual_split_token_v2_sm80_config(1536, 11008)["GD"] == 2 and ds._pick_dual_split_token_v3_config(64, 128, 256)["GH"] == 2
    os.environ["FLASH_SVD_DUAL_SPLIT_V2_BD"] = "64"
    os.environ["FLASH_SVD_DUAL_SPLIT_V2_WARPS"] = "junk"
    try:
        cfg = ds._pick_dual_split_token_v2_config(1536, 11008)
        assert cfg["BD"] == 64 and cfg["warps"] == 8
    finally:
        del os.environ["FLASH_SVD_DUAL_SPLIT_V2_BD"], os.environ["FLASH_SVD_DUAL_SPLIT_V2_WARPS"]
    assert ds.flashsvd_ffn_dual_split_token_v3 is ds.flashsvd_mlp_dual_split_triton_v3
