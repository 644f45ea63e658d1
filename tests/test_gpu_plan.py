"""Rank padding, the two attention-decode backends and plan generation on the GPU.

The oracle decodes the UNPADDED model on the CPU; the GPU runs it unpadded (ranks that are not multiples of 8
take the element-wise loads), padded in place, through both backends and through the persistent step.
Tolerances as in test_gpu_model.py (hidden states 1e-2 per teacher-forced layer stack of this depth: 3e-2)."""
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, model_from_oracle

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _odd():
    # ranks 204 / 300: rows of 408 and 600 bytes, not multiples of 16
    mw = O.make_model(d=1024, n_heads=8, n_kv_heads=4, head_dim=128, ffn=2048, attn_rank=204, mlp_rank=300,
                      n_layers=2, vocab=2048, dtype=BF16, seed=11)
    prompt = torch.randint(0, 2048, (1, 21), generator=torch.Generator().manual_seed(2))
    return mw, prompt


def _decode(model, prompt, n_new, forced=None):
    """Per-kernel decode; returns tokens [n_new] and hidden states [n_new-1, d] (teacher-forced on ``forced``)."""
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    Lp = prompt.shape[1]
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 4, device="cuda", dtype=BF16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp))
    tok = out.logits[:, -1].float().argmax(-1, keepdim=True)
    toks, hid = [int(tok)], []
    for s in range(1, n_new):
        inp = tok if forced is None else forced[:, s - 1:s].cuda()
        pos = torch.full((1,), Lp + s - 1, dtype=torch.int32, device="cuda")
        logits, h = model.decode_step(inp, cache, pos, return_hidden=True)
        cache._seen_tokens += 1
        tok = logits[:, -1].float().argmax(-1, keepdim=True)
        toks.append(int(tok))
        hid.append(h[0].float().cpu())
    return toks, torch.stack(hid)


def test_odd_ranks_unpadded_and_padded_against_oracle():
    from flashsvd_amd import plan as P
    mw, prompt = _odd()
    n_new = 6
    ref_tok, ref_hid, _ = O.greedy_decode(mw, prompt, n_new, "dense", return_hidden=True)
    model = model_from_oracle(mw)
    toks_u, hid_u = _decode(model, prompt, n_new, forced=ref_tok)
    rep = P.pad_model_ranks(model, 128, "uniform_layer")
    assert rep["layers"][0]["q"] == (204, 256) and rep["layers"][1]["gate"] == (300, 384)
    assert model.model.layers[0].self_attn._qkv_rank_tuple() == (256, 256, 256)
    toks_p, hid_p = _decode(model, prompt, n_new, forced=ref_tok)
    for s in range(1, n_new):
        r = ref_hid[0, s].float()
        tol = dict(abs_tol=3 * bounds(r)["abs_tol"], rel_tol=3e-2)
        assert_close_bf16(hid_u[s - 1], r, f"unpadded hidden, step {s}", **tol)
        assert_close_bf16(hid_p[s - 1], r, f"padded hidden, step {s}", **tol)
    assert toks_u[0] == toks_p[0] == int(ref_tok[0, 0])


def test_exact_and_packed_backends_agree(monkeypatch):
    mw, prompt = _odd()
    model = model_from_oracle(mw)
    n_new = 6
    monkeypatch.setenv("FLASH_SVD_DENSE_DECODE_BACKEND", "packed")
    toks_p, hid_p = _decode(model, prompt, n_new)
    monkeypatch.setenv("FLASH_SVD_DENSE_DECODE_BACKEND", "exact")
    toks_e, hid_e = _decode(model, prompt, n_new, forced=torch.tensor([toks_p]))
    # same rounding points in both forms (every factor linear, RoPE, cache write): a few ulps at most
    assert_close_bf16(hid_e, hid_p, "exact vs packed hidden states", abs_tol=3 * bounds(hid_p)["abs_tol"], rel_tol=3e-2)
    assert toks_e[0] == toks_p[0]


def test_persistent_step_with_ranks_that_differ_per_layer():
    """Unpadded ranks first, then layer 0 padded to 256 / 384 and layer 1 to 384 / 512: the step takes each layer's own ranks."""
    from flashsvd_amd import plan as P
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import PersistentDecoder
    mw, prompt = _odd()
    model = model_from_oracle(mw)
    # ranks off the 128 grid (204 / 300 here) are served from zero-padded twins the decoder builds itself
    n0, Lp0 = 5, prompt.shape[1]
    toks_0, _ = _decode(model, prompt, n0)
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp0 + n0 + 4, device="cuda", dtype=BF16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp0))
    t0 = out.logits[:, -1].float().argmax(-1, keepdim=True)
    dec0 = PersistentDecoder(model, cache)
    dec0.set_state(t0, Lp0)
    dec0.step(n0 - 1)
    assert [int(t0)] + dec0.tokens().cpu().tolist() == toks_0
    l0, l1 = model.model.layers
    P.pad_attention_ranks(l0.self_attn, 128, "uniform_layer")
    P.pad_mlp_ranks(l0.mlp, 128)
    P.pad_attention_ranks(l1.self_attn, 384, "uniform_layer")
    P.pad_mlp_ranks(l1.mlp, 512)
    assert l0.self_attn._qkv_rank_tuple() == (256,) * 3 and l1.self_attn._qkv_rank_tuple() == (384,) * 3
    assert l0.mlp.gate_v_proj.out_features == 384 and l1.mlp.gate_v_proj.out_features == 512
    n_new, Lp = 8, prompt.shape[1]
    toks_k, _ = _decode(model, prompt, n_new)
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 4, device="cuda", dtype=BF16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp))
    tok0 = out.logits[:, -1].float().argmax(-1, keepdim=True)
    dec = PersistentDecoder(model, cache)
    dec.set_state(tok0, Lp)
    dec.step(n_new - 1)
    assert [int(tok0)] + dec.tokens().cpu().tolist() == toks_k


@pytest.mark.parametrize("mode", ["attention", "reconstruct"])
def test_generate_and_apply_plan(mode, tmp_path):
    from flashsvd_amd import plan as P
    mw, prompt = _odd()
    model = model_from_oracle(mw)
    lines = []
    plan = P.generate_dense_decode_plan(model, mode=mode, warmup=1, iters=3, past_buckets=(0, 64), pad_multiples=(1, 8, 64),
                                        checkpoint="synthetic", log=lines.append)
    assert plan["format"] == (P.PLAN_FORMAT_ATTENTION if mode == "attention" else P.PLAN_FORMAT_RECONSTRUCT)
    assert sorted(plan["layers"]) == ["0", "1"] and len(lines) == (4 if mode == "attention" else 2)
    for entry in plan["layers"].values():
        assert entry["qkv_ranks"] == [204, 204, 204] and entry["backend"] in ("exact", "packed")
        assert entry["split_sizes"] in ([204, 204, 204], [208, 208, 208], [256, 256, 256])
        rows = entry["buckets"]["0"]["candidates"] if mode == "attention" else entry["candidates"]
        assert len(rows) == (6 if mode == "attention" else 4)
        assert all(r["ms"] > 0 and r["ms"] == r["ms"] for r in rows)
        if mode == "reconstruct":
            assert sorted(r["impl"] for r in rows) == ["exact", "packed_flat", "packed_flat", "packed_linear"]
    # the model was left as it was, and decodes the same before and after the plan is applied (padding is exact
    # up to fp32 summation order)
    assert model.model.layers[0].self_attn._qkv_rank_tuple() == (204, 204, 204)
    assert getattr(model.model.layers[0].self_attn, "_dense_decode_plan", None) is None
    toks_before, hid_before = _decode(model, prompt, 5)
    path = P.save_plan(plan, tmp_path / "plan.json")
    applied = P.apply_dense_decode_plan(model, P.load_plan(path))
    assert set(applied) == {0, 1}
    toks_after, hid_after = _decode(model, prompt, 5, forced=torch.tensor([toks_before]))
    assert_close_bf16(hid_after, hid_before, "hidden states after applying the plan", abs_tol=3 * bounds(hid_before)["abs_tol"],
                      rel_tol=3e-2)
    assert toks_after[0] == toks_before[0]
