"""Correctness report, speed table and decode profiles on the GPU (small seeded model).

The report's baseline is the module-by-module form of the same HIP kernels; the CPU oracle decodes the same
model beside it so that the baseline itself is pinned (teacher-forced logits within the multi-layer bound)."""
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, model_from_oracle

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _small():
    mw = O.make_model(d=1024, n_heads=8, n_kv_heads=4, head_dim=128, ffn=2048, attn_rank=256, mlp_rank=384,
                      n_layers=3, vocab=2048, dtype=BF16, seed=3)
    return mw, model_from_oracle(mw)


def test_three_mode_report_against_oracle():
    from flashsvd_amd import report as R
    mw, model = _small()
    prompt_len, steps = 24, 6
    ids = torch.randint(0, 2048, (1, prompt_len + steps), generator=torch.Generator().manual_seed(4))
    rep = R.check_decode_correctness(model, input_ids=ids.cuda(), prompt_len=prompt_len, decode_steps=steps)
    assert set(rep["modes"]) == {"flash_legacy", "flash_test", "flash_step"}
    for label, m in rep["modes"].items():
        # logits of this model are O(1); the modes differ by rounding order / fused rounding only
        assert m["full_rel_linf"] <= 3e-2 and m["decode_rel_linf"] <= 3e-2, (label, m)
        assert abs(m["decode_ce"] - rep["baseline"]["decode_ce"]) <= 5e-2 and m["greedy_token_match"] >= 0.5, (label, m)
    assert rep["modes"]["flash_legacy"]["full_max_abs"] == 0.0          # same prefill kernels, same rounding mode
    assert len(rep["tokens"]["baseline"]) == steps and len(rep["tokens"]["flash_step"]) == steps
    lines = R.format_correctness_report(rep, header="Config: test")
    assert lines[0] == "==== FlashSVD Decode Correctness ====" and lines[2].startswith("baseline full_seq_ce=")
    assert sum(l.startswith("- flash_") for l in lines) == 6
    # the baseline itself against the CPU oracle: teacher-forced logits of the same tokens
    R.configure_mode("baseline", backend="baseline")
    try:
        got = R.run_decode_teacher_forced(model, ids.cuda(), prompt_len=prompt_len, decode_steps=steps)
    finally:
        for name in R._MODE_ENV:
            import os
            os.environ.pop(name, None)
    cache = O.DenseCache(mw, 1, prompt_len + steps + 4, BF16)
    cos, sin = O.rope_tables(prompt_len + steps + 4, mw.head_dim, mw.rope_theta, BF16)
    ref = [O.model_forward(mw, ids[:, :prompt_len], 0, cache, cos, sin)[:, -1]]
    for s in range(steps - 1):
        ref.append(O.model_forward(mw, ids[:, prompt_len + s:prompt_len + s + 1], prompt_len + s, cache, cos, sin)[:, -1])
    ref = torch.stack(ref, 1).float()
    assert_close_bf16(got, ref, "baseline teacher-forced logits vs oracle", abs_tol=3 * bounds(ref)["abs_tol"], rel_tol=3e-2)


def test_main_table_rows_from_live_runs(tmp_path):
    from flashsvd_amd import report as R
    _, model = _small()
    rows = R.collect_main_table([("Synthetic", "0.5", "in-memory")], load=lambda p: model, repeats=2, prompt_len=32, new_tokens=8,
                                warmup=2)
    assert rows[0]["status"] == "ok" and rows[0]["ok_repeats"] == 2
    assert rows[0]["flash_decode_ms"] > 0 and rows[0]["baseline_decode_ms"] > rows[0]["flash_decode_ms"]
    md = R.build_markdown(results=rows, config={"gpu": torch.cuda.get_device_name(0)}, md_path=tmp_path / "t.md")
    assert "| Synthetic | 0.5 | 2/2 |" in md


def test_module_profile_on_both_engines(monkeypatch, capsys):
    from flashsvd_amd import api
    _, model = _small()
    monkeypatch.setenv("FLASHSVD_AMD_DECODE_ENGINE", "graph")
    r = api.decode_kvcache_eval(model, prompt_len=40, new_tokens=6, warmup=2, profile_decode=True, profile_decode_steps=3)
    p = r["decode_profile"]
    assert r["decode_engine"] == "graph" and p["steps"] == 3 and p["seq"] == 48
    assert p["breakdown_ms"]["attn_total"] > 0 and p["breakdown_ms"]["mlp_total"] > 0 and p["breakdown_ms"]["lm_head"] > 0
    assert set(p["per_module_ms"]) == {"embed_tokens", "lm_head"} | {f"layer{i}.{k}" for i in range(3) for k in ("attn", "mlp")}
    parts = sum(p["breakdown_ms"].values()) + p["other_ms"]
    assert parts == pytest.approx(p["total_forward_ms_per_token"], rel=1e-6)
    assert "=== Decode Profile (module device time) ===" in capsys.readouterr().out
    monkeypatch.setenv("FLASHSVD_AMD_DECODE_ENGINE", "persistent")
    r = api.decode_kvcache_eval(model, prompt_len=40, new_tokens=6, warmup=2, profile_decode=True)
    p = r["decode_profile"]
    assert r["decode_engine"] == "persistent" and p["breakdown_ms"]["attn_total"] > 0 and p["breakdown_ms"]["mlp_total"] > 0
