"""Report tooling: metrics, repeat statistics, markdown table, profile folding (host logic, no GPU).

Formulas follow the reference's benchmark/decode/check_flashsvd_decode_correctness.py:183-197,270-276 and
benchmark/decode/collect_lowrankarena_main_table.py:157-295; profile categories utils/evaluator.py:646-660."""
import math
import os

import pytest
import torch

from flashsvd_amd import api, report as R


def test_metrics_known_values():
    x = torch.tensor([[1.0, -4.0], [2.0, 0.5]])
    y = torch.tensor([[1.5, -4.0], [1.0, 0.5]])
    assert R.max_abs(x, y) == 1.0 and R.mean_abs(x, y) == pytest.approx(0.375)
    assert R.rel_linf(x, y) == pytest.approx(0.25) and R.rel_linf(torch.zeros(3), torch.ones(3)) == 0.0
    assert R.token_match(torch.tensor([[1, 2, 3, 4]]), torch.tensor([[1, 9, 3, 4]])) == 0.75
    # uniform logits over V classes: CE = ln V, whatever the targets
    assert R.cross_entropy_from_logits(torch.zeros(2, 3, 7), torch.randint(0, 7, (2, 3))) == pytest.approx(math.log(7))
    # a one-hot-ish row: CE = -log softmax at the target
    logits = torch.tensor([[[2.0, 0.0, 0.0]]])
    assert R.cross_entropy_from_logits(logits, torch.tensor([[0]])) == pytest.approx(-math.log(math.e ** 2 / (math.e ** 2 + 2)))


def test_compare_mode_drops_last_full_position():
    g = torch.Generator().manual_seed(0)
    base = {"full_logits": torch.randn(1, 5, 6, generator=g), "decode_logits": torch.randn(1, 3, 6, generator=g),
            "greedy_tokens": torch.tensor([[1, 2, 3]])}
    cur = {"full_logits": base["full_logits"].clone(), "decode_logits": base["decode_logits"] + 0.5,
           "greedy_tokens": torch.tensor([[1, 2, 4]])}
    cur["full_logits"][:, -1] += 100.0          # the last prompt position predicts a token that is not a target
    m = R.compare_mode(base, cur, torch.randint(0, 6, (1, 4)), torch.randint(0, 6, (1, 3)))
    assert m["full_max_abs"] == 0.0 and m["decode_max_abs"] == pytest.approx(0.5) and m["decode_mean_abs"] == pytest.approx(0.5)
    assert m["greedy_token_match"] == pytest.approx(2 / 3)
    line = R.format_mode_line("flash_test", m)
    assert line.startswith("- flash_test: full_max_abs=0 ") and "| greedy_token_match=0.666667" in line


def test_configure_mode_flags(monkeypatch):
    for name in R._MODE_ENV:
        monkeypatch.delenv(name, raising=False)
    R.configure_mode("baseline", backend="baseline", enable_baseline_dense_kvcache=True)
    assert os.environ["SVDLLM_FLASH_FALLBACK"] == "1" and os.environ["FLASH_SVD_DISABLE_FFN"] == "1"
    assert os.environ["FLASH_SVD_FFN_BACKEND"] == "flashsvd_mlp_dual_split_exact_legacy"
    assert os.environ["FLASH_SVD_DENSE_DECODE_BACKEND"] == "exact" and os.environ["FLASH_SVD_BASELINE_DENSE_KVCACHE"] == "1"
    assert os.environ["FLASH_SVD_MLP_CUDA_GRAPH"] == "0"
    from flashsvd_amd.llama import mlp_rounding_mode
    assert mlp_rounding_mode() == 0
    R.configure_mode("flash", backend="flashsvd_mlp_dual_split_triton_v2_sm80", use_graph=True, graph_scope="layer_tail")
    assert os.environ["SVDLLM_FLASH_FALLBACK"] == "0" and os.environ["FLASH_SVD_ENABLE_EXPERIMENTAL_FFN"] == "1"
    assert os.environ["FLASH_SVD_MLP_CUDA_GRAPH"] == "1" and os.environ["FLASH_SVD_MLP_CUDA_GRAPH_SCOPE"] == "layer_tail"
    assert os.environ["FLASH_SVD_DENSE_DECODE_BACKEND"] == "packed" and mlp_rounding_mode() == 1
    R.configure_mode("flash", backend="flashsvd_mlp_dual_split_exact_legacy")
    assert os.environ["FLASH_SVD_ENABLE_EXPERIMENTAL_FFN"] == "0" and mlp_rounding_mode() == 0
    with pytest.raises(ValueError, match="Unsupported mode"):
        R.configure_mode("turbo", backend="x")


def _bench(prefill_s, decode_s, prompt=512, new=32):
    return {"prefill_time_s": prefill_s, "decode_time_s": decode_s, "prefill_tok_s": prompt / prefill_s,
            "decode_tok_s": new / decode_s, "decode_ms_per_token": decode_s * 1000 / new}


def test_pair_row_and_aggregate():
    r1 = R.pair_row(_bench(0.2, 1.6), _bench(0.1, 0.4))
    assert r1["prefill_speedup_x"] == pytest.approx(2.0) and r1["decode_speedup_x"] == pytest.approx(4.0)
    assert r1["baseline_e2e_time_s"] == pytest.approx(1.8) and r1["e2e_speedup_x"] == pytest.approx(3.6)
    r2 = R.pair_row(_bench(0.2, 1.2), _bench(0.1, 0.4))
    agg = R.aggregate_repeat_rows([dict(r1, repeat_index=1), dict(r2, repeat_index=2)])
    assert agg["status"] == "ok" and agg["ok_repeats"] == 2 and agg["requested_repeats"] == 2
    assert agg["decode_speedup_x"] == pytest.approx(3.5) and agg["decode_speedup_x_std"] == pytest.approx(math.sqrt(0.5))
    assert agg["decode_speedup_x_min"] == pytest.approx(3.0) and agg["decode_speedup_x_max"] == pytest.approx(4.0)
    assert set(f"{k}{s}" for k in R.METRIC_KEYS for s in ("", "_std", "_min", "_max")) <= set(agg)
    part = R.aggregate_repeat_rows([dict(r1, repeat_index=1), {"status": "error", "error": "boom", "repeat_index": 2}])
    assert part["status"] == "partial" and part["ok_repeats"] == 1 and part["decode_speedup_x_std"] == 0.0
    err = R.aggregate_repeat_rows([{"status": "error", "error": "boom", "traceback": "tb"}])
    assert err == {"status": "error", "ok_repeats": 0, "requested_repeats": 1, "error": "boom", "traceback": "tb"}
    assert R.aggregate_repeat_rows([])["error"] == "all repeats failed"


def test_markdown_rows(tmp_path):
    r1 = dict(R.pair_row(_bench(0.2, 1.6), _bench(0.1, 0.4)), repeat_index=1)
    ok = dict(family_name="SVD-LLM v1", ratio="0.5", checkpoint="/ck/a", repeats=[r1, {"status": "error", "error": "boom", "repeat_index": 2}])
    ok.update(R.aggregate_repeat_rows(ok["repeats"]))
    bad = dict(family_name="Basis Sharing", ratio="0.4", status="error", error="KeyError: missing", requested_repeats=0, checkpoint="/ck/b")
    cfg = dict(gpu="MI355X", device="cuda:0", dtype="bf16", prompt_len=512, new_tokens=32, warmup=3, batch_size=1, repeats=2,
               ffn_backend="flashsvd_mlp_dual_split_prod", decode_engine="auto")
    md = R.build_markdown(results=[ok, bad], config=cfg, md_path=tmp_path / "t.md")
    assert "| SVD-LLM v1 | 0.5 | 1/2 | 0.200 | 0.100 | 2.00x ± 0.00 | 50.000 | 12.500 | 4.00x ± 0.00 | 1.800 | 0.500 | 3.60x ± 0.00 |" in md
    assert "| Basis Sharing | 0.4 | 0/0 | fail | fail | fail | fail | fail | fail | fail | fail | fail |" in md
    assert "| SVD-LLM v1 | 0.5 | 1/2 | 2560 | 5120 | 20 | 80 | `/ck/a` |" in md
    assert "| SVD-LLM v1 | 0.5 | 2 | fail | fail | fail | fail | fail | boom |" in md
    assert "## Failures" in md and "- `Basis Sharing 0.4`: `KeyError: missing`" in md and "- GPU: `MI355X`" in md
    # every table row has as many cells as its header
    for block in md.split("\n\n"):
        rows = [l for l in block.splitlines() if l.startswith("|")]
        if rows:
            assert len({l.count("|") for l in rows}) == 1, block


def test_checkpoint_specs():
    assert R.parse_checkpoint_specs("SVD-LLM v1:0.5=/a/b, Basis Sharing:0.4=/c") == [("SVD-LLM v1", "0.5", "/a/b"),
                                                                                     ("Basis Sharing", "0.4", "/c")]
    assert R.parse_checkpoint_specs("=/x") == [("model", "-", "/x")]
    with pytest.raises(ValueError, match="expected"):
        R.parse_checkpoint_specs("/just/a/path")
    with pytest.raises(ValueError, match="no checkpoints"):
        R.parse_checkpoint_specs(" , ")


def test_collect_main_table_keeps_going_after_failures(monkeypatch):
    calls = []

    def fake_pair(model, **kw):
        calls.append(model)
        if model == "m2" and len([c for c in calls if c == "m2"]) == 1:
            raise RuntimeError("first repeat fails")
        return _bench(0.2, 1.6), _bench(0.1, 0.4)
    monkeypatch.setattr(R, "run_pair", fake_pair)

    def load(path):
        if path == "/missing":
            raise FileNotFoundError("no config.json")
        return path.strip("/")
    rows = R.collect_main_table([("A", "0.5", "/m1"), ("B", "0.5", "/m2"), ("C", "0.5", "/missing")], load=load, repeats=2)
    assert [r["status"] for r in rows] == ["ok", "partial", "error"]
    assert rows[1]["repeats"][0]["error"] == "RuntimeError: first repeat fails" and rows[1]["ok_repeats"] == 1
    assert rows[2]["error"].startswith("FileNotFoundError") and rows[0]["decode_speedup_x"] == pytest.approx(4.0)


def test_profile_folding():
    phases = {n: {"total": t} for n, t in (("embed", 2.0), ("attn_rank_proj", 10.0), ("qkv_u", 10.0), ("attn", 5.0), ("attn_merge", 1.0),
                                            ("o_v", 8.0), ("o_u", 6.0), ("mlp_rank_proj", 12.0), ("swiglu", 18.0), ("down_v", 20.0),
                                            ("down_u", 10.0), ("lm_head", 50.0), ("argmax", 3.0))}
    prof = api.decode_profile_from_phases(phases, 4, 0.5)
    b = prof["breakdown_ms"]
    assert b["attn_total"] == pytest.approx(4 * 0.040) and b["mlp_total"] == pytest.approx(4 * 0.060)
    assert b["lm_head"] == pytest.approx(0.053) and b["embed_tokens"] == pytest.approx(0.002)
    assert b["ln1_total"] == b["ln2_total"] == b["final_norm"] == 0.0
    assert prof["other_ms"] == pytest.approx(0.5 - 0.455) and set(b) == set(api._PROFILE_CATEGORIES)
    lines = api.format_decode_profile(prof)
    assert lines[1] == "=== Decode Profile (module device time) ===" and "total_forward 0.500 ms/token" in lines[2]
    assert lines[3].split(":")[0].strip() == "mlp_total" and "( 48.0%)" in lines[3]
    assert any(l.startswith("Top 10/10 modules:") for l in lines)
    # a total below the parts clamps "other" at zero
    assert api.decode_profile_from_phases(phases, 4, 0.1)["other_ms"] == 0.0
