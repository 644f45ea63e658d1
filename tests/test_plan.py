"""Dense-decode plan: rank padding, candidate rules, selection and the plan file (host logic, no GPU).

Rules follow the reference's benchmark/attn/generate_dense_decode_plan.py:28-150 (parsers, candidates) and
:312-462 (selection, file layout)."""
import json
import math

import pytest
import torch

from flashsvd_amd import llama, plan as P


def tiny_model(ranks_per_layer, mlp_ranks, dtype=torch.float64, seed=0):
    from types import SimpleNamespace
    cfg = SimpleNamespace(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8, intermediate_size=48,
                          num_hidden_layers=len(ranks_per_layer), vocab_size=11, rope_theta=10000.0, rms_norm_eps=1e-6,
                          hidden_act="silu", max_position_embeddings=64)
    model = llama.SVDLlamaForCausalLM(cfg, attn_ranks=dict(q=8, k=8, v=8, o=8), mlp_rank=8)
    g = torch.Generator().manual_seed(seed)
    for layer, (rq, rk, rv, ro), (rg, rd) in zip(model.model.layers, ranks_per_layer, mlp_ranks):
        a, m = layer.self_attn, layer.mlp
        for p, r, out, inp in (("q", rq, 32, 32), ("k", rk, 16, 32), ("v", rv, 16, 32), ("o", ro, 32, 32)):
            getattr(a, f"{p}_v_proj").weight = torch.nn.Parameter(torch.randn(r, inp, generator=g, dtype=dtype), requires_grad=False)
            getattr(a, f"{p}_u_proj").weight = torch.nn.Parameter(torch.randn(out, r, generator=g, dtype=dtype), requires_grad=False)
        for p, r, out, inp in (("gate", rg, 48, 32), ("up", rg, 48, 32), ("down", rd, 32, 48)):
            getattr(m, f"{p}_v_proj").weight = torch.nn.Parameter(torch.randn(r, inp, generator=g, dtype=dtype), requires_grad=False)
            getattr(m, f"{p}_u_proj").weight = torch.nn.Parameter(torch.randn(out, r, generator=g, dtype=dtype), requires_grad=False)
        for blk, names in ((a, "qkvo"), (m, ("gate", "up", "down"))):
            for p in names:
                for f in "uv":
                    lin = getattr(blk, f"{p}_{f}_proj")
                    lin.out_features, lin.in_features = lin.weight.shape
    return model


def test_parsers():
    assert P.parse_pad_multiples("1, 8,8, 0,16") == [1, 8, 16]          # 0 clamps to 1, duplicates dropped
    assert P.parse_pad_multiples("") == [1, 8, 16, 32, 64]
    assert P.parse_int_list("512,0,512", default=[0, 512]) == [512, 0]
    assert P.parse_int_list(" , ", default=[0, 512]) == [0, 512]
    assert P.is_finite_number("1.5") and not P.is_finite_number(float("nan")) and not P.is_finite_number(float("inf"))
    assert not P.is_finite_number(None)


def test_padded_ranks():
    assert P.padded_ranks((1492, 1100, 1024), 8) == (1496, 1104, 1024)
    assert P.padded_ranks((1492, 1100, 1024), 64) == (1536, 1152, 1024)
    assert P.padded_ranks((1492, 1100, 1024), 64, "uniform_layer") == (1536, 1536, 1536)
    assert P.padded_ranks((5, 7), 1) == (5, 7) and P.padded_ranks((5, 7), 0) == (5, 7)
    with pytest.raises(ValueError, match="pad mode"):
        P.padded_ranks((5,), 8, "diagonal")


def test_padding_is_exact_and_in_place():
    model = tiny_model([(5, 7, 6, 9), (12, 3, 3, 4)], [(10, 13), (16, 5)])
    x = torch.randn(3, 32, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    h = torch.randn(3, 48, dtype=torch.float64, generator=torch.Generator().manual_seed(2))

    def products(m):
        out = []
        for layer in m.model.layers:
            a, f = layer.self_attn, layer.mlp
            out += [getattr(a, f"{p}_u_proj")(getattr(a, f"{p}_v_proj")(x)) for p in "qkvo"]
            out += [getattr(f, f"{p}_u_proj")(getattr(f, f"{p}_v_proj")(x)) for p in ("gate", "up")]
            out.append(f.down_u_proj(f.down_v_proj(h)))
        return out
    before = products(model)
    rep = P.pad_model_ranks(model, 8, "uniform_layer")
    a0, a1 = model.model.layers[0].self_attn, model.model.layers[1].self_attn
    assert a0._qkv_rank_tuple() == (8, 8, 8) and a1._qkv_rank_tuple() == (16, 16, 16)
    assert a0._unpadded_qkv_ranks == (5, 7, 6) and a0.low_rank == 8
    assert rep["layers"][0] == {"q": (5, 8), "k": (7, 8), "v": (6, 8), "o": (9, 16), "gate": (10, 16), "up": (10, 16), "down": (13, 16)}
    assert rep["layers"][1]["gate"] == (16, 16) and rep["layers"][1]["down"] == (5, 8)
    assert a0.q_v_proj.out_features == 8 and a0.q_u_proj.in_features == 8 and a0.o_u_proj.in_features == 16
    # the added rows / columns are zero, and the products did not move by a single bit (fp64, zeros add nothing)
    assert float(a0.q_v_proj.weight[5:].abs().max()) == 0.0 and float(a0.q_u_proj.weight[:, 5:].abs().max()) == 0.0
    for b, a in zip(before, products(model)):
        assert torch.equal(a, b)
    assert rep["added_bytes"] == sum(
        ((t - r) * (inp + out)) * 8 for (r, t, inp, out) in
        [(5, 8, 32, 32), (7, 8, 32, 16), (6, 8, 32, 16), (9, 16, 32, 32), (10, 16, 32, 48), (10, 16, 32, 48), (13, 16, 48, 32),
         (12, 16, 32, 32), (3, 16, 32, 16), (3, 16, 32, 16), (4, 8, 32, 32), (5, 8, 48, 32)])
    # idempotent
    assert P.pad_model_ranks(model, 8, "uniform_layer")["added_bytes"] == 0


def test_padding_keeps_shared_weights_shared():
    model = tiny_model([(5, 5, 5, 5), (5, 5, 5, 5)], [(6, 6), (6, 6)])
    l0, l1 = model.model.layers
    l1.self_attn.q_v_proj.weight = l0.self_attn.q_v_proj.weight
    P.pad_model_ranks(model, 8)
    assert l1.self_attn.q_v_proj.weight is l0.self_attn.q_v_proj.weight and l0.self_attn.q_v_proj.weight.shape == (8, 32)
    assert l1.self_attn.q_u_proj.weight is not l0.self_attn.q_u_proj.weight


def test_pad_factor_pair_errors():
    model = tiny_model([(5, 5, 5, 5)], [(6, 6)])
    a = model.model.layers[0].self_attn
    with pytest.raises(ValueError, match="cannot pad rank 5 down to 4"):
        P.pad_factor_pair(a.q_v_proj, a.q_u_proj, 4)
    with pytest.raises(ValueError, match="does not chain"):
        P.pad_factor_pair(a.q_v_proj, model.model.layers[0].mlp.gate_u_proj, 8)
    assert P.pad_factor_pair(a.q_v_proj, a.q_u_proj, 5) is False


def test_reconstruct_candidates_follow_the_reference_rule():
    res = dict(exact_ms=1.0, rq=100, rk=100, rv=100, packed_linear_ms=0.5, packed_torch_ms=0.4)
    c = P.build_candidates(layer_idx=3, actual_ranks=(100, 100, 100), result=res, pad_multiple=1, include_exact=True)
    assert [(x["backend"], x["impl"]) for x in c] == [("exact", "exact"), ("packed", "packed_linear")]   # flat not distinct
    assert c[1]["speedup_vs_exact"] == 2.0 and c[0]["pad_multiple"] == 1 and c[0]["split_sizes"] == [100, 100, 100]
    res = dict(exact_ms=1.0, rq=104, rk=104, rv=104, packed_linear_ms=float("nan"), packed_torch_ms=0.4)
    c = P.build_candidates(layer_idx=3, actual_ranks=(100, 100, 100), result=res, pad_multiple=8, include_exact=False)
    assert [(x["impl"], x["pad_multiple"], x["split_sizes"]) for x in c] == [("packed_flat", 8, [104, 104, 104])]
    # unpadded sizes but no usable packed_linear time: flat steps in
    res = dict(exact_ms=1.0, rq=100, rk=100, rv=100, packed_linear_ms=float("nan"), packed_torch_ms=0.4)
    c = P.build_candidates(layer_idx=3, actual_ranks=(100, 100, 100), result=res, pad_multiple=1, include_exact=False)
    assert [x["impl"] for x in c] == ["packed_flat"]
    res["packed_torch_ms"] = float("inf")
    assert P.build_candidates(layer_idx=3, actual_ranks=(100, 100, 100), result=res, pad_multiple=1, include_exact=False) == []


def test_selection_prefers_packed_on_ties():
    c = P.build_attention_candidates(layer_idx=0, actual_ranks=(5, 5, 5), split_sizes=(8, 8, 8), exact_ms=0.2, packed_ms=0.2,
                                     pad_multiple=8)
    assert P.select_best(c)["backend"] == "packed"
    c = P.build_attention_candidates(layer_idx=0, actual_ranks=(5, 5, 5), split_sizes=(8, 8, 8), exact_ms=0.1, packed_ms=0.2,
                                     pad_multiple=8)
    best = P.select_best(c)
    assert best["backend"] == "exact" and best["split_sizes"] == [5, 5, 5] and best["pad_multiple"] == 1


def _measurements():
    def cands(layer, exact, packed_by_mult, actual):
        out = []
        for mult, ms in packed_by_mult.items():
            out += P.build_attention_candidates(layer_idx=layer, actual_ranks=actual, split_sizes=P.padded_ranks(actual, mult),
                                                exact_ms=exact, packed_ms=ms, pad_multiple=mult)
        return out
    return {
        0: {"actual_ranks": (100, 100, 100), "buckets": {0: cands(0, 0.30, {1: 0.20, 8: 0.10, 64: 0.12}, (100, 100, 100)),
                                                          512: cands(0, 0.35, {1: 0.25, 8: 0.16, 64: 0.15}, (100, 100, 100))}},
        1: {"actual_ranks": (60, 40, 40), "buckets": {0: cands(1, 0.05, {1: 0.20, 8: 0.10, 64: 0.12}, (60, 40, 40)),
                                                       512: cands(1, 0.50, {1: 0.25, 8: 0.16, 64: 0.17}, (60, 40, 40))}},
    }


def test_assemble_plan_layout(tmp_path):
    plan = P.assemble_plan(_measurements(), mode="attention", source={"checkpoint": "x", "mode": "attention"})
    assert plan["format"] == "flashsvd_dense_decode_plan_v2"
    assert set(plan) == {"format", "source", "defaults", "summary", "layers"}
    l0, l1 = plan["layers"]["0"], plan["layers"]["1"]
    assert (l0["backend"], l0["impl"], l0["pad_multiple"], l0["split_sizes"], l0["bucket"]) == \
        ("packed", "packed_attention", 8, [104, 104, 104], "104_104_104")
    assert l0["default_past_bucket"] == 0 and l0["qkv_ranks"] == [100, 100, 100] and l0["best_ms"] == 0.10
    assert l0["best_speedup_vs_exact"] == pytest.approx(3.0)
    assert l0["buckets"]["512"]["pad_multiple"] == 64 and l0["buckets"]["512"]["split_sizes"] == [128, 128, 128]
    assert [c["ms"] for c in l0["buckets"]["0"]["candidates"]] == sorted(c["ms"] for c in l0["buckets"]["0"]["candidates"])
    assert len(l0["buckets"]["0"]["candidates"]) == 6
    assert l1["backend"] == "exact" and l1["split_sizes"] == [60, 40, 40] and l1["buckets"]["512"]["backend"] == "packed"
    assert plan["defaults"] == {"backend": "packed", "pad_multiple": 8}
    assert plan["summary"]["backend_counts"] == {"packed": 3, "exact": 1}
    assert plan["summary"]["pad_counts"] == {"8": 2, "64": 1, "1": 1}
    assert plan["summary"]["past_bucket_counts"] == {"0": 2, "512": 2}
    assert plan["summary"]["bucket_counts"]["104_104_104"] == 1
    path = P.save_plan(plan, tmp_path / "sub" / "plan.json")
    assert P.load_plan(path) == json.loads(json.dumps(plan))
    # v1 layout for reconstruct mode: one bucket (-1), candidates at layer level, no bucket table
    res = dict(exact_ms=1.0, rq=100, rk=100, rv=100, packed_linear_ms=0.5, packed_torch_ms=0.4)
    m = {0: {"actual_ranks": (100, 100, 100),
             "buckets": {-1: P.build_candidates(layer_idx=0, actual_ranks=(100, 100, 100), result=res, pad_multiple=1, include_exact=True)}}}
    v1 = P.assemble_plan(m, mode="reconstruct", source={})
    assert v1["format"] == "flashsvd_dense_decode_plan_v1" and "buckets" not in v1["layers"]["0"]
    assert [c["impl"] for c in v1["layers"]["0"]["candidates"]] == ["packed_linear", "exact"]
    assert v1["summary"]["past_bucket_counts"] == {}


def test_load_plan_rejects_other_files(tmp_path):
    (tmp_path / "a.json").write_text(json.dumps({"format": "something_else", "layers": {}}))
    with pytest.raises(ValueError, match="not a dense-decode plan"):
        P.load_plan(tmp_path / "a.json")
    (tmp_path / "b.json").write_text(json.dumps({"format": P.PLAN_FORMAT_ATTENTION}))
    with pytest.raises(ValueError, match="no layer table"):
        P.load_plan(tmp_path / "b.json")


def test_plan_choice_buckets():
    plan = P.assemble_plan(_measurements(), mode="attention", source={})
    e = plan["layers"]["1"]
    assert P.plan_choice(e) == "exact"                       # layer default
    assert P.plan_choice(e, 0) == "exact" and P.plan_choice(e, 511) == "exact"
    assert P.plan_choice(e, 512) == "packed" and P.plan_choice(e, 100000) == "packed"
    assert P.plan_choice(None) == "packed" and P.plan_choice({"backend": "auto"}) == "packed"
    with pytest.raises(ValueError, match="dense-decode backend"):
        P.plan_choice({"backend": "cutlass"})


def test_apply_plan_pads_and_sets_backends():
    model = tiny_model([(100, 100, 100, 100), (60, 40, 40, 50), (9, 9, 9, 9)], [(8, 8)] * 3, dtype=torch.float32)
    plan = P.assemble_plan(_measurements(), mode="attention", source={})
    out = P.apply_dense_decode_plan(model, plan)
    assert out == {0: ("packed", (104, 104, 104)), 1: ("exact", (60, 40, 40)), 2: ("packed", (16, 16, 16))}   # layer 2: defaults
    a0, a1, a2 = (l.self_attn for l in model.model.layers)
    assert a0._qkv_rank_tuple() == (104, 104, 104) and a0.o_v_proj.out_features == 100
    assert a0._dense_decode_backend() == "packed" and a1._dense_decode_backend() == "exact" and a2._dense_decode_backend() == "packed"

    class Cache:
        def __init__(self, n): self.n = n
        def get_seq_length(self): return self.n
    assert a1._dense_decode_backend(Cache(3)) == "exact" and a1._dense_decode_backend(Cache(600)) == "packed"
    # a second application sees the padded model as the one the plan was measured on
    assert P.apply_dense_decode_plan(model, plan)[0] == ("packed", (104, 104, 104))
    other = tiny_model([(96, 96, 96, 96)], [(8, 8)], dtype=torch.float32)
    with pytest.raises(ValueError, match="measured for ranks"):
        P.apply_dense_decode_plan(other, plan)
    # without padding only the backends are installed
    fresh = tiny_model([(100, 100, 100, 100), (60, 40, 40, 50)], [(8, 8)] * 2, dtype=torch.float32)
    assert P.apply_dense_decode_plan(fresh, plan, pad=False)[0] == ("packed", (100, 100, 100))


def test_backend_env(monkeypatch):
    a = tiny_model([(8, 8, 8, 8)], [(8, 8)], dtype=torch.float32).model.layers[0].self_attn
    monkeypatch.delenv("FLASH_SVD_DENSE_DECODE_BACKEND", raising=False)
    assert a._dense_decode_backend() == "packed"
    for raw, want in (("auto", "packed"), ("exact", "exact"), ("PACKED", "packed")):
        monkeypatch.setenv("FLASH_SVD_DENSE_DECODE_BACKEND", raw)
        assert a._dense_decode_backend() == want
    monkeypatch.setenv("FLASH_SVD_DENSE_DECODE_BACKEND", "cutlass")
    with pytest.raises(ValueError, match="FLASH_SVD_DENSE_DECODE_BACKEND"):
        a._dense_decode_backend()
