"""PackedQuantLinear: buffers, quantisation rule and helpers against the oracle's restatement of
src/quant/packed_quant_linear.py and src/quant/common.py (host logic, no GPU)."""
import pytest
import torch
import torch.nn as nn

from flashsvd_amd import quant as Q
from oracle import flashsvd_oracle as O


@pytest.mark.parametrize("bits,group,sym", [(4, 32, False), (4, 128, True), (4, -1, False), (8, 64, False), (4, 40, False)])
def test_pack_weight_equals_oracle(bits, group, sym):
    g = torch.Generator().manual_seed(bits + group)
    lin = nn.Linear(200, 24, bias=True)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(24, 200, generator=g) * 0.05)
        lin.weight[3, :64] = 0.0                                   # a dead group
        lin.bias.copy_(torch.randn(24, generator=g))
    m = Q.PackedQuantLinear.from_linear(lin, bits=bits, group_size=group, sym=sym, compute_dtype=torch.float32)
    qw, sc, zr = O.quantize_weight(lin.weight, bits=bits, group_size=group, sym=sym)
    assert torch.equal(m.qweight, qw) and torch.equal(m.scales, sc) and torch.equal(m.zeros, zr)
    assert set(m.state_dict()) == {"qweight", "scales", "zeros", "bias"}
    w = O.dequantize_weight(qw, sc, zr, in_features=200, bits=bits, group_size=group)
    assert torch.equal(m.dequantize(dtype=torch.float32), w) and torch.equal(m.weight, w)
    assert torch.equal(m.dequantize(dtype=torch.bfloat16), w.to(torch.bfloat16))
    assert torch.equal(m.bias, lin.bias.detach())
    with pytest.raises(RuntimeError, match="GPU kernels only"):
        m(torch.zeros(1, 200))


def test_state_dict_round_trip_and_shapes():
    lin = nn.Linear(256, 16, bias=False)
    m = Q.PackedQuantLinear.from_linear(lin, bits=4, group_size=64, sym=False)
    fresh = Q.PackedQuantLinear(in_features=256, out_features=16, bits=4, group_size=64, bias=False)
    assert fresh.qweight.shape == (16, 128) and fresh.scales.shape == (16, 4) and fresh.zeros.shape == (16, 4)
    fresh.load_state_dict(m.state_dict())
    assert torch.equal(fresh.dequantize(dtype=torch.float32), m.dequantize(dtype=torch.float32))
    with pytest.raises(ValueError, match="4/8 bits"):
        Q.PackedQuantLinear(in_features=8, out_features=8, bits=3, group_size=8, bias=False)
    with pytest.raises(ValueError, match="weight shape mismatch"):
        fresh.pack_weight(torch.zeros(16, 255), bias=None, sym=False)


def test_which_calls_stream_int4(monkeypatch):
    monkeypatch.delenv("FLASH_SVD_QUANT_BACKEND", raising=False)
    m = Q.PackedQuantLinear(in_features=512, out_features=8, bits=4, group_size=128, bias=False)
    assert m.streams_int4(1) and m.streams_int4(16) and not m.streams_int4(17)
    assert not Q.PackedQuantLinear(in_features=384, out_features=8, bits=4, group_size=128, bias=False).streams_int4(1)   # K % 256
    assert not Q.PackedQuantLinear(in_features=512, out_features=8, bits=4, group_size=96, bias=False).streams_int4(1)    # group
    assert not Q.PackedQuantLinear(in_features=512, out_features=8, bits=8, group_size=128, bias=False).streams_int4(1)
    assert Q.PackedQuantLinear(in_features=512, out_features=8, bits=4, group_size=-1, bias=False).streams_int4(1)
    monkeypatch.setenv("FLASH_SVD_QUANT_BACKEND", "dense")
    assert not m.streams_int4(1)
    monkeypatch.setenv("FLASH_SVD_QUANT_BACKEND", "int4")
    assert m.streams_int4(4096)
    monkeypatch.setenv("FLASH_SVD_QUANT_BACKEND", "off")
    with pytest.raises(ValueError, match="FLASH_SVD_QUANT_BACKEND"):
        m.streams_int4(1)


def test_replace_and_rank_map():
    from tests.test_plan import tiny_model
    model = tiny_model([(8, 8, 8, 8), (16, 8, 8, 8)], [(8, 8), (8, 16)], dtype=torch.float32)
    names = Q.factor_linear_names(model)
    assert len(names) == 2 * 14 and names[0] == "model.layers.0.self_attn.q_v_proj" and len(set(names)) == len(names)
    n = Q.replace_linears_with_packed_quant_inplace(model, module_names=names[:4] + names[:2] + ["", "model.norm"], bits=4,
                                                    group_size=-1, sym=False)
    assert n == 4                                                  # duplicates, empty names and non-linears are skipped
    a0 = model.model.layers[0].self_attn
    assert isinstance(a0.q_v_proj, Q.PackedQuantLinear) and isinstance(a0.k_u_proj, Q.PackedQuantLinear)
    assert isinstance(a0.v_v_proj, nn.Linear) and Q.is_quantized(*a0._factor_modules())
    assert not Q.is_quantized(*model.model.layers[1].self_attn._factor_modules())
    rm = Q.extract_flashsvd_rank_map(model)
    assert rm["0"]["self_attn"] == {"q_rank": 8, "k_rank": 8, "v_rank": 8, "o_rank": 8}
    assert rm["1"]["self_attn"]["q_rank"] == 16 and rm["1"]["mlp"] == {"gate_rank": 8, "up_rank": 8, "down_rank": 16}
    assert a0._qkv_rank_tuple() == (8, 8, 8)
