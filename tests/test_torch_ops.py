"""The custom operators flashsvd_hip::* (flashsvd_amd/torch_ops.py): registration, schemas and the fake / meta shape
functions run here without a GPU; the device implementations are exercised by every GPU test, which reach the library
through these operators, and by torch.library.opcheck in the GPU part below."""
import pytest
import torch

BF16 = torch.bfloat16


def _m(*shape, dtype=BF16):
    return torch.empty(*shape, dtype=dtype, device="meta")


def test_every_operator_is_registered_with_a_schema():
    from flashsvd_amd import torch_ops as T
    for name in T.OP_NAMES:
        packet = getattr(torch.ops.flashsvd_hip, name)
        schema = str(packet.default._schema)
        assert schema.startswith(f"flashsvd_hip::{name}("), schema
    # mutated arguments are declared: the caches of the append / attention operators, the output overloads
    assert "Tensor(a!) k_cache" in str(torch.ops.flashsvd_hip.qkv_rope_append.default._schema)
    assert "Tensor(a!) out" in str(torch.ops.flashsvd_hip.linear.out._schema)
    assert "Tensor(a!) pk_cache" in str(torch.ops.flashsvd_hip.rankkv_append.default._schema)


def test_meta_shape_functions():
    ops = torch.ops.flashsvd_hip
    B, d, R, D, H, Hk, Dh, S = 3, 256, 64, 512, 4, 2, 128, 40
    x = _m(B, 1, d)
    assert ops.linear(x, _m(R, d)).shape == (B, 1, R)
    assert ops.linear(x, _m(R, d), None, _m(d), 1e-6, None, 0).dtype == BF16
    out = _m(B, 1, R)
    assert ops.linear.out(x, _m(R, d), out=out) is out
    assert ops.swiglu_linear(_m(B, 2 * R), _m(D, R), _m(D, R), R).shape == (B, D)
    assert ops.rmsnorm(x, _m(d)).shape == x.shape
    kc = _m(B, S, Hk, Dh)
    q = ops.qkv_rope_append(_m(B, 3 * R), _m(H * Dh, R), _m(Hk * Dh, R), _m(Hk * Dh, R), _m(S, Dh // 2), _m(S, Dh // 2),
                            _m(B, dtype=torch.int32), kc, _m(B, S, Hk, Dh), H, Hk, Dh)
    assert q.shape == (B, H, Dh)
    assert ops.attn_decode_densekv(q, kc, kc, _m(B, dtype=torch.int32)).shape == (B, H, Dh)
    assert ops.attn_decode_rankkv(q, _m(B, S, R), _m(B, S, R), _m(Hk * Dh, R), _m(Hk * Dh, R), None, None,
                                  _m(B, dtype=torch.int32), Hk).shape == (B, H, Dh)
    assert ops.rope_attn_prefill(_m(B, 9, H, Dh), _m(B, S, Hk, Dh), _m(B, S, Hk, Dh)).shape == (B, 9, H, Dh)
    Q, K, V = ops.reconstruct_qkv_token(_m(B, H, R), _m(B, Hk, R), _m(B, Hk, R), _m(H, R, Dh), _m(Hk, R, Dh), _m(Hk, R, Dh))
    assert Q.shape == (B, H, Dh) and K.shape == V.shape == (B, Hk, Dh)
    assert ops.xw_linear(_m(B, d), _m(d, R)).shape == (B, R)
    assert ops.mlp_dual_split(_m(B, R), _m(B, R), _m(R, D), _m(R, D), _m(D, R), _m(R, d), None, 2, 128).shape == (B, d)
    assert ops.rankkv_append(_m(B, R), _m(B, R), _m(B, S, R), _m(B, S, R), _m(B, dtype=torch.int32)) is None
    assert ops.lowrank_expand_heads(_m(B, 9, R), _m(H * Dh, R), H, Dh, _m(B, 9, H, Dh)) is None


def test_host_tensors_raise_value_error_through_the_dispatcher():
    from flashsvd_amd import hip_ops
    with pytest.raises(ValueError, match="GPU tensor"):
        hip_ops.linear(torch.zeros(1, 64, dtype=BF16), torch.zeros(8, 64, dtype=BF16))
    with pytest.raises(ValueError, match="GPU tensor"):
        torch.ops.flashsvd_hip.rmsnorm(torch.zeros(1, 64, dtype=BF16), torch.ones(64, dtype=BF16))


@pytest.mark.gpu
def test_opcheck_and_fake_tensor_tracing_on_the_device():
    """torch.library.opcheck (schema and fake-tensor consistency against the real kernels) on the hot operators, and a
    make_fx trace of a low-rank MLP through fake tensors that records the custom operators as graph nodes."""
    from torch.fx.experimental.proxy_tensor import make_fx
    from tests.util import rand_bf16
    ops = torch.ops.flashsvd_hip
    d, R, D = 512, 128, 768
    x = rand_bf16(1, d, seed=1).cuda()
    vw, gu, uu = rand_bf16(2 * R, d, std=0.05, seed=2).cuda(), rand_bf16(D, R, std=0.05, seed=3).cuda(), rand_bf16(D, R, std=0.05, seed=4).cuda()
    dv, du, nw = rand_bf16(R, D, std=0.05, seed=5).cuda(), rand_bf16(d, R, std=0.05, seed=6).cuda(), torch.ones(d, dtype=BF16, device="cuda")
    checks = ("test_schema", "test_faketensor")
    torch.library.opcheck(ops.linear.default, (x, vw, None, nw, 1e-6, None, 0), test_utils=checks)
    torch.library.opcheck(ops.linear.out, (x, vw), dict(out=torch.empty(1, 2 * R, dtype=BF16, device="cuda")), test_utils=checks)
    p = ops.linear(x, vw, None, nw)
    torch.library.opcheck(ops.swiglu_linear.default, (p, gu, uu, R), test_utils=checks)
    torch.library.opcheck(ops.rmsnorm.default, (x, nw), test_utils=checks)
    H, Dh, S = 2, 128, 32
    kc, vc = rand_bf16(1, S, H, Dh, seed=7).cuda(), rand_bf16(1, S, H, Dh, seed=8).cuda()
    lens = torch.tensor([20], dtype=torch.int32, device="cuda")
    q = rand_bf16(1, H, Dh, seed=9).cuda()
    torch.library.opcheck(ops.attn_decode_densekv.default, (q, kc, vc, lens), dict(nsplit=2), test_utils=checks)

    def mlp(x, vw, gu, uu, dv, du, nw):
        p = ops.linear(x, vw, None, nw, 1e-6)
        h = ops.swiglu_linear(p, gu, uu, R)
        return ops.linear(ops.linear(h, dv), du, None, None, 1e-6, x)

    args = (x, vw, gu, uu, dv, du, nw)
    g = make_fx(mlp, tracing_mode="fake")(*args)
    targets = [n.target for n in g.graph.nodes if n.op == "call_function"]
    assert targets.count(ops.linear.default) == 3 and ops.swiglu_linear.default in targets
    assert torch.equal(g(*args), mlp(*args))
