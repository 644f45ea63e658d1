"""GPU parity of the operator-level API that keeps the reference's names and layouts
(reconstruct_qkv_token*, flashsvd_mlp_dual_split_*), against the CPU oracle.  bf16/fp16 results
within max-abs 2e-2 / max-rel 1e-2 (two bf16 ulps where |ref| >= 2); fp32 within 1e-4."""
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16

pytestmark = pytest.mark.gpu


def rnd(*shape, dtype=torch.bfloat16, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def tol(ref, dtype):
    if dtype == torch.float32:
        return dict(abs_tol=1e-4 * max(1.0, float(ref.abs().max())), rel_tol=1e-4)
    m = float(ref.float().abs().max())
    return dict(abs_tol=2e-2 if m < 2 else 2 * m * 2.0 ** -7, rel_tol=1e-2)


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available()
    import flashsvd_amd.kernels as k
    return k


SHAPES = [(1, 32, 32, 128, 1024), (2, 8, 2, 64, 52), (3, 4, 4, 128, 200), (1, 2, 1, 64, 8)]


@pytest.mark.parametrize("B,H,Hk,Dh,R", SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_reconstruct_shared_all_variants(K, B, H, Hk, Dh, R, dtype):
    Pq, Pk, Pv = rnd(B, R, dtype=dtype, seed=1), rnd(B, R, dtype=dtype, seed=2), rnd(B, R, dtype=dtype, seed=3)
    Vq, Vk, Vv = rnd(H, R, Dh, dtype=dtype, std=0.05, seed=4), rnd(Hk, R, Dh, dtype=dtype, std=0.05, seed=5), rnd(Hk, R, Dh, dtype=dtype, std=0.05, seed=6)
    bq, bk, bv = rnd(H, Dh, dtype=dtype, std=0.1, seed=7), rnd(Hk, Dh, dtype=dtype, std=0.1, seed=8), rnd(Hk, Dh, dtype=dtype, std=0.1, seed=9)
    ref = O.reconstruct_qkv_token_shared(Pq, Pk, Pv, Vq, Vk, Vv, bq, bk, bv)
    g = [t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)]
    gb = dict(bq=bq.cuda(), bk=bk.cuda(), bv=bv.cuda())
    outs = {
        "shared": K.reconstruct_qkv_token_shared(*g, **gb, BD=128, BR=128, num_warps=8, num_stages=2),
        "hetero": K.reconstruct_qkv_token_shared_hetero(*g, **gb),
        "headwise": K.reconstruct_qkv_token(g[0][:, None].expand(B, H, R), g[1][:, None].expand(B, Hk, R),
                                            g[2][:, None].expand(B, Hk, R), *g[3:], **gb),
    }
    flats = K.pack_qkv_shared_bases(*g[3:])
    assert flats[0].shape == (R, H * Dh) and flats[1].shape == (R, Hk * Dh)
    outs["prepacked"] = K.reconstruct_qkv_token_shared_prepacked(*g[:3], *flats, H=H, Hk=Hk, Dh=Dh, **gb)
    ref_pre = O.reconstruct_qkv_token_shared_prepacked(Pq, Pk, Pv, *O.pack_qkv_shared_bases(Vq, Vk, Vv), H=H, Hk=Hk, Dh=Dh, bq=bq, bk=bk, bv=bv)
    for name, got in outs.items():
        r = ref_pre if name == "prepacked" else ref
        for a, b, nm in zip(got, r, "QKV"):
            assert a.dtype == dtype and a.is_contiguous()
            assert_close_bf16(a, b, f"{name} {nm}", **tol(b, dtype))
    # no bias
    got = K.reconstruct_qkv_token_shared(*g)
    for a, b in zip(got, O.reconstruct_qkv_token_shared(Pq, Pk, Pv, Vq, Vk, Vv)):
        assert_close_bf16(a, b, "no bias", **tol(b, dtype))


def test_reconstruct_headwise_distinct_P(K):
    B, H, Hk, Dh, R = 2, 8, 4, 64, 40
    Pq, Pk, Pv = rnd(B, H, R, seed=1), rnd(B, Hk, R, seed=2), rnd(B, Hk, R, seed=3)
    Vq, Vk, Vv = rnd(H, R, Dh, std=0.1, seed=4), rnd(Hk, R, Dh, std=0.1, seed=5), rnd(Hk, R, Dh, std=0.1, seed=6)
    got = K.reconstruct_qkv_token(*[t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)])
    for a, b in zip(got, O.reconstruct_qkv_token(Pq, Pk, Pv, Vq, Vk, Vv)):
        assert_close_bf16(a, b, "headwise", **tol(b, torch.bfloat16))


def test_reconstruct_hetero_ranks(K):
    B, H, Hk, Dh = 2, 8, 4, 128
    Rq, Rk, Rv = 1492, 300, 24
    Pq, Pk, Pv = rnd(B, Rq, seed=1), rnd(B, Rk, seed=2), rnd(B, Rv, seed=3)
    Vq, Vk, Vv = rnd(H, Rq, Dh, std=0.03, seed=4), rnd(Hk, Rk, Dh, std=0.05, seed=5), rnd(Hk, Rv, Dh, std=0.1, seed=6)
    got = K.reconstruct_qkv_token_shared_hetero(*[t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)])
    for a, b, nm in zip(got, O.reconstruct_qkv_token_shared_hetero(Pq, Pk, Pv, Vq, Vk, Vv), "QKV"):
        assert_close_bf16(a, b, nm, **tol(b, torch.bfloat16))


def test_reconstruct_errors(K):
    c = lambda *s: rnd(*s).cuda()
    with pytest.raises(ValueError, match="expects all tensors on CUDA"):
        K.reconstruct_qkv_token_shared(rnd(1, 8), c(1, 8), c(1, 8), c(2, 8, 64), c(2, 8, 64), c(2, 8, 64))
    with pytest.raises(ValueError, match="2D"):
        K.reconstruct_qkv_token_shared(c(1, 2, 8), c(1, 8), c(1, 8), c(2, 8, 64), c(2, 8, 64), c(2, 8, 64))
    with pytest.raises(ValueError, match="Mismatched"):
        K.reconstruct_qkv_token_shared(c(1, 8), c(1, 16), c(1, 8), c(2, 8, 64), c(2, 8, 64), c(2, 8, 64))
    with pytest.raises(ValueError, match="Expected bq shape"):
        K.reconstruct_qkv_token_shared(c(1, 8), c(1, 8), c(1, 8), c(2, 8, 64), c(2, 8, 64), c(2, 8, 64), bq=c(3, 64))
    with pytest.raises(ValueError, match="Expected Vk rank"):
        K.reconstruct_qkv_token_shared_hetero(c(1, 8), c(1, 16), c(1, 8), c(2, 8, 64), c(2, 8, 64), c(2, 8, 64))
    with pytest.raises(ValueError, match="Vq_flat shape"):
        K.reconstruct_qkv_token_shared_prepacked(c(1, 8), c(1, 8), c(1, 8), c(8, 100), c(8, 128), c(8, 128), H=2, Hk=2, Dh=64)


MLP_SHAPES = [(1, 1, 1536, 11008, 4096), (8, 1, 1536, 11008, 4096), (32, 1, 1536, 11008, 4096), (2, 3, 52, 300, 72), (1, 1, 256, 1376, 512)]


@pytest.mark.parametrize("B,L,R,D,Hd", MLP_SHAPES)
def test_dual_split_variants_bf16(K, B, L, R, D, Hd):
    dt = torch.bfloat16
    PUp, PGate = rnd(B, L, R, seed=1), rnd(B, L, R, seed=2)
    GateU, UpU = rnd(R, D, std=0.03, seed=3), rnd(R, D, std=0.03, seed=4)
    DownV, DownU, b2 = rnd(D, R, std=0.03, seed=5), rnd(R, Hd, std=0.03, seed=6), rnd(Hd, std=0.1, seed=7)
    g = [t.cuda() for t in (PUp, PGate, GateU, UpU, DownV, DownU)]
    ref2 = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2)
    ref1 = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=128, variant="v1", work_dtype=dt)
    ref3 = O.dual_split_mlp_v3(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=128, BR2=R)
    s2d = torch.empty(B * L, R, dtype=torch.float32, device="cuda")
    outs = {
        "v1": (K.flashsvd_mlp_dual_split_triton_v1(*g, b2.cuda()), ref1),
        "v1_fp32": (K.flashsvd_mlp_dual_split_triton_v1(*g, b2.cuda(), store_partials_fp32=True), ref2),
        "v2": (K.flashsvd_mlp_dual_split_triton_v2(*g, b2.cuda(), workspace_s2d=s2d), ref2),
        "v2_sm80": (K.flashsvd_mlp_dual_split_triton_v2_sm80(*g, b2.cuda()), ref2),
        "v3": (K.flashsvd_mlp_dual_split_triton_v3(*g, b2.cuda()), ref3),
        "pcat_s": (K.flashsvd_mlp_dual_split_triton_pcat_s(torch.cat([g[0], g[1]], -1), *g[2:], b2.cuda()), ref2),
        "alias": (K.flashsvd_ffn_dual_split_token_v2(*g), O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU)),
    }
    for name, (got, ref) in outs.items():
        assert got.shape == (B, L, Hd) and got.dtype == dt
        assert_close_bf16(got, ref, name, **tol(ref, dt))
    # workspace_s2d holds the fp32 S of the call
    g32 = (PGate.reshape(-1, R).float() @ GateU.float())
    u32 = (PUp.reshape(-1, R).float() @ UpU.float())
    S = ((g32 * torch.sigmoid(g32)) * u32).to(dt).float() @ DownV.float()
    assert_close_bf16(s2d, S, "S in workspace_s2d", abs_tol=1e-2 * float(S.abs().max()), rel_tol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_dual_split_other_dtypes(K, dtype):
    B, L, R, D, Hd = 2, 1, 96, 520, 64
    PUp, PGate = rnd(B, L, R, dtype=dtype, seed=1), rnd(B, L, R, dtype=dtype, seed=2)
    GateU, UpU = rnd(R, D, dtype=dtype, std=0.05, seed=3), rnd(R, D, dtype=dtype, std=0.05, seed=4)
    DownV, DownU = rnd(D, R, dtype=dtype, std=0.05, seed=5), rnd(R, Hd, dtype=dtype, std=0.05, seed=6)
    ref = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU)
    got = K.flashsvd_mlp_dual_split_triton_v2(*[t.cuda() for t in (PUp, PGate, GateU, UpU, DownV, DownU)])
    assert_close_bf16(got, ref, str(dtype), **tol(ref, dtype))


def test_dual_split_two_calls_reuse_scratch(K):
    # second, smaller call after a larger one: counters must have returned to zero
    for (B, R, D, Hd) in ((4, 128, 1000, 256), (1, 64, 300, 128)):
        PUp, PGate = rnd(B, 1, R, seed=1), rnd(B, 1, R, seed=2)
        GateU, UpU, DownV, DownU = rnd(R, D, std=0.05, seed=3), rnd(R, D, std=0.05, seed=4), rnd(D, R, std=0.05, seed=5), rnd(R, Hd, std=0.05, seed=6)
        ref = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU)
        got = K.flashsvd_mlp_dual_split_triton_v2(*[t.cuda() for t in (PUp, PGate, GateU, UpU, DownV, DownU)])
        assert_close_bf16(got, ref, f"call {B}", **tol(ref, torch.bfloat16))


def test_dual_split_errors(K):
    c = lambda *s: rnd(*s).cuda()
    with pytest.raises(ValueError, match=r"PUp/PGate must be \[B, L, R\]"):
        K.flashsvd_mlp_dual_split_triton_v2(c(1, 8), c(1, 8), c(8, 32), c(8, 32), c(32, 8), c(8, 16))
    with pytest.raises(ValueError, match="GateU must be"):
        K.flashsvd_mlp_dual_split_triton_v2(c(1, 1, 8), c(1, 1, 8), c(9, 32), c(9, 32), c(32, 8), c(8, 16))
    with pytest.raises(ValueError, match="DownV must be"):
        K.flashsvd_mlp_dual_split_triton_v1(c(1, 1, 8), c(1, 1, 8), c(8, 32), c(8, 32), c(31, 8), c(8, 16))
    with pytest.raises(ValueError, match="workspace_s2d must have dtype float32"):
        K.flashsvd_mlp_dual_split_triton_v2(c(1, 1, 8), c(1, 1, 8), c(8, 32), c(8, 32), c(32, 8), c(8, 16), workspace_s2d=c(1, 8))
    with pytest.raises(ValueError, match="PCat last dim must be even"):
        K.flashsvd_mlp_dual_split_triton_pcat_s(c(1, 1, 9), c(4, 32), c(4, 32), c(32, 4), c(4, 16))
    with pytest.raises(AssertionError):
        K.flashsvd_mlp_dual_split_triton_v2(rnd(1, 1, 8), c(1, 1, 8), c(8, 32), c(8, 32), c(32, 8), c(8, 16))


def test_reference_layout_fast_route_against_the_input_major_kernels(K, monkeypatch):
    """bf16 v2-type MLP calls and shared-coefficient reconstruction run on nn.Linear-layout twins of their operands (one
    copy per tensor, reused while the tensor is unchanged) through the product-path kernels; the input-major kernels
    (FLASHSVD_AMD_REFERENCE_LAYOUT_FAST=0) are the same arithmetic in another summation order.  Both at the 7B shapes."""
    from flashsvd_amd.kernels import _common
    dt = torch.bfloat16
    B, R, D, Hd = 8, 1536, 11008, 4096
    PUp, PGate = rnd(B, 1, R, seed=1), rnd(B, 1, R, seed=2)
    GateU, UpU = rnd(R, D, std=0.03, seed=3), rnd(R, D, std=0.03, seed=4)
    DownV, DownU, b2 = rnd(D, R, std=0.03, seed=5), rnd(R, Hd, std=0.03, seed=6), rnd(Hd, std=0.1, seed=7)
    ref = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2)
    g = [t.cuda() for t in (PUp, PGate, GateU, UpU, DownV, DownU)]
    n0 = _common.TWIN_BUILDS[0]
    fast = K.flashsvd_mlp_dual_split_triton_v2(*g, b2.cuda())
    assert _common.TWIN_BUILDS[0] == n0 + 4                         # GateU, UpU, DownV, DownU
    again = K.flashsvd_mlp_dual_split_triton_v2(*g, b2.cuda())
    assert _common.TWIN_BUILDS[0] == n0 + 4 and torch.equal(fast, again)
    monkeypatch.setenv("FLASHSVD_AMD_REFERENCE_LAYOUT_FAST", "0")
    slow = K.flashsvd_mlp_dual_split_triton_v2(*g, b2.cuda())
    monkeypatch.delenv("FLASHSVD_AMD_REFERENCE_LAYOUT_FAST")
    for got, nm in ((fast, "product-path route"), (slow, "input-major route")):
        assert_close_bf16(got, ref, nm, **tol(ref, dt))
    # an operand written in place must not be served from a stale twin
    g[5].mul_(2.0)
    doubled = K.flashsvd_mlp_dual_split_triton_v2(*g, None)
    ref2 = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, (DownU.float() * 2).to(dt))
    assert_close_bf16(doubled, ref2, "after an in-place update of DownU", **tol(ref2, dt))
    # reconstruction: coefficients as adjacent views of one packed row (the reference's split of hidden @ packed_qkv_rank)
    Bq, H, Dh, Ra = 1, 32, 128, 1024
    packed = rnd(Bq, 3 * Ra, seed=11)
    Vq, Vk, Vv = (rnd(H, Ra, Dh, std=0.03, seed=12 + i) for i in range(3))
    pg = packed.cuda()
    gq, gk, gv = pg[:, :Ra], pg[:, Ra:2 * Ra], pg[:, 2 * Ra:]
    vq, vk, vv = Vq.cuda(), Vk.cuda(), Vv.cuda()
    refq = O.reconstruct_qkv_token_shared(packed[:, :Ra], packed[:, Ra:2 * Ra], packed[:, 2 * Ra:], Vq, Vk, Vv)
    fastq = K.reconstruct_qkv_token_shared(gq, gk, gv, vq, vk, vv)
    monkeypatch.setenv("FLASHSVD_AMD_REFERENCE_LAYOUT_FAST", "0")
    slowq = K.reconstruct_qkv_token_shared(gq, gk, gv, vq, vk, vv)
    for got, nm in ((fastq, "product-path route"), (slowq, "input-major route")):
        for a, b, c in zip(got, refq, "QKV"):
            assert a.shape == b.shape and a.is_contiguous()
            assert_close_bf16(a, b, f"reconstruct {nm} {c}", **tol(b, dt))
