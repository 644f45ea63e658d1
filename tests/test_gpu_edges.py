"""Edge cases of the HIP path against the CPU oracle, through the C ABI: smallest shapes, empty and full caches, single
prompt tokens, rows one past every tile boundary.  Same tolerance as the other GPU parity tests."""
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, rand_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from flashsvd_amd import hip_ops
    return hip_ops


@pytest.mark.parametrize("B,N,K", [(1, 1, 8), (1, 3, 16), (2, 1, 4096), (3, 1, 32), (16, 17, 32), (33, 1, 64), (128, 1, 64), (129, 65, 64)])
def test_linear_smallest_shapes(ops, B, N, K):
    x, w = rand_bf16(B, K, seed=1), rand_bf16(N, K, std=0.1, seed=2)
    bias, res = rand_bf16(N, std=0.1, seed=3), rand_bf16(B, N, seed=4)
    y = ops.linear(x.cuda(), w.cuda(), bias.cuda(), residual=res.cuda())
    ref = res + O.lin(x, w, bias)
    assert_close_bf16(y, ref, f"linear {B}x{N}x{K}", **bounds(ref))


@pytest.mark.parametrize("B,D,R", [(1, 1, 8), (2, 3, 16), (3, 1, 32), (17, 2, 32), (128, 1, 64), (130, 33, 64)])
def test_swiglu_smallest_shapes(ops, B, D, R):
    p = rand_bf16(B, 2 * R, seed=1)
    gu, uu = rand_bf16(D, R, std=0.2, seed=2), rand_bf16(D, R, std=0.2, seed=3)
    h = ops.swiglu_linear(p.cuda(), gu.cuda(), uu.cuda(), up_off=R, mode=0)
    g, u = p[:, :R].float() @ gu.float().t(), p[:, R:].float() @ uu.float().t()
    ref = torch.nn.functional.silu(g.to(torch.bfloat16)) * u.to(torch.bfloat16)
    assert_close_bf16(h, ref, f"swiglu {B}x{D}x{R}", **bounds(ref))


@pytest.mark.parametrize("Dh", [64, 128])
def test_attention_over_an_empty_and_a_full_cache(ops, Dh):
    """Row 0 has no cached key (the appended token is all it attends to), row 1 fills the cache to its last slot."""
    B, H, Hk, S = 2, 4, 2, 40
    cos, sin = O.rope_tables(S, Dh, dtype=torch.bfloat16)
    q, kn, vn = rand_bf16(B, H, Dh, seed=1), rand_bf16(B, Hk, Dh, seed=2), rand_bf16(B, Hk, Dh, seed=3)
    kc, vc = rand_bf16(B, S, Hk, Dh, seed=4), rand_bf16(B, S, Hk, Dh, seed=5)
    lens = torch.tensor([0, S - 1], dtype=torch.int32)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    ref = O.flash_attn_with_kvcache(q[:, None], kc_ref, vc_ref, k=kn[:, None], v=vn[:, None], cache_seqlens=lens,
                                    rotary_cos=cos, rotary_sin=sin, causal=True)
    kcg, vcg = kc.cuda(), vc.cuda()
    for nsplit in (1, 4):
        kcg.copy_(kc); vcg.copy_(vc)
        out = ops.attn_decode_densekv(q.cuda(), kcg, vcg, lens.cuda(), k_new=kn.cuda(), v_new=vn.cuda(), cos=cos.cuda(), sin=sin.cuda(), nsplit=nsplit)
        assert_close_bf16(out, ref[:, 0], f"attention, empty / full cache, nsplit {nsplit}")
        assert_close_bf16(kcg, kc_ref, "k cache after the append")
        assert torch.equal(vcg.cpu(), vc_ref)


def test_attention_single_cached_key_is_its_value(ops):
    B, H, Dh, S = 1, 2, 128, 8
    q = rand_bf16(B, H, Dh, seed=1)
    kc, vc = rand_bf16(B, S, H, Dh, seed=2), rand_bf16(B, S, H, Dh, seed=3)
    out = ops.attn_decode_densekv(q.cuda(), kc.cuda(), vc.cuda(), torch.tensor([1], dtype=torch.int32).cuda(), nsplit=2)
    assert torch.equal(out.cpu(), vc[:, 0]), "softmax over one key has weight 1: the output is that key's value row"


@pytest.mark.parametrize("M", [2, 127, 129, 257])
def test_prompt_attention_row_counts_around_the_tile_sizes(M):
    """The fused prompt attention on row counts one off the 64- and 128-row tiles, against the oracle."""
    from flashsvd_amd.kernels.flashsvdropeattn import FlashSVDRoPEAttention, QKVFactors
    from tests.test_gpu_prefill import _Rot, _factors
    B, H, Hk, R, dh = 1, 4, 2, 72, 128
    Pq, Pk, Pv, Vq, Vk, Vv = _factors(B, H, Hk, M, R, dh, False, seed=7)
    cos, sin = O.rope_tables(M, dh, dtype=torch.bfloat16)
    ref = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin)
    mod = FlashSVDRoPEAttention(H, dh, _Rot(dh), bm=64, bn=64, br=64)
    out = mod(QKVFactors(*[t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)]), None, torch.arange(M, device="cuda")[None])
    assert_close_bf16(out, ref, f"prompt attention, {M} tokens", **bounds(ref))


def test_rmsnorm_rows_and_widths(ops):
    for B, K in ((1, 8), (3, 24), (5, 4096), (130, 64)):
        x, w = rand_bf16(B, K, seed=1), rand_bf16(K, seed=2) * 0.1 + 1
        y = ops.rmsnorm(x.cuda(), w.cuda(), 1e-6)
        assert_close_bf16(y, O.rms_norm(x, w, 1e-6), f"rmsnorm {B}x{K}")
