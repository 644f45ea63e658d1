"""GPU parity of the projection / attention primitives against the CPU oracle, called through
the C ABI (flashsvd_amd.hip_ops -> libflashsvd_hip.so).  Tolerance: bf16 outputs within
max-abs 2e-2 and max-rel 1e-2 of the oracle on the same seeded inputs."""
import math
import os

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


@pytest.mark.parametrize("B,N,K", [(1, 3072, 4096), (1, 1536, 11008), (1, 4096, 1536), (1, 4096, 1024),
                                   (2, 257, 512), (3, 64, 264), (5, 33, 1492), (1, 7, 100), (8, 128, 4096)])
def test_linear_plain(ops, B, N, K):
    x, w = rand_bf16(B, K, seed=1), rand_bf16(N, K, std=0.02, seed=2)
    y = ops.linear(x.cuda(), w.cuda())
    assert_close_bf16(y, O.lin(x, w), f"linear {B}x{N}x{K}")


@pytest.mark.parametrize("cfg", [1, 2, 4, 0x101, 0x102])
def test_linear_tilings_agree(ops, cfg):
    x, w = rand_bf16(1, 2048, seed=3), rand_bf16(515, 2048, std=0.02, seed=4)
    y = ops.linear(x.cuda(), w.cuda(), cfg=cfg)
    assert_close_bf16(y, O.lin(x, w), f"cfg {cfg:#x}")


def test_linear_norm_bias_residual(ops):
    B, N, K = 2, 512, 4096
    x, w = rand_bf16(B, K, seed=1), rand_bf16(N, K, std=0.02, seed=2)
    nw, bias, res = rand_bf16(K, seed=3) * 0.1 + 1, rand_bf16(N, std=0.1, seed=4), rand_bf16(B, N, seed=5)
    y = ops.linear(x.cuda(), w.cuda(), bias.cuda(), norm_weight=nw.cuda(), eps=1e-6, residual=res.cuda())
    ref = res + O.lin(O.rms_norm(x, nw, 1e-6), w, bias)
    assert_close_bf16(y, ref, "norm+bias+residual")


def test_linear_strided_rows(ops):
    # x and out are row slices of wider buffers; weight is a row slice of a packed matrix
    xw = rand_bf16(2, 3000, seed=1).cuda()
    W = rand_bf16(300, 1024, std=0.02, seed=2).cuda()
    outw = torch.zeros(2, 500, dtype=torch.bfloat16, device="cuda")
    y = ops.linear(xw[:, 8:8 + 1024], W[100:228])
    assert_close_bf16(y, O.lin(xw[:, 8:1032].cpu(), W[100:228].cpu()), "strided")


def test_rmsnorm(ops):
    x, w = rand_bf16(3, 4096, seed=1), rand_bf16(4096, seed=2) * 0.1 + 1
    assert_close_bf16(ops.rmsnorm(x.cuda(), w.cuda(), 1e-6), O.rms_norm(x, w, 1e-6), "rmsnorm")


@pytest.mark.parametrize("B,D,R,mode", [(1, 11008, 1536, 0), (1, 11008, 1536, 1), (3, 1376, 256, 0), (2, 100, 52, 1)])
def test_swiglu_linear(ops, B, D, R, mode):
    p = rand_bf16(B, 2 * R, seed=1)
    gu, uu = rand_bf16(D, R, std=0.05, seed=2), rand_bf16(D, R, std=0.05, seed=3)
    h = ops.swiglu_linear(p.cuda(), gu.cuda(), uu.cuda(), up_off=R, mode=mode)
    g, u = p[:, :R].float() @ gu.float().t(), p[:, R:].float() @ uu.float().t()
    if mode == 0:
        ref = torch.nn.functional.silu(g.to(torch.bfloat16)) * u.to(torch.bfloat16)
    else:
        ref = ((g * torch.sigmoid(g)) * u).to(torch.bfloat16)
    assert_close_bf16(h, ref, f"swiglu mode {mode}")


@pytest.mark.parametrize("B,H,Hk,Dh,Rq,Rk,Rv", [(1, 32, 32, 128, 1024, 1024, 1024), (2, 8, 2, 64, 128, 96, 72), (3, 4, 4, 64, 52, 52, 52)])
def test_qkv_rope_append(ops, B, H, Hk, Dh, Rq, Rk, Rv):
    S = 40
    p = rand_bf16(B, Rq + Rk + Rv, seed=1)
    qu, ku, vu = rand_bf16(H * Dh, Rq, std=0.05, seed=2), rand_bf16(Hk * Dh, Rk, std=0.05, seed=3), rand_bf16(Hk * Dh, Rv, std=0.05, seed=4)
    cos, sin = O.rope_tables(S, Dh, dtype=torch.bfloat16)
    pos = torch.tensor([(7 * b + 5) % S for b in range(B)], dtype=torch.int32)
    kc = torch.zeros(B, S, Hk, Dh, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros_like(kc)
    q = ops.qkv_rope_append(p.cuda(), qu.cuda(), ku.cuda(), vu.cuda(), cos.cuda(), sin.cuda(), pos.cuda(), kc, vc,
                            num_heads=H, num_kv_heads=Hk, head_dim=Dh)
    pq, pk, pv = p[:, :Rq], p[:, Rq:Rq + Rk], p[:, Rq + Rk:]
    for b in range(B):
        c, s = cos[pos[b]], sin[pos[b]]
        qr = O.apply_rope(O.lin(pq[b:b + 1], qu).reshape(H, Dh), c, s)
        kr = O.apply_rope(O.lin(pk[b:b + 1], ku).reshape(Hk, Dh), c, s)
        vr = O.lin(pv[b:b + 1], vu).reshape(Hk, Dh)
        assert_close_bf16(q[b], qr, "q")
        assert_close_bf16(kc[b, pos[b]], kr, "k row")
        assert_close_bf16(vc[b, pos[b]], vr, "v row")
    # nothing else in the caches was touched
    mask = torch.ones(B, S, dtype=torch.bool)
    for b in range(B):
        mask[b, pos[b]] = False
    assert torch.all(kc.cpu()[mask] == 0) and torch.all(vc.cpu()[mask] == 0)


@pytest.mark.parametrize("B,H,Hk,Dh,L,S,nsplit", [(1, 32, 32, 128, 512, 560, 8), (1, 32, 32, 128, 513, 560, 16),
                                                 (2, 8, 2, 64, 37, 64, 3), (3, 4, 4, 128, 1, 16, 2),
                                                 (1, 32, 8, 128, 4096, 4100, 16), (2, 4, 4, 64, 100, 128, 1),
                                                 # grouped-query caches with the chip full: four / two query heads per workgroup
                                                 (16, 32, 8, 128, 300, 320, 4), (16, 32, 16, 128, 130, 160, 2), (64, 32, 8, 128, 70, 96, 1),
                                                 (32, 16, 4, 128, 260, 300, 5)])
def test_attn_decode_densekv_prerotated(ops, B, H, Hk, Dh, L, S, nsplit):
    q = rand_bf16(B, H, Dh, seed=1)
    kc, vc = rand_bf16(B, S, Hk, Dh, seed=2), rand_bf16(B, S, Hk, Dh, seed=3)
    lens = torch.tensor([max(1, L - 3 * b) for b in range(B)], dtype=torch.int32)
    out = ops.attn_decode_densekv(q.cuda(), kc.cuda(), vc.cuda(), lens.cuda(), nsplit=nsplit)
    for b in range(B):
        n = int(lens[b])
        ref = O.dense_decode_attn(q[b:b + 1], kc[b:b + 1, :n], vc[b:b + 1, :n])
        assert_close_bf16(out[b:b + 1], ref, f"attn b={b}")


def test_attn_decode_two_calls_same_workspace(ops):
    # counters must return to zero so that a second call (smaller) is still right
    B, H, Hk, Dh, S = 1, 8, 8, 128, 300
    ws = ops.attn_workspace(B, H, Dh, 8, "cuda")
    q = rand_bf16(B, H, Dh, seed=1)
    kc, vc = rand_bf16(B, S, Hk, Dh, seed=2), rand_bf16(B, S, Hk, Dh, seed=3)
    for n in (290, 17):
        lens = torch.tensor([n], dtype=torch.int32)
        out = ops.attn_decode_densekv(q.cuda(), kc.cuda(), vc.cuda(), lens.cuda(), nsplit=8, workspace=ws)
        assert_close_bf16(out, O.dense_decode_attn(q, kc[:, :n], vc[:, :n]), f"n={n}")


def test_attn_decode_flash_attn_kvcache_contract(ops):
    B, H, Hk, Dh, S = 2, 8, 4, 128, 96
    cos, sin = O.rope_tables(S, Dh, dtype=torch.bfloat16)
    q, kn, vn = rand_bf16(B, H, Dh, seed=1), rand_bf16(B, Hk, Dh, seed=2), rand_bf16(B, Hk, Dh, seed=3)
    kc, vc = rand_bf16(B, S, Hk, Dh, seed=4), rand_bf16(B, S, Hk, Dh, seed=5)
    lens = torch.tensor([70, 33], dtype=torch.int32)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    ref = O.flash_attn_with_kvcache(q[:, None], kc_ref, vc_ref, k=kn[:, None], v=vn[:, None], cache_seqlens=lens,
                                    rotary_cos=cos, rotary_sin=sin, causal=True)
    kcg, vcg = kc.cuda(), vc.cuda()
    out = ops.attn_decode_densekv(q.cuda(), kcg, vcg, lens.cuda(), k_new=kn.cuda(), v_new=vn.cuda(), cos=cos.cuda(), sin=sin.cuda(), nsplit=4)
    assert_close_bf16(out, ref[:, 0], "fa2 contract out")
    assert_close_bf16(kcg, kc_ref, "k cache after append")
    assert torch.equal(vcg.cpu(), vc_ref)


def test_errors_are_python_exceptions(ops):
    x, w = rand_bf16(1, 64).cuda(), rand_bf16(8, 32).cuda()
    with pytest.raises(ValueError):
        ops.linear(x, w)
    with pytest.raises(ValueError):
        ops.linear(x.float(), rand_bf16(8, 64).cuda())
    with pytest.raises(ValueError):
        ops.linear(x.cpu(), rand_bf16(8, 64).cuda())
    from flashsvd_amd._lib import FlashSVDHipError
    q = rand_bf16(1, 2, 32).cuda()  # head_dim 32 unsupported
    kc = rand_bf16(1, 8, 2, 32).cuda()
    with pytest.raises(FlashSVDHipError):
        ops.attn_decode_densekv(q, kc, kc.clone(), torch.tensor([4], dtype=torch.int32).cuda(), nsplit=1)


# ---- three rows and more: the matrix-core path (csrc/mfma_gemv.hip) behind the same entry points
@pytest.mark.parametrize("B,N,K", [(3, 512, 4096), (4, 1536, 11008), (5, 48, 1024), (8, 3072, 4096), (16, 1536, 11008), (17, 100, 2048), (32, 4096, 1536),
                                   (64, 256, 512), (70, 33, 256), (8, 40, 96)])
def test_linear_batched_matrix_cores(ops, B, N, K):
    x, w = rand_bf16(B, K, seed=1), rand_bf16(N, K, std=0.02, seed=2)
    bias, res = rand_bf16(N, std=0.1, seed=4), rand_bf16(B, N, seed=5)
    y = ops.linear(x.cuda(), w.cuda(), bias.cuda(), residual=res.cuda())
    assert_close_bf16(y, res + O.lin(x, w, bias), f"batched linear {B}x{N}x{K}")
    # the vector kernels (explicit tiling) give the same rounding points
    y_vec = ops.linear(x.cuda(), w.cuda(), bias.cuda(), residual=res.cuda(), cfg=1)
    assert_close_bf16(y, y_vec.cpu(), "matrix-core vs vector path")


def test_linear_batched_with_norm(ops):
    B, N, K = 8, 512, 4096
    x, w = rand_bf16(B, K, seed=1), rand_bf16(N, K, std=0.02, seed=2)
    nw = rand_bf16(K, seed=3) * 0.1 + 1
    y = ops.linear(x.cuda(), w.cuda(), norm_weight=nw.cuda(), eps=1e-6)
    assert_close_bf16(y, O.lin(O.rms_norm(x, nw, 1e-6), w), "batched norm + linear")


@pytest.mark.parametrize("B,D,R,mode", [(3, 11008, 1536, 0), (4, 1376, 256, 1), (8, 11008, 1536, 0), (32, 1376, 256, 1), (5, 100, 64, 0), (33, 64, 96, 1), (32, 11008, 1536, 0),
                                        (100, 1376, 256, 1), (20, 200, 192, 0)])
def test_swiglu_batched_matrix_cores(ops, B, D, R, mode):
    p = rand_bf16(B, 2 * R, seed=1)
    gu, uu = rand_bf16(D, R, std=0.05, seed=2), rand_bf16(D, R, std=0.05, seed=3)
    h = ops.swiglu_linear(p.cuda(), gu.cuda(), uu.cuda(), up_off=R, mode=mode)
    g, u = p[:, :R].float() @ gu.float().t(), p[:, R:].float() @ uu.float().t()
    if mode == 0:
        ref = torch.nn.functional.silu(g.to(torch.bfloat16)) * u.to(torch.bfloat16)
    else:
        ref = ((g * torch.sigmoid(g)) * u).to(torch.bfloat16)
    assert_close_bf16(h, ref, f"batched swiglu mode {mode}", **bounds(ref))


# ---- 8..32 rows of a wide matrix (two 16-row tiles per compute unit and more): one workgroup per compute unit walks its
#      tiles with the activation fragments in registers (mfma_resident_kernel); one to six chunks of K per wave, ragged N,
#      bias and residual, both SwiGLU rounding modes
@pytest.mark.parametrize("B,N,K", [(8, 12288, 1024), (16, 8200, 2048), (32, 8200, 4096), (20, 8192, 6144), (9, 32000, 4096)])
def test_linear_wide_matrix_resident_form(ops, B, N, K):
    x, w = rand_bf16(B, K, seed=1), rand_bf16(N, K, std=0.02, seed=2)
    bias, res = rand_bf16(N, std=0.1, seed=4), rand_bf16(B, N, seed=5)
    y = ops.linear(x.cuda(), w.cuda(), bias.cuda(), residual=res.cuda())
    assert_close_bf16(y, res + O.lin(x, w, bias), f"resident linear {B}x{N}x{K}")
    y2 = ops.linear(x.cuda(), w.cuda())
    assert_close_bf16(y2, O.lin(x, w), f"resident linear {B}x{N}x{K}, no epilogue terms")
    assert torch.equal(y2, ops.linear(x.cuda(), w.cuda())), "repeat differs"


@pytest.mark.parametrize("B,D,R,mode", [(16, 8200, 2432, 0), (32, 11008, 2432, 1), (8, 8200, 512, 1), (24, 14336, 2048, 0)])
def test_swiglu_wide_matrix_resident_form(ops, B, D, R, mode):
    p = rand_bf16(B, 2 * R, seed=1)
    gu, uu = rand_bf16(D, R, std=0.05, seed=2), rand_bf16(D, R, std=0.05, seed=3)
    h = ops.swiglu_linear(p.cuda(), gu.cuda(), uu.cuda(), up_off=R, mode=mode)
    g, u = p[:, :R].float() @ gu.float().t(), p[:, R:].float() @ uu.float().t()
    if mode == 0:
        ref = torch.nn.functional.silu(g.to(torch.bfloat16)) * u.to(torch.bfloat16)
    else:
        ref = ((g * torch.sigmoid(g)) * u).to(torch.bfloat16)
    assert_close_bf16(h, ref, f"resident swiglu mode {mode}", **bounds(ref))
    assert torch.equal(h, ops.swiglu_linear(p.cuda(), gu.cuda(), uu.cuda(), up_off=R, mode=mode)), "repeat differs"


# ---- 128 rows and more (prefill): the tiled matrix-core kernel (csrc/mfma_gemm.hip) behind the same entry points
#      (shapes chosen to reach every tile form: 64 x 64 in K steps of 64 / 128, 128 x 64 and 128 x 128 with four and with
#      eight waves, 128 x 256 from 2048 big tiles on, loads through registers and straight into LDS, ragged edges in rows
#      and columns)
@pytest.mark.parametrize("B,N,K", [(512, 3072, 4096), (128, 128, 64), (200, 1000, 1536), (129, 130, 192), (384, 1536, 11008),
                                   (1024, 64, 1024), (500, 3050, 1152), (1000, 3000, 1088), (1024, 3072, 1024), (2048, 4096, 256),
                                   (2040, 2900, 192), (1150, 4090, 320), (4096, 8192, 64), (4100, 8200, 96)])
def test_linear_prefill_rows_tiled_kernel(ops, B, N, K):
    x, w = rand_bf16(B, K, seed=1), rand_bf16(N, K, std=0.02, seed=2)
    bias, res = rand_bf16(N, std=0.1, seed=4), rand_bf16(B, N, seed=5)
    y = ops.linear(x.cuda(), w.cuda(), bias.cuda(), residual=res.cuda())
    ref = res + O.lin(x, w, bias)
    assert_close_bf16(y, ref, f"tiled linear {B}x{N}x{K}", **bounds(ref))
    y_plain = ops.linear(x.cuda(), w.cuda())
    ref = O.lin(x, w)
    assert_close_bf16(y_plain, ref, f"tiled linear, no epilogue {B}x{N}x{K}", **bounds(ref))
    # strided operands: x a column slice, y a column slice of wider buffers
    xw = torch.zeros(B, K + 64, dtype=torch.bfloat16)
    xw[:, 64:] = x
    out = torch.zeros(B, N + 8, dtype=torch.bfloat16, device="cuda")
    ops.linear(xw.cuda()[:, 64:], w.cuda(), out=out[:, 8:])
    assert torch.equal(out[:, 8:].cpu(), y_plain.cpu()) and float(out[:, :8].abs().max()) == 0.0


@pytest.mark.parametrize("B,D,R,mode", [(512, 11008, 1536, 0), (130, 200, 64, 1), (256, 1376, 256, 1)])
def test_swiglu_prefill_rows_tiled_kernel(ops, B, D, R, mode):
    p = rand_bf16(B, 2 * R, seed=1)
    gu, uu = rand_bf16(D, R, std=0.05, seed=2), rand_bf16(D, R, std=0.05, seed=3)
    h = ops.swiglu_linear(p.cuda(), gu.cuda(), uu.cuda(), up_off=R, mode=mode)
    g, u = p[:, :R].float() @ gu.float().t(), p[:, R:].float() @ uu.float().t()
    if mode == 0:
        ref = torch.nn.functional.silu(g.to(torch.bfloat16)) * u.to(torch.bfloat16)
    else:
        ref = ((g * torch.sigmoid(g)) * u).to(torch.bfloat16)
    assert_close_bf16(h, ref, f"tiled swiglu mode {mode}", **bounds(ref))


# ---- 3..32 rows: weights streamed through a wave's own LDS ring (its load counter is the only synchronisation)
@pytest.mark.parametrize("B", [3, 8, 16, 17, 32])
def test_small_batch_streaming_projections_repeat_bit_identically(ops, B):
    """Shapes of the 7B MLP and an attention projection; every call of 20 gives the same bits (a chunk read before it
    has landed would show as a difference between calls) and they match the oracle."""
    d, R, D = 4096, 1536, 11008
    x, p, h = rand_bf16(B, d, seed=1).cuda(), rand_bf16(B, 2 * R, seed=2).cuda(), rand_bf16(B, D, seed=3).cuda()
    w_rank = rand_bf16(2 * R, d, std=0.02, seed=4).cuda()
    gu, uu = rand_bf16(D, R, std=0.03, seed=5).cuda(), rand_bf16(D, R, std=0.03, seed=6).cuda()
    w_down = rand_bf16(d, R, std=0.03, seed=7).cuda()
    w_long = rand_bf16(1000, D - 0, std=0.01, seed=8).cuda()          # long K, ragged last weight tile
    res = rand_bf16(B, d, seed=9).cuda()
    os.environ["FLASHSVD_AMD_SPLITK"] = "0"                          # keep the narrow matrix on this kernel too
    ops.release_split_workspace(x.device)
    try:
        calls = {
            "rank": lambda: ops.linear(x, w_rank),
            "pair": lambda: ops.swiglu_linear(p, gu, uu, up_off=R, mode=0),
            "down_u": lambda: ops.linear(p[:, :R], w_down, residual=res),
            "long": lambda: ops.linear(h, w_long),
        }
        first = {k: f() for k, f in calls.items()}
        for _ in range(20):
            for k, f in calls.items():
                assert torch.equal(f(), first[k]), k
    finally:
        del os.environ["FLASHSVD_AMD_SPLITK"]
        assert ops.ensure_split_workspace(x.device)
    ref = O.lin(x.cpu(), w_rank.cpu())
    assert_close_bf16(first["rank"], ref, "rank projection", **bounds(ref))
    g, u = p.cpu()[:, :R].float() @ gu.cpu().float().t(), p.cpu()[:, R:].float() @ uu.cpu().float().t()
    ref = torch.nn.functional.silu(g.to(torch.bfloat16)) * u.to(torch.bfloat16)
    assert_close_bf16(first["pair"], ref, "pair", **bounds(ref))
    ref = res.cpu() + O.lin(p.cpu()[:, :R], w_down.cpu())
    assert_close_bf16(first["down_u"], ref, "down_u", **bounds(ref))
    ref = O.lin(h.cpu(), w_long.cpu())
    assert_close_bf16(first["long"], ref, "long K", **bounds(ref))


# ---- K split over workgroups (registered scratch): same entry points, 17..127 rows, and 3..16 rows of a matrix with
#      fewer than 128 sixteen-row tiles, and prompt rows of projections with few 64 x 64 tiles or a very long K
@pytest.mark.parametrize("B,N,K", [(17, 1536, 11008), (32, 1024, 4096), (100, 200, 1536), (127, 4096, 1536), (64, 3072, 4096),
                                   (8, 1536, 11008), (3, 200, 1536), (16, 2032, 4096),
                                   (128, 1024, 4096), (300, 1536, 11008), (512, 1000, 4096), (1024, 1536, 11008)])
def test_linear_k_split_matches_unsplit_and_repeats(ops, B, N, K):
    x, w = rand_bf16(B, K, seed=1).cuda(), rand_bf16(N, K, std=0.02, seed=2).cuda()
    bias, res = rand_bf16(N, std=0.1, seed=4).cuda(), rand_bf16(B, N, seed=5).cuda()
    dev = x.device
    assert ops.ensure_split_workspace(dev)
    y1 = ops.linear(x, w, bias, residual=res)
    y2 = ops.linear(x, w, bias, residual=res)           # arrival counters are back at zero; partial sums in a fixed order
    assert torch.equal(y1, y2)
    ref = res.cpu() + O.lin(x.cpu(), w.cpu(), bias.cpu())
    assert_close_bf16(y1, ref, f"k-split linear {B}x{N}x{K}", **bounds(ref))
    os.environ["FLASHSVD_AMD_SPLITK"] = "0"             # keeps the wrapper from registering again
    ops.release_split_workspace(dev)
    try:
        y0 = ops.linear(x, w, bias, residual=res)
        assert_close_bf16(y0, ref, f"unsplit linear {B}x{N}x{K}", **bounds(ref))
    finally:
        del os.environ["FLASHSVD_AMD_SPLITK"]
        assert ops.ensure_split_workspace(dev)


def test_set_workspace_rejects_bad_buffers(ops, lib):
    buf = torch.empty(2 << 20, dtype=torch.uint8, device="cuda")
    assert lib.fsvd_set_workspace(buf.data_ptr() + 16, 1 << 20, None) != 0
    assert b"aligned" in lib.fsvd_last_error()
    assert lib.fsvd_set_workspace(buf.data_ptr(), 4096, None) != 0
    assert b"too small" in lib.fsvd_last_error()
    # the registered scratch of the wrapper is untouched by the refused calls
    x, w = rand_bf16(8, 1024, seed=1).cuda(), rand_bf16(64, 1024, std=0.02, seed=2).cuda()
    assert_close_bf16(ops.linear(x, w), O.lin(x.cpu(), w.cpu()), "after refused registrations")
