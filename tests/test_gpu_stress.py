"""The stress configuration AT ITS SIZE: 7B-shaped model at parameter ratio ~0.8 (attention rank 1664),
decode at batch 16 over a 4096-token rank-space cache, prefill at batch 8 x 2048 tokens.

The GPU kernels run the full shape; the CPU oracle checks a sample of (batch row, head) pairs — a pair is a few
GFLOP on the host, the whole shape would be 0.9 TFLOP — within the decode tolerance (max-abs 2e-2 / max-rel 1e-2;
the absolute bound becomes two bf16 ulps where max|ref| >= 2).  Semantics: benchmark/attn/decode_compare.py:675-750
(streaming rank-space decode) with its own cross-check against dense attention on the rebuilt cache (:2238-2250),
and kernels/attn/prefill/rope_sdpa.py:67-248 for the prompt pass."""
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, rand_bf16

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
H, DH, R = 32, 128, 1664


def test_rank_decode_batch16_ctx4096_rank1664_sampled_pairs():
    from flashsvd_amd.kernels import rank_decode as RD
    B, L, S = 16, 4096, 4104
    cos, sin = O.rope_tables(S, DH, dtype=BF16)
    q = rand_bf16(B, H, DH, seed=1)
    Pk, Pv = rand_bf16(B, S, R, seed=2), rand_bf16(B, S, R, seed=3)
    ku, vu = rand_bf16(H * DH, R, std=R ** -0.5, seed=4), rand_bf16(H * DH, R, std=R ** -0.5, seed=5)   # nn.Linear layout
    Vk, Vv = ku.reshape(H, DH, R).transpose(1, 2), vu.reshape(H, DH, R).transpose(1, 2)                   # [H, R, Dh]
    # ragged: full context in most rows, a few shorter ones (one ends inside a 16-key tile)
    lens = torch.full((B,), L, dtype=torch.int32)
    lens[3], lens[5], lens[12] = 4001, 2049, 777
    g = [t.cuda() for t in (q, Pk, Pv, ku, vu, cos, sin, lens)]
    print("launch rank_decode B=16 ctx=4096 R=1664", flush=True)
    out = RD.rank_decode(*g, num_kv_heads=H)
    torch.cuda.synchronize()
    again = RD.rank_decode(*g, num_kv_heads=H)
    assert torch.equal(out, again), "two calls on the same inputs differ"
    out = out.cpu()
    assert torch.isfinite(out.float()).all()
    for b, h in ((0, 0), (0, 31), (3, 7), (5, 17), (12, 30), (15, 13), (15, 31)):
        n = int(lens[b])
        ref = O.rank_decode_attn(q[b:b + 1, h:h + 1], Pk[b:b + 1, :n], Pv[b:b + 1, :n], Vk[h:h + 1], Vv[h:h + 1], cos[:n], sin[:n])
        assert_close_bf16(out[b:b + 1, h:h + 1], ref, f"row {b} head {h} ({n} keys)", **bounds(ref))
    # the reference's own check: dense attention over the rebuilt, rotated cache
    b, h, n = 5, 17, int(lens[5])
    K = O.apply_rope_fp32(Pk[b, :n].float() @ Vk[h].float(), cos[:n], sin[:n])
    V = Pv[b, :n].float() @ Vv[h].float()
    ref = O.dense_decode_attn(q[b:b + 1, h:h + 1].float(), K[None, :, None], V[None, :, None])
    assert_close_bf16(out[b:b + 1, h:h + 1], ref, "vs dense attention on the rebuilt cache", **bounds(ref))


def test_prefill_batch8_x2048_rank1664_sampled_pairs():
    from flashsvd_amd.kernels.flashsvdropeattn import FlashSVDRoPEAttention, QKVFactors
    B, M = 8, 2048
    pq, pk, pv = (rand_bf16(B, 1, M, R, seed=10 + i) for i in range(3))     # shared-rank coefficients, one row per token
    s = R ** -0.5
    Vq, Vk, Vv = (rand_bf16(H, R, DH, std=s, seed=13 + i) for i in range(3))
    cos, sin = O.rope_tables(M, DH, dtype=BF16)

    class Rot:
        inv_freq = 1.0 / (10000.0 ** (torch.arange(0, DH // 2, dtype=torch.float32) / (DH // 2)))

    mod = FlashSVDRoPEAttention(H, DH, Rot())
    f = QKVFactors(pq.cuda().expand(B, H, M, R), pk.cuda().expand(B, H, M, R), pv.cuda().expand(B, H, M, R),
                   Vq.cuda(), Vk.cuda(), Vv.cuda())
    print("launch prefill 8 x 2048 R=1664", flush=True)
    out = mod(f, None, torch.arange(M, device="cuda")[None])
    assert out.shape == (B, M, H, DH) and out.dtype == BF16
    out = out.cpu()
    assert torch.isfinite(out.float()).all()
    for b, h in ((0, 0), (3, 19), (7, 31)):
        ref = O.rope_sdpa_prefill(pq[b:b + 1], pk[b:b + 1], pv[b:b + 1], Vq[h:h + 1], Vk[h:h + 1], Vv[h:h + 1], cos, sin)   # [1, M, 1, dh]
        assert_close_bf16(out[b:b + 1, :, h:h + 1], ref, f"batch {b} head {h}, all {M} rows", **bounds(ref))
