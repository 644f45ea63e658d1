"""GPU parity of the full-sequence low-rank RoPE attention (matrix-core rebuild of q/k/v + causal flash
attention) against the CPU oracle; bf16 within max-abs 2e-2 / max-rel 1e-2."""
import os

import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, model_from_oracle, rand_bf16

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


class _Rot:
    def __init__(self, dh, theta=10000.0):
        half = dh // 2
        self.inv_freq = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float32) / half))


def _factors(B, H, Hk, M, R, dh, shared, seed=0):
    if shared:
        pq, pk, pv = (rand_bf16(B, 1, M, R, seed=seed + i) for i in range(3))
        Pq, Pk, Pv = pq.expand(B, H, M, R), pk.expand(B, Hk, M, R), pv.expand(B, Hk, M, R)
    else:
        Pq, Pk, Pv = rand_bf16(B, H, M, R, seed=seed), rand_bf16(B, Hk, M, R, seed=seed + 1), rand_bf16(B, Hk, M, R, seed=seed + 2)
    s = R ** -0.5
    Vq, Vk, Vv = rand_bf16(H, R, dh, std=s, seed=seed + 3), rand_bf16(Hk, R, dh, std=s, seed=seed + 4), rand_bf16(Hk, R, dh, std=s, seed=seed + 5)
    return Pq, Pk, Pv, Vq, Vk, Vv


@pytest.mark.parametrize("B,H,Hk,M,R,shared", [(1, 32, 32, 512, 1024, True), (2, 4, 2, 100, 40, False), (3, 2, 2, 1, 16, True),
                                               (1, 8, 8, 333, 1664, True), (2, 4, 4, 65, 8, False)])
def test_rope_attention_module_vs_oracle(B, H, Hk, M, R, shared):
    from flashsvd_amd.kernels.flashsvdropeattn import FlashSVDRoPEAttention, QKVFactors
    dh = 128
    Pq, Pk, Pv, Vq, Vk, Vv = _factors(B, H, Hk, M, R, dh, shared)
    cos, sin = O.rope_tables(M, dh, dtype=BF16)
    ref = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin)
    mod = FlashSVDRoPEAttention(H, dh, _Rot(dh), bm=64, bn=64, br=64)
    g = [t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)]
    out = mod(QKVFactors(*g), None, torch.arange(M, device="cuda")[None])
    assert out.shape == (B, M, H, dh) and out.dtype == BF16
    assert_close_bf16(out, ref, "prefill", **bounds(ref))


@pytest.mark.parametrize("H,Hk,shared", [(8, 8, True), (8, 2, False)])
def test_rope_attention_in_head_groups_gives_the_same_bits(monkeypatch, H, Hk, shared):
    """q, K, V are rebuilt and attended one group of kv heads at a time when their temporaries would exceed the byte budget
    (FLASHSVD_AMD_PREFILL_TEMP_BYTES); a head's result does not depend on which heads share its pass.  Biases, a padding
    mask and grouped queries included; budgets that give groups of one, of three (a ragged last group) and all heads."""
    from flashsvd_amd import hip_ops
    from flashsvd_amd.kernels.rope_attn import FlashSVDRoPEAttention, QKVFactors
    B, M, R, dh = 2, 200, 64, 128
    Pq, Pk, Pv, Vq, Vk, Vv = _factors(B, H, Hk, M, R, dh, shared, seed=30)
    bq = rand_bf16(H * dh, std=0.1, seed=40)
    bk = bv = None
    if H == Hk:
        bk, bv = rand_bf16(H * dh, std=0.1, seed=41), rand_bf16(H * dh, std=0.1, seed=42)
    pad = torch.ones(B, M, dtype=torch.long)
    pad[1, :5] = 0
    mod = FlashSVDRoPEAttention(H, dh, _Rot(dh))
    g = [t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)]
    f = QKVFactors(*g, bq=bq.cuda(), bk=None if bk is None else bk.cuda(), bv=None if bv is None else bv.cuda())
    per_kv_head = (B * M * (H // Hk) + 2 * B * M) * dh * 2
    outs = {}
    for name, budget in (("all", 0), ("one", 1), ("three", 3 * per_kv_head)):
        monkeypatch.setenv("FLASHSVD_AMD_PREFILL_TEMP_BYTES", str(budget))
        want = {"all": Hk, "one": 1, "three": min(3, Hk)}[name]
        assert hip_ops.prefill_head_groups(B, M, M, H, Hk, dh) == want
        outs[name] = mod(f, pad.cuda(), torch.arange(M, device="cuda")[None]).cpu()
    assert torch.equal(outs["all"], outs["one"]) and torch.equal(outs["all"], outs["three"])
    cos, sin = O.rope_tables(M, dh, dtype=BF16)
    ref = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin, bq=bq, bk=bk, bv=bv, pad_mask=pad)
    assert_close_bf16(outs["one"], ref, "prefill in head groups", **bounds(ref))


@pytest.mark.parametrize("M", [70, 150])     # 64-query kernel / 128-query kernel with LDS-shared tiles
def test_rope_attention_masks_biases_positions(M):
    from flashsvd_amd.kernels.rope_attn import FlashSVDRoPEAttention, QKVFactors
    B, H, Hk, R, dh = 2, 4, 4, 48, 128
    Pq, Pk, Pv, Vq, Vk, Vv = _factors(B, H, Hk, M, R, dh, False, seed=10)
    bq, bk, bv = rand_bf16(H * dh, std=0.1, seed=20), rand_bf16(H * dh, std=0.1, seed=21), rand_bf16(H * dh, std=0.1, seed=22)
    # left-padded second row, per-row positions
    pad = torch.ones(B, M, dtype=torch.long)
    pad[1, :9] = 0
    pos = torch.stack([torch.arange(M), (torch.arange(M) - 9).clamp_min(0)])
    ang = pos.float()[..., None] * _Rot(dh).inv_freq
    cos, sin = torch.cos(ang).to(BF16), torch.sin(ang).to(BF16)
    ref = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin, bq=bq, bk=bk, bv=bv, pad_mask=pad)
    mod = FlashSVDRoPEAttention(H, dh, _Rot(dh))
    g = [t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)]
    out = mod(QKVFactors(*g, bq=bq.cuda(), bk=bk.cuda(), bv=bv.cuda()), pad.cuda(), pos.cuda())
    assert torch.all(out[1, :9] == 0)                     # rows whose keys are all padded give 0
    assert_close_bf16(out, ref, "pad + bias + positions", **bounds(ref))
    # additive mask that forbids a band of keys for every query
    add = torch.zeros(B, 1, M, M)
    add[:, :, :, 5:12] = float("-inf")
    add[0, :, :, 0] = -1.5
    ref2 = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos[:1].expand(B, M, dh // 2), sin[:1].expand(B, M, dh // 2), add_mask=add)
    out2 = mod(QKVFactors(*g), add.to(BF16).cuda(), pos[:1].cuda())
    assert_close_bf16(out2, ref2, "additive mask", **bounds(ref2))
    with pytest.raises(ValueError, match=r"expects Pq \[B,H,M,R\]"):
        mod(QKVFactors(g[0][0], *g[1:]), None, pos.cuda())
    with pytest.raises(ValueError, match="position_ids last dim"):
        mod(QKVFactors(*g), None, pos[:, :5].cuda())
    with pytest.raises(NotImplementedError):
        mod(QKVFactors(*[t.float() for t in g]), None, pos.cuda())


def test_expand_and_prefill_attention_primitives():
    from flashsvd_amd import hip_ops
    B, M, H, Hk, dh, R, S, start = 2, 40, 4, 2, 128, 72, 96, 13
    cos, sin = O.rope_tables(S, dh, dtype=BF16)
    p = rand_bf16(B, M, R, seed=1)
    u = rand_bf16(Hk * dh, R, std=R ** -0.5, seed=2)
    kc = torch.zeros(B, S, Hk, dh, dtype=BF16, device="cuda")
    pos0 = torch.full((B,), start, dtype=torch.int32, device="cuda")
    hip_ops.lowrank_expand_heads(p.cuda(), u.cuda(), num_heads=Hk, head_dim=dh, out=kc, cos=cos.cuda(), sin=sin.cuda(),
                                 positions=pos0, dst_by_position=True)
    ref = O.apply_rope(O.lin(p, u).reshape(B, M, Hk, dh), cos[start:start + M][None, :, None], sin[start:start + M][None, :, None])
    assert_close_bf16(kc[:, start:start + M], ref, "expand into cache rows", **bounds(ref))
    assert torch.all(kc[:, :start] == 0) and torch.all(kc[:, start + M:] == 0)
    # chunked prefill: queries at positions start.. attend over the prefix already in the cache
    kfull, vfull = rand_bf16(B, S, Hk, dh, seed=3), rand_bf16(B, S, Hk, dh, seed=4)
    q = rand_bf16(B, M, H, dh, seed=5)
    out = hip_ops.attn_prefill(q.cuda(), kfull.cuda(), vfull.cuda(), q_pos0=pos0, causal=True)
    for m in (0, 17, M - 1):
        n = start + m + 1
        refm = O.dense_decode_attn(q[:, m], kfull[:, :n], vfull[:, :n])
        assert_close_bf16(out[:, m], refm, f"row {m}", **bounds(refm))


@pytest.mark.parametrize("B,M", [(3, 520), (2, 500), (1, 300)])
def test_prefill_attention_row_tile_forms(B, M):
    """The three forms of the LDS-shared prompt attention: 128 query rows per workgroup (B = 3: enough row tile / head /
    batch triples), 64 rows with four waves (B = 2), 64 rows with a second group of waves on every other key tile (B = 1:
    no more workgroups than compute units); grouped heads, a prefix already in the cache, a ragged last tile."""
    from flashsvd_amd import hip_ops
    H, Hk, dh, S, start = 32, 8, 128, 560, 29
    kfull, vfull = rand_bf16(B, S, Hk, dh, seed=31), rand_bf16(B, S, Hk, dh, seed=32)
    q = rand_bf16(B, M, H, dh, seed=33)
    pos0 = torch.full((B,), start, dtype=torch.int32, device="cuda")
    out = hip_ops.attn_prefill(q.cuda(), kfull.cuda(), vfull.cuda(), q_pos0=pos0, causal=True)
    for m in (0, 15, 16, 63, 64, 127, 128, 299, 300, 511, 512, M - 1):
        if m >= M:
            continue
        n = start + m + 1
        refm = O.dense_decode_attn(q[:, m], kfull[:, :n], vfull[:, :n])
        assert_close_bf16(out[:, m], refm, f"row {m}", **bounds(refm))


@pytest.mark.parametrize("B,M,R", [(1, 512, 1024), (2, 130, 64), (3, 50, 192)])
def test_expand_long_prompts_tiled_kernel(B, M, R):
    """128 token rows and more with a rank that is a multiple of 64: the LDS-tiled expansion; same result as the
    oracle and as the per-wave kernel (rank 72 above takes that one)."""
    from flashsvd_amd import hip_ops
    H, dh, start = 3, 128, 7
    S = start + M + 5
    cos, sin = O.rope_tables(S, dh, dtype=BF16)
    p = rand_bf16(B, M, R, seed=1)
    u = rand_bf16(H * dh, R, std=R ** -0.5, seed=2)
    bias = rand_bf16(H * dh, std=0.1, seed=3)
    pos0 = torch.tensor([start + b for b in range(B)], dtype=torch.int32, device="cuda")
    # rotated, by position, into cache rows
    kc = torch.zeros(B, S, H, dh, dtype=BF16, device="cuda")
    hip_ops.lowrank_expand_heads(p.cuda(), u.cuda(), num_heads=H, head_dim=dh, out=kc, cos=cos.cuda(), sin=sin.cuda(),
                                 positions=pos0, dst_by_position=True)
    for b in range(B):
        s0 = start + b
        ref = O.apply_rope(O.lin(p[b], u).reshape(M, H, dh), cos[s0:s0 + M][:, None], sin[s0:s0 + M][:, None])
        assert_close_bf16(kc[b, s0:s0 + M], ref, f"rotated rows of batch {b}", **bounds(ref))
        assert torch.all(kc[b, :s0] == 0) and torch.all(kc[b, s0 + M:] == 0)
    # not rotated, with bias, by token index into a query-shaped buffer (strided coefficient rows)
    wide = torch.zeros(B, M, R + 64, dtype=BF16)
    wide[..., 64:] = p
    q = torch.zeros(B, M, H, dh, dtype=BF16, device="cuda")
    hip_ops.lowrank_expand_heads(wide.cuda()[..., 64:], u.cuda(), num_heads=H, head_dim=dh, out=q, bias=bias.cuda(), positions=pos0)
    ref = O.lin(p, u, bias).reshape(B, M, H, dh)
    assert_close_bf16(q, ref, "plain expansion with bias", **bounds(ref))


@pytest.mark.parametrize("B,M,Rq,Rk,Rv", [(1, 512, 1024, 1024, 1024), (2, 130, 128, 64, 192), (2, 40, 64, 64, 64), (1, 256, 128, 72, 64)])
def test_expand_multi_equals_separate_calls(B, M, Rq, Rk, Rv):
    """q / k / v expansions in one call: bit-identical to three separate calls, whether the call becomes one launch
    (128 rows and more, ranks multiples of 64) or falls back to one launch per expansion (short prompt, rank 72)."""
    from flashsvd_amd import hip_ops
    H, Hk, dh, start = 4, 2, 128, 5
    S = start + M + 3
    cos, sin = (t.cuda() for t in O.rope_tables(S, dh, dtype=BF16))
    packed = rand_bf16(B, M, Rq + Rk + Rv, seed=1).cuda()        # the rank coefficients as the model holds them: one row
    pq, pk, pv = packed[..., :Rq], packed[..., Rq:Rq + Rk], packed[..., Rq + Rk:]
    uq, uk, uv = (rand_bf16(h * dh, r, std=r ** -0.5, seed=s).cuda() for h, r, s in ((H, Rq, 2), (Hk, Rk, 3), (Hk, Rv, 4)))
    bq = rand_bf16(H * dh, std=0.1, seed=5).cuda()
    pos0 = torch.tensor([start + b for b in range(B)], dtype=torch.int32, device="cuda")

    def buffers():
        return (torch.zeros(B, M, H, dh, dtype=BF16, device="cuda"), torch.zeros(B, S, Hk, dh, dtype=BF16, device="cuda"),
                torch.zeros(B, S, Hk, dh, dtype=BF16, device="cuda"))

    q1, k1, v1 = buffers()
    hip_ops.lowrank_expand_heads(pq, uq, num_heads=H, head_dim=dh, out=q1, cos=cos, sin=sin, positions=pos0, bias=bq)
    hip_ops.lowrank_expand_heads(pk, uk, num_heads=Hk, head_dim=dh, out=k1, cos=cos, sin=sin, positions=pos0, dst_by_position=True)
    hip_ops.lowrank_expand_heads(pv, uv, num_heads=Hk, head_dim=dh, out=v1, positions=pos0, dst_by_position=True)
    q2, k2, v2 = buffers()
    hip_ops.lowrank_expand_heads_multi(
        [dict(p=pq, u=uq, num_heads=H, out=q2, rotate=True, bias=bq),
         dict(p=pk, u=uk, num_heads=Hk, out=k2, rotate=True, dst_by_position=True),
         dict(p=pv, u=uv, num_heads=Hk, out=v2, dst_by_position=True)],
        head_dim=dh, cos=cos, sin=sin, positions=pos0)
    assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(v1, v2)
    ref = O.lin(pv.cpu(), uv.cpu()).reshape(B, M, Hk, dh)
    for b in range(B):
        assert_close_bf16(v2[b, start + b:start + b + M], ref[b], f"v rows of batch {b}", **bounds(ref[b]))
    # two expansions, and token rows that do not match
    k3, v3 = buffers()[1:]
    hip_ops.lowrank_expand_heads_multi([dict(p=pk, u=uk, num_heads=Hk, out=k3, rotate=True, dst_by_position=True),
                                        dict(p=pv, u=uv, num_heads=Hk, out=v3, dst_by_position=True)],
                                       head_dim=dh, cos=cos, sin=sin, positions=pos0)
    assert torch.equal(k1, k3) and torch.equal(v1, v3)
    with pytest.raises(ValueError, match="same token rows"):
        hip_ops.lowrank_expand_heads_multi([dict(p=pk, u=uk, num_heads=Hk, out=k3), dict(p=pv[:, :M - 1], u=uv, num_heads=Hk, out=v3)], head_dim=dh)


def test_model_prefill_mfma_equals_decode_route():
    mw = O.make_model(d=512, n_heads=4, n_kv_heads=2, head_dim=128, ffn=1024, attn_rank=96, mlp_rank=128, n_layers=2,
                      vocab=300, dtype=BF16, seed=7, std=0.05)
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    model = model_from_oracle(mw)
    ids = torch.randint(0, 300, (2, 50), generator=torch.Generator().manual_seed(3))
    outs = {}
    for route in ("mfma", "decode"):
        os.environ["FLASHSVD_AMD_PREFILL"] = route
        try:
            cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=2, max_cache_len=64, device="cuda", dtype=BF16)
            o = model(ids.cuda(), past_key_values=cache, cache_position=torch.arange(50))
            outs[route] = (o.logits.clone(), o.hidden_states.clone(), cache.key_cache[0][:, :50].clone(), cache.value_cache[1][:, :50].clone())
        finally:
            del os.environ["FLASHSVD_AMD_PREFILL"]
    ref_logits, ref_hidden = O.model_forward(mw, ids, last_only=False, return_hidden=True)
    for route, (lg, hid, k0, v1) in outs.items():
        assert_close_bf16(hid, ref_hidden, f"{route} hidden", rel_tol=3e-2)
    assert_close_bf16(outs["mfma"][2], outs["decode"][2], "layer-0 K rows of the two routes", abs_tol=float("inf"), rel_tol=1e-2)
    assert (outs["mfma"][2] != outs["decode"][2]).float().mean() < 0.01   # same rounding points: all but a few ulp flips identical
