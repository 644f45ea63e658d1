"""Pins for the CPU oracle: each check is independent of the oracle's own formula
(float64 brute force, a library routine, or a mathematical invariant), chosen so that a
dropped term, wrong sign/index or transposed operand fails it."""
import math

import numpy as np
import pytest
import torch

from oracle import flashsvd_oracle as O

torch.manual_seed(1234)


def _rand(*shape, dtype=torch.float32, scale=1.0, seed=None):
    g = torch.Generator().manual_seed(seed if seed is not None else int(np.prod(shape)) % 9973)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ---------------------------------------------------------------- linear pair
def test_lin_matches_float64_loops():
    x, w = _rand(3, 7), _rand(5, 7)
    ref = np.zeros((3, 5))
    for i in range(3):
        for o in range(5):
            for k in range(7):
                ref[i, o] += float(x[i, k]) * float(w[o, k])
    assert np.allclose(O.lin(x, w).numpy(), ref, atol=1e-6)


def test_lowrank_pair_full_rank_is_dense_linear():
    d = 16
    q, _ = torch.linalg.qr(_rand(d, d))
    W = _rand(24, d)
    # v = Q^T (orthonormal, [R=d, in]), u = W Q -> u v = W
    y = O.lowrank_pair(_rand(4, d, seed=5), q.t().contiguous(), (W @ q).contiguous())
    assert torch.allclose(y, torch.nn.functional.linear(_rand(4, d, seed=5), W), atol=1e-5)


@pytest.mark.parametrize("dt,half_ulp", [(torch.bfloat16, 2 ** -8), (torch.float16, 2 ** -11)], ids=["bf16", "fp16"])
def test_lin_16bit_rounds_once_from_fp32(dt, half_ulp):
    x, w = _rand(2, 64, dtype=dt), _rand(8, 64, dtype=dt)
    exact = (x.double() @ w.double().t())
    y = O.lin(x, w)
    assert y.dtype == dt
    # one rounding of an (almost) exact sum to the 16-bit type: error <= 1/2 ulp (unit roundoff 2^-8 bf16, 2^-11 fp16) + fp32 noise;
    # a second rounding on the way (e.g. through the other 16-bit type) would double it
    assert torch.all((y.double() - exact).abs() <= exact.abs() * half_ulp * 1.02 + 1e-6)
    assert torch.equal(y, (x.float() @ w.float().t()).to(dt))


# ---------------------------------------------------------------- rmsnorm
def test_rms_norm_matches_transformers():
    from transformers.models.llama.modeling_llama import LlamaRMSNorm
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        n = LlamaRMSNorm(32, eps=1e-6).to(dt)
        with torch.no_grad():
            n.weight.copy_(_rand(32, seed=3).to(dt))
        x = _rand(2, 3, 32, dtype=dt, seed=4)
        assert torch.equal(O.rms_norm(x, n.weight.detach(), 1e-6), n(x).detach())


# ---------------------------------------------------------------- rope
def test_rope_tables_closed_form():
    cos, sin = O.rope_tables(9, 8, 10000.0)
    for p in (0, 1, 8):
        for i in range(4):
            a = p * 10000.0 ** (-i / 4)
            assert abs(float(cos[p, i]) - math.cos(a)) < 1e-5
            assert abs(float(sin[p, i]) - math.sin(a)) < 1e-5
    assert torch.all(cos[0] == 1) and torch.all(sin[0] == 0)


def test_rope_invariants():
    Dh = 16
    cos, sin = O.rope_tables(40, Dh)
    q, k = _rand(Dh, seed=1), _rand(Dh, seed=2)
    # position 0 is the identity
    assert torch.equal(O.apply_rope(q, cos[0], sin[0]), q)
    # norm preserved per (i, i+half) pair
    r = O.apply_rope(q, cos[17], sin[17])
    assert torch.allclose(r[:8] ** 2 + r[8:] ** 2, q[:8] ** 2 + q[8:] ** 2, atol=1e-5)
    # <rope(q,m), rope(k,n)> depends only on n-m
    d1 = O.apply_rope(q, cos[3], sin[3]) @ O.apply_rope(k, cos[10], sin[10])
    d2 = O.apply_rope(q, cos[23], sin[23]) @ O.apply_rope(k, cos[30], sin[30])
    assert abs(float(d1 - d2)) < 1e-4
    # and differs for another offset (a sign error in sin keeps norms but breaks this)
    d3 = O.apply_rope(q, cos[3], sin[3]) @ O.apply_rope(k, cos[11], sin[11])
    assert abs(float(d1 - d3)) > 1e-4


def test_rope_matches_transformers_apply_rotary():
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    Dh, T = 16, 6
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        cos_h, sin_h = O.rope_tables(T, Dh, dtype=dt)
        cos = torch.cat([cos_h, cos_h], -1)[None]
        sin = torch.cat([sin_h, sin_h], -1)[None]
        q = _rand(1, 2, T, Dh, dtype=dt, seed=7)  # [B,H,T,Dh]
        k = _rand(1, 2, T, Dh, dtype=dt, seed=8)
        qe, ke = apply_rotary_pos_emb(q, k, cos, sin)
        mine = O.apply_rope(q, cos_h[None, None], sin_h[None, None])
        assert torch.allclose(mine.float(), qe.float(), atol={torch.float32: 0, torch.bfloat16: 2 ** -7 * 4, torch.float16: 2 ** -10 * 4}[dt])
        if dt == torch.float32:
            assert torch.allclose(O.apply_rope_fp32(k, cos_h[None, None], sin_h[None, None]), ke, atol=1e-6)


# ---------------------------------------------------------------- reconstruct
def test_reconstruct_variants_agree_and_match_flat_gemm():
    B, H, Hk, R, Dh = 2, 4, 2, 24, 8
    Pq, Pk, Pv = _rand(B, R, seed=1), _rand(B, R, seed=2), _rand(B, R, seed=3)
    Vq, Vk, Vv = _rand(H, R, Dh, seed=4), _rand(Hk, R, Dh, seed=5), _rand(Hk, R, Dh, seed=6)
    bq, bk, bv = _rand(H, Dh, seed=7), _rand(Hk, Dh, seed=8), _rand(Hk, Dh, seed=9)
    Qs, Ks, Vs = O.reconstruct_qkv_token_shared(Pq, Pk, Pv, Vq, Vk, Vv, bq, bk, bv)
    # brute force
    ref = np.zeros((B, H, Dh))
    for b in range(B):
        for h in range(H):
            for d in range(Dh):
                ref[b, h, d] = sum(float(Pq[b, r]) * float(Vq[h, r, d]) for r in range(R)) + float(bq[h, d])
    assert np.allclose(Qs.numpy(), ref, atol=1e-5)
    # headwise with broadcast P == shared
    Qh, Kh, Vh = O.reconstruct_qkv_token(Pq[:, None].expand(B, H, R), Pk[:, None].expand(B, Hk, R),
                                         Pv[:, None].expand(B, Hk, R), Vq, Vk, Vv, bq, bk, bv)
    assert torch.allclose(Qh, Qs, atol=1e-6) and torch.allclose(Kh, Ks, atol=1e-6) and torch.allclose(Vh, Vs, atol=1e-6)
    # prepacked == shared; flat identity
    fq, fk, fv = O.pack_qkv_shared_bases(Vq, Vk, Vv)
    assert fq.shape == (R, H * Dh)
    Qp, Kp, Vp = O.reconstruct_qkv_token_shared_prepacked(Pq, Pk, Pv, fq, fk, fv, H=H, Hk=Hk, Dh=Dh, bq=bq, bk=bk, bv=bv)
    assert torch.allclose(Qp, Qs, atol=1e-5) and torch.allclose(Kp, Ks, atol=1e-5) and torch.allclose(Vp, Vs, atol=1e-5)
    assert torch.allclose((Pk @ fk)[:, Dh:2 * Dh] + bk[1], Ks[:, 1], atol=1e-5)
    # hetero ranks
    Q2, K2, V2 = O.reconstruct_qkv_token_shared_hetero(Pq, Pk[:, :16], Pv[:, :8], Vq, Vk[:, :16], Vv[:, :8])
    assert torch.allclose(K2, torch.einsum("br,hrd->bhd", Pk[:, :16], Vk[:, :16]), atol=1e-5)
    assert torch.allclose(V2, torch.einsum("br,hrd->bhd", Pv[:, :8], Vv[:, :8]), atol=1e-5)


# ---------------------------------------------------------------- decode attention
def test_dense_decode_attn_matches_sdpa_gqa():
    B, H, Hk, L, Dh = 2, 4, 2, 9, 8
    q, k, v = _rand(B, H, Dh, seed=1), _rand(B, L, Hk, Dh, seed=2), _rand(B, L, Hk, Dh, seed=3)
    out = O.dense_decode_attn(q, k, v)
    kk = k.permute(0, 2, 1, 3).repeat_interleave(H // Hk, dim=1)
    vv = v.permute(0, 2, 1, 3).repeat_interleave(H // Hk, dim=1)
    ref = torch.nn.functional.scaled_dot_product_attention(q[:, :, None], kk, vv)[:, :, 0]
    assert torch.allclose(out, ref, atol=1e-5)


def test_flash_attn_with_kvcache_append_then_attend():
    B, H, Hk, Dh, S = 2, 4, 2, 8, 12
    cos, sin = O.rope_tables(S, Dh)
    kraw, vraw = _rand(B, S, Hk, Dh, seed=1), _rand(B, S, Hk, Dh, seed=2)
    qraw = _rand(B, S, H, Dh, seed=3)
    n = 7
    kc = torch.zeros(B, S, Hk, Dh)
    vc = torch.zeros(B, S, Hk, Dh)
    kc[:, :n] = O.apply_rope_fp32(kraw[:, :n], cos[:n][None, :, None], sin[:n][None, :, None])
    vc[:, :n] = vraw[:, :n]
    seqlens = torch.full((B,), n, dtype=torch.int32)
    out = O.flash_attn_with_kvcache(qraw[:, n:n + 1], kc, vc, k=kraw[:, n:n + 1], v=vraw[:, n:n + 1],
                                    cache_seqlens=seqlens, rotary_cos=cos, rotary_sin=sin, causal=True)
    # cache mutated at position n
    assert torch.allclose(kc[:, n], O.apply_rope_fp32(kraw[:, n], cos[n], sin[n]))
    assert torch.equal(vc[:, n], vraw[:, n]) and torch.all(kc[:, n + 1:] == 0)
    # equals last row of full causal SDPA over n+1 rotated tokens
    qr = O.apply_rope_fp32(qraw[:, :n + 1], cos[:n + 1][None, :, None], sin[:n + 1][None, :, None])
    kr = O.apply_rope_fp32(kraw[:, :n + 1], cos[:n + 1][None, :, None], sin[:n + 1][None, :, None])
    ref = torch.nn.functional.scaled_dot_product_attention(
        qr.permute(0, 2, 1, 3), kr.permute(0, 2, 1, 3).repeat_interleave(2, 1),
        vraw[:, :n + 1].permute(0, 2, 1, 3).repeat_interleave(2, 1), is_causal=True)
    assert torch.allclose(out[:, 0], ref[:, :, -1], atol=1e-5)


def test_rank_decode_equals_dense_on_reconstructed_kv_and_is_block_invariant():
    B, H, Hk, L, R, Dh = 2, 4, 2, 37, 12, 8
    cos, sin = O.rope_tables(L, Dh)
    q = _rand(B, H, Dh, seed=1)
    Pk, Pv = _rand(B, L, R, seed=2), _rand(B, L, R, seed=3)
    Vk, Vv = _rand(Hk, R, Dh, seed=4), _rand(Hk, R, Dh, seed=5)
    K = torch.einsum("blr,krd->blkd", Pk, Vk)
    V = torch.einsum("blr,krd->blkd", Pv, Vv)
    Kr = O.apply_rope_fp32(K, cos[None, :, None], sin[None, :, None])
    ref = O.dense_decode_attn(q, Kr, V)
    outs = [O.rank_decode_attn(q, Pk, Pv, Vk, Vv, cos, sin, BN=bn) for bn in (1, 5, 16, 64)]
    for o in outs:
        assert torch.allclose(o, ref, atol=2e-5)
    # V-absorption identity: sum_n p_n (Pv_n Vv) == (sum_n p_n Pv_n) Vv
    scores = torch.einsum("bkgd,blkd->bkgl", q.reshape(B, Hk, 2, Dh), Kr) / math.sqrt(Dh)
    p = torch.softmax(scores, -1)
    absorbed = torch.einsum("bkgr,krd->bkgd", torch.einsum("bkgl,blr->bkgr", p, Pv), Vv).reshape(B, H, Dh)
    assert torch.allclose(absorbed, ref, atol=2e-5)
    # headwise variant with expanded shared P agrees
    hw = O.rank_decode_attn_headwise(q, Pk[:, :, None].expand(B, L, Hk, R), Pv[:, :, None].expand(B, L, Hk, R), Vk, Vv, cos, sin)
    assert torch.allclose(hw, ref, atol=2e-5)


# ---------------------------------------------------------------- fused prefill
def test_rope_sdpa_prefill_equals_reconstruct_rope_sdpa():
    B, H, Hk, M, R, dh = 2, 4, 2, 11, 6, 8
    cos, sin = O.rope_tables(M, dh)
    Pq, Pk, Pv = _rand(B, H, M, R, seed=1), _rand(B, Hk, M, R, seed=2), _rand(B, Hk, M, R, seed=3)
    Vq, Vk, Vv = _rand(H, R, dh, seed=4), _rand(Hk, R, dh, seed=5), _rand(Hk, R, dh, seed=6)
    out = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin)
    q = O.apply_rope_fp32(torch.einsum("bhmr,hrd->bhmd", Pq, Vq), cos[None, None], sin[None, None])
    k = O.apply_rope_fp32(torch.einsum("bhmr,hrd->bhmd", Pk, Vk), cos[None, None], sin[None, None])
    v = torch.einsum("bhmr,hrd->bhmd", Pv, Vv)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), is_causal=True)
    assert torch.allclose(out, ref.permute(0, 2, 1, 3), atol=1e-5)
    # last row == decode over the same keys
    dec = O.dense_decode_attn(q[:, :, -1], k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3))
    assert torch.allclose(out[:, -1], dec, atol=1e-5)
    # left-padded batch row: padded keys masked; a query whose keys are all masked gives 0
    pad = torch.ones(B, M, dtype=torch.long)
    pad[1, :3] = 0
    outp = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin, pad_mask=pad)
    assert torch.all(outp[1, :3] == 0)
    assert torch.allclose(outp[0], out[0], atol=1e-6)
    ref1 = torch.nn.functional.scaled_dot_product_attention(
        q[1:, :, 3:], k[1:, :, 3:].repeat_interleave(2, 1), v[1:, :, 3:].repeat_interleave(2, 1), is_causal=True)
    assert torch.allclose(outp[1, 3:], ref1[0].permute(1, 0, 2), atol=1e-5)


# ---------------------------------------------------------------- MLP
def test_dual_split_closed_form_and_partition_invariance():
    B, L, R, D, Hd = 2, 1, 10, 37, 12
    PUp, PGate = _rand(B, L, R, seed=1), _rand(B, L, R, seed=2)
    GateU, UpU = _rand(R, D, seed=3), _rand(R, D, seed=4)
    DownV, DownU, b2 = _rand(D, R, seed=5), _rand(R, Hd, seed=6), _rand(Hd, seed=7)
    y = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2)
    g = (PGate.double() @ GateU.double())
    u = (PUp.double() @ UpU.double())
    ref = ((g / (1 + torch.exp(-g))) * u) @ DownV.double() @ DownU.double() + b2.double()
    assert torch.allclose(y.double(), ref, atol=1e-5)
    # swapping gate/up must change the answer (catches transposed operands)
    assert not torch.allclose(O.dual_split_mlp(PGate, PUp, GateU, UpU, DownV, DownU, b2).double(), ref, atol=1e-3)
    for bd in (1, 8, 16, 64):
        assert torch.allclose(O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=bd), y, atol=1e-5)
    assert torch.allclose(O.dual_split_mlp_pcat(torch.cat([PUp, PGate], -1), GateU, UpU, DownV, DownU, b2), y, atol=1e-6)
    assert torch.allclose(O.dual_split_mlp_v3(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=16, BR2=4), y, atol=1e-5)


def test_mlp_forward_full_rank_is_hf_llama_mlp():
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP
    d, ffn = 16, 24
    cfg = LlamaConfig(hidden_size=d, intermediate_size=ffn, hidden_act="silu", mlp_bias=False, num_attention_heads=2)
    mlp = LlamaMLP(cfg)
    R = d  # full rank factors: v orthonormal [R,in], u = W v^T
    qd, _ = torch.linalg.qr(_rand(d, d, seed=1))
    qf, _ = torch.linalg.qr(_rand(ffn, ffn, seed=2))
    Wg, Wu, Wd = mlp.gate_proj.weight.detach(), mlp.up_proj.weight.detach(), mlp.down_proj.weight.detach()
    z = torch.zeros(1)
    bw = O.BlockWeights(q_v=z, q_u=z, k_v=z, k_u=z, v_v=z, v_u=z, o_v=z, o_u=z,
                        gate_v=qd.t().contiguous(), gate_u=Wg @ qd, up_v=qd.t().contiguous(), up_u=Wu @ qd,
                        down_v=qf.t().contiguous(), down_u=Wd @ qf, ln1=z, ln2=z)
    x = _rand(3, d, seed=3)
    assert torch.allclose(O.mlp_forward(bw, x), mlp(x).detach(), atol=1e-5)


# ---------------------------------------------------------------- whole model
def _tiny(dtype=torch.float32, n_layers=2, kvh=2):
    return O.make_model(d=32, n_heads=4, n_kv_heads=kvh, head_dim=8, ffn=48, attn_rank=12, mlp_rank=16,
                        n_layers=n_layers, vocab=50, dtype=dtype, seed=0, std=0.3)


def test_model_matches_transformers_llama_with_dense_weights():
    from transformers import LlamaConfig, LlamaForCausalLM
    mw = _tiny()
    cfg = LlamaConfig(vocab_size=50, hidden_size=32, intermediate_size=48, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, head_dim=8, rms_norm_eps=1e-6,
                      rope_theta=10000.0, attention_bias=False, mlp_bias=False, tie_word_embeddings=False,
                      max_position_embeddings=64, attn_implementation="eager")
    hf = LlamaForCausalLM(cfg).eval()
    with torch.no_grad():
        hf.model.embed_tokens.weight.copy_(mw.embed)
        hf.lm_head.weight.copy_(mw.lm_head)
        hf.model.norm.weight.copy_(mw.norm)
        for layer, b in zip(hf.model.layers, mw.blocks):
            a, m = layer.self_attn, layer.mlp
            a.q_proj.weight.copy_(b.q_u @ b.q_v); a.k_proj.weight.copy_(b.k_u @ b.k_v)
            a.v_proj.weight.copy_(b.v_u @ b.v_v); a.o_proj.weight.copy_(b.o_u @ b.o_v)
            m.gate_proj.weight.copy_(b.gate_u @ b.gate_v); m.up_proj.weight.copy_(b.up_u @ b.up_v)
            m.down_proj.weight.copy_(b.down_u @ b.down_v)
            layer.input_layernorm.weight.copy_(b.ln1); layer.post_attention_layernorm.weight.copy_(b.ln2)
    ids = torch.randint(0, 50, (2, 9), generator=torch.Generator().manual_seed(3))
    with torch.no_grad():
        ref = hf(input_ids=ids).logits
    mine = O.model_forward(mw, ids, last_only=False)
    assert torch.allclose(mine, ref, atol=2e-4, rtol=1e-3)


@pytest.mark.parametrize("cache_kind", ["dense", "rank"])
def test_cached_greedy_decode_equals_full_recompute(cache_kind):
    mw = _tiny()
    prompt = torch.randint(0, 50, (2, 6), generator=torch.Generator().manual_seed(5))
    toks, hid, _ = O.greedy_decode(mw, prompt, 5, cache_kind=cache_kind, return_hidden=True)
    seq = prompt
    for step in range(5):
        logits, h = O.model_forward(mw, seq, return_hidden=True)
        assert torch.allclose(h[:, -1], hid[:, step], atol=1e-4)
        nxt = logits[:, -1].argmax(-1, keepdim=True)
        assert torch.equal(nxt, toks[:, step:step + 1])
        seq = torch.cat([seq, nxt], 1)


@pytest.mark.parametrize("dt,noise", [(torch.bfloat16, 0.15), (torch.float16, 0.02)], ids=["bf16", "fp16"])
def test_rank_cache_and_dense_cache_agree_16bit(dt, noise):
    mw = _tiny(dt)
    prompt = torch.randint(0, 50, (1, 8), generator=torch.Generator().manual_seed(6))
    _, hd, _ = O.greedy_decode(mw, prompt, 4, "dense", return_hidden=True)
    _, hr, _ = O.greedy_decode(mw, prompt, 4, "rank", return_hidden=True)
    assert hd.dtype == dt and (hd.float() - hr.float()).abs().max() < noise  # rounding noise of the type only; same algebra


# ---- group-wise int4 weights (src/quant/packed_quant_linear.py) --------------------------------
def test_int4_pack_layout_by_hand():
    q = torch.tensor([[1, 2, 3, 15, 0, 7, 9]], dtype=torch.uint8)            # odd length: one padding nibble
    packed = O.pack_int4(q)
    assert packed.tolist() == [[0x21, 0xF3, 0x70, 0x09]]                       # even column low nibble, odd column high
    assert O.unpack_int4(packed, 7).tolist() == q.tolist()
    g = torch.Generator().manual_seed(0)
    q = torch.randint(0, 16, (5, 64), generator=g, dtype=torch.uint8)
    assert torch.equal(O.unpack_int4(O.pack_int4(q), 64), q)


def test_int4_quantize_by_hand():
    # one row, two groups of 4.  group 0: min -1.5, max 6 -> scale 0.5, zero = round(3) = 3
    # group 1: all zero -> range [-1, 1]: scale 2/15, zero = round(1 / fp32(2/15)) = round(7.4999996) = 7
    w = torch.tensor([[-1.5, 0.0, 6.0, 2.26, 0.0, 0.0, 0.0, 0.0]])
    qw, sc, zr = O.quantize_weight(w, bits=4, group_size=4, sym=False)
    assert sc.dtype == torch.float16 and zr.dtype == torch.int16 and qw.dtype == torch.uint8
    assert sc.tolist() == [[0.5, float(torch.tensor(2 / 15).half())]] and zr.tolist() == [[3, 7]]
    assert O.unpack_int4(qw, 8).tolist() == [[0, 3, 15, 8, 7, 7, 7, 7]]        # 2.26/0.5 = 4.52 -> 5, + 3
    deq = O.dequantize_weight(qw, sc, zr, in_features=8, group_size=4)
    assert deq.tolist() == [[-1.5, 0.0, 6.0, 2.5, 0.0, 0.0, 0.0, 0.0]]
    # symmetric: zero point 8, scale = 2*max|w|/15, clamp keeps q within 0..15
    qw, sc, zr = O.quantize_weight(w, bits=4, group_size=-1, sym=True)
    assert zr.tolist() == [[8]] and sc.shape == (1, 1) and float(sc[0, 0]) == float(torch.tensor(12 / 15).half())
    assert O.unpack_int4(qw, 8).tolist() == [[6, 8, 15, 11, 8, 8, 8, 8]]       # 6/0.8 = 7.5 -> 8 (even) + 8 = 16 -> clamp 15
    # 8 bits keep one byte per weight
    qw8, sc8, zr8 = O.quantize_weight(w, bits=8, group_size=4)
    assert qw8.shape == (1, 8) and int(qw8.max()) == 255 and int(qw8.min()) == 0


def test_int4_round_trip_error_bound_and_linear_closed_form():
    g = torch.Generator().manual_seed(1)
    w = torch.randn(24, 96, generator=g) * 0.05
    for group, sym in ((32, False), (32, True), (-1, False), (40, False)):       # 40: ragged last group
        qw, sc, zr = O.quantize_weight(w, group_size=group, sym=sym)
        G = 1 if group <= 0 else -(-96 // group)
        assert sc.shape == (24, G) and zr.shape == (24, G) and qw.shape == (24, 48)
        deq = O.dequantize_weight(qw, sc, zr, in_features=96, group_size=group)
        width = 96 if group <= 0 else group
        bound = sc.float().repeat_interleave(width, dim=1)[:, :96]
        # rounding to the grid costs at most half a step; the scale is stored in fp16 (2^-11 relative) and
        # multiplies a level distance |q - z| of at most 15
        assert bool(((w - deq).abs() <= bound * (0.5 + 15 * 2 ** -11) * (1 + 2 ** -10) + 1e-7).all()), (group, sym)
    # the linear is x @ (s * (q - z))^T: check against float64 arithmetic written out element by element
    qw, sc, zr = O.quantize_weight(w, group_size=32)
    x = torch.randn(3, 96, generator=g)
    y = O.quant_linear(x, qw, sc, zr, group_size=32)
    q = O.unpack_int4(qw, 96).double()
    ref = torch.zeros(3, 24, dtype=torch.float64)
    for n in range(24):
        for k in range(96):
            ref[:, n] += x[:, k].double() * (sc[n, k // 32].double() * (q[n, k] - zr[n, k // 32].double()))
    assert torch.allclose(y.double(), ref, rtol=1e-5, atol=1e-6)
    # bf16 activations: the dequantised weight is rounded to bf16 before the product
    xb = x.to(torch.bfloat16)
    yb = O.quant_linear(xb, qw, sc, zr, group_size=32)
    wb = O.dequantize_weight(qw, sc, zr, in_features=96, group_size=32, dtype=torch.bfloat16)
    assert yb.dtype == torch.bfloat16 and torch.equal(yb, (xb.float() @ wb.float().t()).to(torch.bfloat16))


# ---------------------------------------------------------------- argument-level pins
def test_rope_sdpa_prefill_biases_and_additive_mask_match_sdpa():
    """bq / bk / bv and the additive mask against torch SDPA on explicitly biased, rotated q / k / v.  The kernel
    indexes bk and bv with the QUERY head (kernels/attn/prefill/rope_sdpa.py:176-183,229-230): under GQA two query
    heads that share a kv head then see different keys, which an index by kv head would not reproduce."""
    B, H, Hk, M, R, dh = 2, 4, 2, 9, 5, 8
    rep = H // Hk
    cos, sin = O.rope_tables(M, dh)
    Pq, Pk, Pv = _rand(B, H, M, R, seed=11), _rand(B, Hk, M, R, seed=12), _rand(B, Hk, M, R, seed=13)
    Vq, Vk, Vv = _rand(H, R, dh, seed=14), _rand(Hk, R, dh, seed=15), _rand(Hk, R, dh, seed=16)
    bq, bk, bv = _rand(H * dh, seed=17), _rand(H * dh, seed=18), _rand(H * dh, seed=19)
    add = _rand(B, 1, M, M, seed=20)
    out = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin, bq=bq, bk=bk, bv=bv, add_mask=add)

    d64 = torch.float64
    c, s = cos.to(d64), sin.to(d64)

    def rot(x):   # [M, dh] rotate-half, written out per pair
        y = torch.empty_like(x)
        for i in range(dh // 2):
            y[:, i] = x[:, i] * c[:, i] - x[:, i + dh // 2] * s[:, i]
            y[:, i + dh // 2] = x[:, i] * s[:, i] + x[:, i + dh // 2] * c[:, i]
        return y

    ref = torch.empty(B, M, H, dh, dtype=d64)
    causal = torch.full((M, M), -float("inf"), dtype=d64).triu(1)
    for b in range(B):
        for h in range(H):
            hk = h // rep
            q = rot(Pq[b, h].to(d64) @ Vq[h].to(d64) + bq[h * dh:(h + 1) * dh].to(d64))
            k = rot(Pk[b, hk].to(d64) @ Vk[hk].to(d64) + bk[h * dh:(h + 1) * dh].to(d64))
            v = Pv[b, hk].to(d64) @ Vv[hk].to(d64) + bv[h * dh:(h + 1) * dh].to(d64)
            ref[b, :, h] = torch.nn.functional.scaled_dot_product_attention(
                q[None], k[None], v[None], attn_mask=(causal + add[b, 0].to(d64))[None])[0]
    assert torch.allclose(out.to(d64), ref, atol=2e-5)
    # a bias indexed by kv head would make heads 0 and 1 (same kv head) share keys: they must not
    bk2 = bk.clone()
    bk2[dh:2 * dh] += 1.0          # query head 1 only
    out2 = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin, bq=bq, bk=bk2, bv=bv, add_mask=add)
    assert torch.allclose(out2[:, :, 0], out[:, :, 0], atol=1e-6) and torch.allclose(out2[:, :, 2:], out[:, :, 2:], atol=1e-6)
    assert not torch.allclose(out2[:, :, 1], out[:, :, 1], atol=1e-3)
    # the additive mask alone (no biases) against SDPA as well
    out3 = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin, add_mask=add)
    q = O.apply_rope_fp32(torch.einsum("bhmr,hrd->bhmd", Pq, Vq), cos[None, None], sin[None, None])
    k = O.apply_rope_fp32(torch.einsum("bhmr,hrd->bhmd", Pk, Vk), cos[None, None], sin[None, None])
    v = torch.einsum("bhmr,hrd->bhmd", Pv, Vv)
    ref3 = torch.nn.functional.scaled_dot_product_attention(
        q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1), attn_mask=causal.float()[None, None] + add)
    assert torch.allclose(out3, ref3.permute(0, 2, 1, 3), atol=1e-5)


def _bf(x):
    """One rounding to bf16, result held in float64 (inputs far inside the fp32 range)."""
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float64)


def test_dual_split_bf16_rounding_points_v1_workspace_and_v3():
    """The bf16 rounding points of the v1 (workspace dtype) and v3 (per-tile s) variants against a float64 restatement
    with every rounding written out.  Operands are small multiples of 1/8 so that every fp32 partial sum is exact and
    a rounding applied at the wrong place (or left out) changes bits; only silu involves a transcendental."""
    bf = torch.bfloat16
    B, L, R, D, Hd, BD, BR2 = 2, 1, 8, 24, 6, 8, 4
    g = torch.Generator().manual_seed(77)

    def grid(*shape, span=8):
        return (torch.randint(-span, span + 1, shape, generator=g).float() / 8).to(bf)

    PUp, PGate = grid(B, L, R), grid(B, L, R)
    GateU, UpU, DownV, DownU, b2 = grid(R, D), grid(R, D), grid(D, R), grid(R, Hd), grid(Hd)
    d64 = torch.float64
    gg = PGate.reshape(B, R).to(d64) @ GateU.to(d64)
    uu = PUp.reshape(B, R).to(d64) @ UpU.to(d64)
    h = _bf((gg / (1 + torch.exp(-gg))) * uu)                       # dual_split_triton.py:207
    tiles = [h[:, d0:d0 + BD] @ DownV[d0:d0 + BD].to(d64) for d0 in range(0, D, BD)]
    # v1, partials through a bf16 workspace, then .sum(1) (bf16 result), then the DownU product (:586-624)
    S_v1_bf = _bf(sum(_bf(t) for t in tiles))
    y_v1_bf = _bf(S_v1_bf @ DownU.to(d64) + b2.to(d64))
    # v1 with fp32 partials / v2: fp32 sum, one rounding of S (:686-721)
    S_f32 = _bf(sum(tiles))
    y_f32 = _bf(S_f32 @ DownU.to(d64) + b2.to(d64))
    got_bf = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=BD, variant="v1", work_dtype=bf)
    got_f32 = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=BD, variant="v1", work_dtype=torch.float32)
    got_v2 = O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=BD, variant="v2")
    assert torch.equal(got_bf.reshape(B, Hd).to(d64), y_v1_bf)
    assert torch.equal(got_f32.reshape(B, Hd).to(d64), y_f32)
    assert torch.equal(got_v2.reshape(B, Hd).to(d64), y_f32)
    assert not torch.equal(y_v1_bf, y_f32), "operands too tame: the workspace rounding changes nothing"
    # v3: s per (D tile, BR2 slice) rounded to bf16, Y summed in fp32, rounded once, b2 added afterwards in bf16 (:427-532,858-966)
    Y = torch.zeros(B, Hd, dtype=d64)
    for d0 in range(0, D, BD):
        for r0 in range(0, R, BR2):
            s = _bf(h[:, d0:d0 + BD] @ DownV[d0:d0 + BD, r0:r0 + BR2].to(d64))
            Y += s @ DownU[r0:r0 + BR2].to(d64)
    y_v3 = _bf(_bf(Y) + b2.to(d64))
    got_v3 = O.dual_split_mlp_v3(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=BD, BR2=BR2)
    assert torch.equal(got_v3.reshape(B, Hd).to(d64), y_v3)
    assert not torch.equal(y_v3, y_f32)


def test_exact_mode_matches_float64_restatement_and_bounds_the_bf16_run():
    """The exact mode (fp64 activations, stored bf16 weights, no rounding between operators) against an independent
    float64 restatement of one block written with numpy and explicit loops over heads and positions; the bf16 run of
    the same block must then sit within a few bf16 roundings of it."""
    mw = _tiny(torch.bfloat16, n_layers=1, kvh=2)
    T, d, H, Hk, Dh = 5, 32, 4, 2, 8
    x = _rand(1, T, d, seed=9).to(torch.bfloat16)
    cos, sin = O.rope_tables(T, Dh, dtype=torch.bfloat16)
    got = O.block_forward(mw, 0, x.double(), 0, None, cos, sin)[0].numpy()
    assert got.dtype == np.float64
    b = mw.blocks[0]
    W = {k: getattr(b, k).double().numpy() for k in ("q_v", "q_u", "k_v", "k_u", "v_v", "v_u", "o_v", "o_u", "gate_v", "gate_u",
                                                      "up_v", "up_u", "down_v", "down_u", "ln1", "ln2")}
    xn = x[0].double().numpy()
    c, s = cos.double().numpy(), sin.double().numpy()

    def rms(v, w):
        return w * (v / np.sqrt((v * v).mean(-1, keepdims=True) + mw.eps))

    def rope(v, t):     # v [Dh]
        half = Dh // 2
        out = np.empty(Dh)
        for i in range(half):
            out[i] = v[i] * c[t, i] - v[i + half] * s[t, i]
            out[i + half] = v[i + half] * c[t, i] + v[i] * s[t, i]
        return out

    h1 = rms(xn, W["ln1"])
    q = (h1 @ W["q_v"].T) @ W["q_u"].T
    k = (h1 @ W["k_v"].T) @ W["k_u"].T
    v = (h1 @ W["v_v"].T) @ W["v_u"].T
    attn = np.zeros((T, H * Dh))
    for t in range(T):
        for hh in range(H):
            hk = hh // (H // Hk)
            qt = rope(q[t, hh * Dh:(hh + 1) * Dh], t)
            sc = np.array([qt @ rope(k[n, hk * Dh:(hk + 1) * Dh], n) for n in range(t + 1)]) / math.sqrt(Dh)
            p = np.exp(sc - sc.max())
            p /= p.sum()
            attn[t, hh * Dh:(hh + 1) * Dh] = sum(p[n] * v[n, hk * Dh:(hk + 1) * Dh] for n in range(t + 1))
    x2 = xn + (attn @ W["o_v"].T) @ W["o_u"].T
    h2 = rms(x2, W["ln2"])
    gg = (h2 @ W["gate_v"].T) @ W["gate_u"].T
    uu = (h2 @ W["up_v"].T) @ W["up_u"].T
    ref = x2 + (((gg / (1 + np.exp(-gg))) * uu) @ W["down_v"].T) @ W["down_u"].T
    assert np.allclose(got, ref, rtol=1e-11, atol=1e-12)
    # fp32 activations: the same up to fp32 accumulation noise
    got32 = O.block_forward(mw, 0, x.float(), 0, None, cos, sin)[0].double().numpy()
    assert np.abs(got32 - ref).max() <= 1e-5 * np.abs(ref).max()
    # the bf16 run differs from the exact one, by bf16 roundings only
    got16 = O.block_forward(mw, 0, x, 0, None, cos, sin)[0].double().numpy()
    err = np.abs(got16 - ref).max() / np.abs(ref).max()
    assert 1e-4 < err < 3e-2, err


def test_teacher_forced_decode_and_layer_trace():
    """forced= feeds the given tokens; with a run's own tokens it reproduces that run; layer_trace returns every
    block's input, chained by block_forward."""
    mw = _tiny(torch.float32)
    prompt = torch.randint(0, 50, (1, 6), generator=torch.Generator().manual_seed(8))
    toks, hid, _, logits = O.greedy_decode(mw, prompt, 5, return_logits=True)
    trace = []
    toks2, hid2, cache2, logits2 = O.greedy_decode(mw, prompt, 5, return_logits=True, forced=toks, layer_trace=trace)
    assert torch.equal(toks, toks2) and torch.equal(logits, logits2)
    assert len(trace) == 4 and all(len(t) == len(mw.blocks) + 1 for t in trace)
    assert torch.equal(trace[2][0][0, 0], mw.embed[toks[0, 2]])
    assert torch.equal(trace[2][-1][:, -1], hid[:, 3])
    other = (toks + 7) % 50
    toks3, _, _, _ = O.greedy_decode(mw, prompt, 5, return_logits=True, forced=other)
    seq = torch.cat([prompt, other[:, :1]], 1)
    assert int(O.model_forward(mw, seq)[0, -1].argmax()) == int(toks3[0, 1])
