"""The fused product path in float16 (dtype code FSVD_FP16 through the C ABI) against the CPU oracle run in float16.

The reference switches its kernels on the input dtype, its dense cache defaults to float16 and its model cast falls back
to float16 (kernels/attn/decode/densekv_reconstruct_triton.py:427-428, runtime/cache/attn_dense_kv.py:26,
scripts/demo_support/api.py:161-165).  Here every entry point of the path takes the element type as an argument; the
kernels are the bf16 ones instantiated with the float16 conversions, V_DOT2_F32_F16 and V_MFMA_F32_16X16X32_F16.

Tolerance: float16 carries three more mantissa bits than bfloat16, so the bar is a quarter of the bf16 one
(max-abs 5e-3, max-rel 2.5e-3); where max|ref| >= 2 the absolute bound is two float16 ulps at max|ref| (one ulp is
0.002 in [2, 4)).  Greedy tokens identical on configuration 1.
"""
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, model_from_oracle

pytestmark = pytest.mark.gpu
FP16 = torch.float16


def rand_fp16(*shape, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(FP16)


def close(got, ref, what):
    assert got.dtype == FP16, f"{what}: result is {got.dtype}"
    m = float(ref.float().abs().max())
    return assert_close_bf16(got, ref, what, abs_tol=5e-3 if m < 2.0 else 2.0 * m * 2.0 ** -10, rel_tol=2.5e-3)


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from flashsvd_amd import hip_ops
    return hip_ops


# one row (vector kernels), three rows and more (matrix cores: streamed, resident, K-split forms), prompt rows (tiles)
@pytest.mark.parametrize("B,N,K", [(1, 3072, 4096), (1, 1536, 11008), (2, 257, 512), (1, 7, 100), (3, 512, 4096), (8, 3072, 4096),
                                   (16, 1536, 11008), (32, 4096, 1536), (17, 100, 2048), (20, 8192, 6144), (100, 200, 1536),
                                   (512, 3072, 4096), (129, 130, 192), (384, 1536, 11008), (2048, 4096, 256)])
def test_linear(ops, B, N, K):
    x, w = rand_fp16(B, K, seed=1), rand_fp16(N, K, std=0.02, seed=2)
    bias, res = rand_fp16(N, std=0.1, seed=4), rand_fp16(B, N, seed=5)
    close(ops.linear(x.cuda(), w.cuda()), O.lin(x, w), f"linear {B}x{N}x{K}")
    close(ops.linear(x.cuda(), w.cuda(), bias.cuda(), residual=res.cuda()), res + O.lin(x, w, bias), f"linear + bias + residual {B}x{N}x{K}")


@pytest.mark.parametrize("B", [1, 2, 8, 200])
def test_linear_with_fused_norm_and_rmsnorm(ops, B):
    N, K = 512, 4096
    x, w = rand_fp16(B, K, seed=1), rand_fp16(N, K, std=0.02, seed=2)
    nw = rand_fp16(K, seed=3) * 0.1 + 1
    close(ops.rmsnorm(x.cuda(), nw.cuda(), 1e-6), O.rms_norm(x, nw, 1e-6), "rmsnorm")
    close(ops.linear(x.cuda(), w.cuda(), norm_weight=nw.cuda(), eps=1e-6), O.lin(O.rms_norm(x, nw, 1e-6), w), "norm + linear")


@pytest.mark.parametrize("B,D,R,mode", [(1, 11008, 1536, 0), (1, 11008, 1536, 1), (2, 100, 52, 1), (8, 11008, 1536, 0), (32, 1376, 256, 1),
                                        (24, 14336, 2048, 0), (512, 11008, 1536, 0), (256, 1376, 256, 1)])
def test_swiglu_linear(ops, B, D, R, mode):
    p = rand_fp16(B, 2 * R, seed=1)
    gu, uu = rand_fp16(D, R, std=0.05, seed=2), rand_fp16(D, R, std=0.05, seed=3)
    h = ops.swiglu_linear(p.cuda(), gu.cuda(), uu.cuda(), up_off=R, mode=mode)
    g, u = p[:, :R].float() @ gu.float().t(), p[:, R:].float() @ uu.float().t()
    if mode == 0:
        ref = torch.nn.functional.silu(g.to(FP16)) * u.to(FP16)
    else:
        ref = ((g * torch.sigmoid(g)) * u).to(FP16)
    close(h, ref, f"swiglu mode {mode} at {B} rows")


@pytest.mark.parametrize("B,H,Hk,Dh,Rq,Rk,Rv", [(1, 32, 32, 128, 1024, 1024, 1024), (2, 8, 2, 64, 128, 96, 72), (3, 4, 4, 64, 52, 52, 52)])
def test_qkv_rope_append(ops, B, H, Hk, Dh, Rq, Rk, Rv):
    S = 40
    p = rand_fp16(B, Rq + Rk + Rv, seed=1)
    qu, ku, vu = rand_fp16(H * Dh, Rq, std=0.05, seed=2), rand_fp16(Hk * Dh, Rk, std=0.05, seed=3), rand_fp16(Hk * Dh, Rv, std=0.05, seed=4)
    cos, sin = O.rope_tables(S, Dh, dtype=FP16)
    pos = torch.tensor([(7 * b + 5) % S for b in range(B)], dtype=torch.int32)
    kc = torch.zeros(B, S, Hk, Dh, dtype=FP16, device="cuda")
    vc = torch.zeros_like(kc)
    q = ops.qkv_rope_append(p.cuda(), qu.cuda(), ku.cuda(), vu.cuda(), cos.cuda(), sin.cuda(), pos.cuda(), kc, vc,
                            num_heads=H, num_kv_heads=Hk, head_dim=Dh)
    pq, pk, pv = p[:, :Rq], p[:, Rq:Rq + Rk], p[:, Rq + Rk:]
    for b in range(B):
        c, s = cos[pos[b]], sin[pos[b]]
        close(q[b], O.apply_rope(O.lin(pq[b:b + 1], qu).reshape(H, Dh), c, s), "q")
        close(kc[b, pos[b]], O.apply_rope(O.lin(pk[b:b + 1], ku).reshape(Hk, Dh), c, s), "k row")
        close(vc[b, pos[b]], O.lin(pv[b:b + 1], vu).reshape(Hk, Dh), "v row")


@pytest.mark.parametrize("B,H,Hk,Dh,L,S,nsplit", [(1, 32, 32, 128, 513, 560, 8), (2, 8, 2, 64, 37, 64, 3), (2, 4, 4, 64, 100, 128, 1),
                                                 (16, 32, 8, 128, 300, 320, 4), (16, 32, 16, 128, 130, 160, 2)])
def test_attn_decode_densekv(ops, B, H, Hk, Dh, L, S, nsplit):
    q = rand_fp16(B, H, Dh, seed=1)
    kc, vc = rand_fp16(B, S, Hk, Dh, seed=2), rand_fp16(B, S, Hk, Dh, seed=3)
    lens = torch.tensor([max(1, L - 3 * b) for b in range(B)], dtype=torch.int32)
    out = ops.attn_decode_densekv(q.cuda(), kc.cuda(), vc.cuda(), lens.cuda(), nsplit=nsplit)
    for b in range(B):
        n = int(lens[b])
        close(out[b:b + 1], O.dense_decode_attn(q[b:b + 1], kc[b:b + 1, :n], vc[b:b + 1, :n]), f"attention b={b}")


def test_attn_decode_appends_and_rotates_the_new_token(ops):
    B, H, Hk, Dh, S, n = 2, 8, 4, 128, 64, 21
    q, kn, vn = rand_fp16(B, H, Dh, seed=1), rand_fp16(B, Hk, Dh, seed=2), rand_fp16(B, Hk, Dh, seed=3)
    kc, vc = rand_fp16(B, S, Hk, Dh, seed=4), rand_fp16(B, S, Hk, Dh, seed=5)
    cos, sin = O.rope_tables(S, Dh, dtype=FP16)
    lens = torch.full((B,), n, dtype=torch.int32)
    kg, vg = kc.cuda(), vc.cuda()
    out = ops.attn_decode_densekv(q.cuda(), kg, vg, lens.cuda(), k_new=kn.cuda(), v_new=vn.cuda(), cos=cos.cuda(), sin=sin.cuda(), nsplit=2)
    ref = O.flash_attn_with_kvcache(q[:, None], kc.clone(), vc.clone(), k=kn[:, None], v=vn[:, None], cache_seqlens=lens,
                                    rotary_cos=cos, rotary_sin=sin)
    close(out, ref[:, 0], "attention with append")


@pytest.mark.parametrize("B,M,R", [(2, 40, 72), (1, 512, 1024), (2, 200, 128)])
def test_expand_heads_and_prompt_attention(ops, B, M, R):
    H, Hk, dh = 8, 4, 128
    S = M + 24
    cos, sin = O.rope_tables(S, dh, dtype=FP16)
    pq, pk, pv = rand_fp16(B, M, R, seed=1), rand_fp16(B, M, R, seed=2), rand_fp16(B, M, R, seed=3)
    uq, uk, uv = rand_fp16(H * dh, R, std=R ** -0.5, seed=4), rand_fp16(Hk * dh, R, std=R ** -0.5, seed=5), rand_fp16(Hk * dh, R, std=R ** -0.5, seed=6)
    q = torch.empty(B, M, H, dh, dtype=FP16, device="cuda")
    kc = torch.zeros(B, S, Hk, dh, dtype=FP16, device="cuda")
    vc = torch.zeros_like(kc)
    pos0 = torch.zeros(B, dtype=torch.int32, device="cuda")
    ops.lowrank_expand_heads_multi(
        [dict(p=pq.cuda(), u=uq.cuda(), num_heads=H, out=q, rotate=True),
         dict(p=pk.cuda(), u=uk.cuda(), num_heads=Hk, out=kc, rotate=True, dst_by_position=True),
         dict(p=pv.cuda(), u=uv.cuda(), num_heads=Hk, out=vc, rotate=False, dst_by_position=True)],
        head_dim=dh, cos=cos.cuda(), sin=sin.cuda(), positions=pos0)
    c, s = cos[:M][None, :, None], sin[:M][None, :, None]
    q_ref = O.apply_rope(O.lin(pq, uq).reshape(B, M, H, dh), c, s)
    k_ref = O.apply_rope(O.lin(pk, uk).reshape(B, M, Hk, dh), c, s)
    v_ref = O.lin(pv, uv).reshape(B, M, Hk, dh)
    close(q, q_ref, "q expansion")
    close(kc[:, :M], k_ref, "k expansion into cache rows")
    close(vc[:, :M], v_ref, "v expansion into cache rows")
    single = torch.zeros_like(kc)
    ops.lowrank_expand_heads(pk.cuda(), uk.cuda(), num_heads=Hk, head_dim=dh, out=single, cos=cos.cuda(), sin=sin.cuda(),
                             positions=pos0, dst_by_position=True)
    assert torch.equal(single.cpu(), kc.cpu()), "one expansion and the batched launch differ"
    out = ops.attn_prefill(q_ref.cuda(), k_ref.cuda(), v_ref.cuda(), q_pos0=pos0, causal=True)
    for m in (0, M // 3, M - 1):
        close(out[:, m], O.dense_decode_attn(q_ref[:, m], k_ref[:, :m + 1], v_ref[:, :m + 1]), f"prompt attention row {m}")


@pytest.mark.parametrize("B,H,Hk,M,R,shared", [(1, 32, 32, 512, 1024, True), (2, 4, 2, 100, 40, False), (1, 8, 8, 333, 1664, True)])
def test_rope_attention_module(B, H, Hk, M, R, shared):
    """FlashSVDRoPEAttention (kernels/flashsvdropeattn.py, the reference's module interface) on float16 factors."""
    from flashsvd_amd.kernels.flashsvdropeattn import FlashSVDRoPEAttention, QKVFactors

    class Rot:
        inv_freq = 1.0 / (10000.0 ** (torch.arange(0, 64, dtype=torch.float32) / 64))

    dh = 128
    if shared:
        pq, pk, pv = (rand_fp16(B, 1, M, R, seed=i) for i in range(3))
        Pq, Pk, Pv = pq.expand(B, H, M, R), pk.expand(B, Hk, M, R), pv.expand(B, Hk, M, R)
    else:
        Pq, Pk, Pv = rand_fp16(B, H, M, R, seed=0), rand_fp16(B, Hk, M, R, seed=1), rand_fp16(B, Hk, M, R, seed=2)
    sc = R ** -0.5
    Vq, Vk, Vv = rand_fp16(H, R, dh, std=sc, seed=3), rand_fp16(Hk, R, dh, std=sc, seed=4), rand_fp16(Hk, R, dh, std=sc, seed=5)
    cos, sin = O.rope_tables(M, dh, dtype=FP16)
    ref = O.rope_sdpa_prefill(Pq, Pk, Pv, Vq, Vk, Vv, cos, sin)
    mod = FlashSVDRoPEAttention(H, dh, Rot(), bm=64, bn=64, br=64)
    out = mod(QKVFactors(*[t.cuda() for t in (Pq, Pk, Pv, Vq, Vk, Vv)]), None, torch.arange(M, device="cuda")[None])
    assert out.shape == (B, M, H, dh)
    close(out, ref, "rope attention module")


def test_mixed_element_types_are_refused(ops):
    x, w = rand_fp16(1, 256, seed=1).cuda(), rand_fp16(64, 256, seed=2).cuda()
    with pytest.raises(ValueError, match="must be torch.float16"):
        ops.linear(x, w.to(torch.bfloat16))
    with pytest.raises(ValueError, match="bfloat16 or torch.float16"):
        ops.linear(x.float(), w.float())


def _greedy(model, prompt, n_new, graph):
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    B, Lp = prompt.shape
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=B, max_cache_len=Lp + n_new + 4, device="cuda", dtype=FP16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp))
    hid = [out.hidden_states[:, -1].clone()]
    tok = out.logits[:, -1].float().argmax(-1, keepdim=True)
    toks = [tok.clone()]
    dec = GraphedDecoder(model, cache, B)
    dec.set_state(tok, Lp)
    if graph:
        dec.capture()
    for _ in range(1, n_new):
        toks.append((dec.step() if graph else dec.eager_step()).clone())
        hid.append(dec.hidden.clone())
    return torch.cat(toks, 1).cpu(), torch.stack(hid, 1).cpu(), cache


@pytest.mark.parametrize("graph", [False, True])
def test_config1_block_greedy_16_identical_in_float16(graph):
    # configuration 1 of the reference (d 512, 8 x 64 heads, ffn 1376, ranks 128 / 256, prompt 128, 16 greedy steps)
    mw, prompt = O.config_c1(FP16)
    model = model_from_oracle(mw)
    assert model.lm_head.weight.dtype == FP16
    ref_tok, ref_hid, ref_cache = O.greedy_decode(mw, prompt, 16, "dense", return_hidden=True)
    tok, hid, cache = _greedy(model, prompt, 16, graph)
    assert torch.equal(tok, ref_tok), f"greedy tokens differ: gpu {tok.tolist()} oracle {ref_tok.tolist()}"
    close(cache.key_cache[0][:, :128], ref_cache.k[0][:, :128], "K cache")
    close(cache.value_cache[0][:, :128], ref_cache.v[0][:, :128], "V cache")
    for s in range(16):
        close(hid[:, s], ref_hid[:, s], f"hidden state at step {s}")


def test_7b_width_layer_teacher_forced_in_float16():
    """One 7B-width layer on the oracle's own layer input: 160 prompt rows (tiled kernels) and one decode token."""
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    mw = O.make_model(d=4096, n_heads=32, n_kv_heads=32, head_dim=128, ffn=11008, attn_rank=1024, mlp_rank=1536,
                      n_layers=1, vocab=1000, dtype=FP16, seed=0)
    model = model_from_oracle(mw)
    T = 160
    ids = torch.randint(0, 1000, (1, T + 1), generator=torch.Generator().manual_seed(1))
    cos, sin = O.rope_tables(T + 8, 128, dtype=FP16)
    x = mw.embed[ids]
    oc = O.DenseCache(mw, 1, T + 8, FP16)
    y_pre = O.block_forward(mw, 0, x[:, :T], 0, oc, cos, sin)
    y_dec = O.block_forward(mw, 0, x[:, T:], T, oc, cos, sin)
    gc = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=T + 8, device="cuda", dtype=FP16)
    layer = model.model.layers[0]
    g_pre = layer(x[:, :T].cuda(), past_key_values=gc, cache_position=torch.arange(T))
    g_dec = layer(x[:, T:].cuda(), past_key_values=gc, cache_position=torch.tensor([T]))
    close(g_pre, y_pre, "prompt rows")
    close(g_dec, y_dec, "decode token")
    close(gc.key_cache[0][:, :T + 1], oc.k[0][:, :T + 1], "K cache")
    close(gc.value_cache[0][:, :T + 1], oc.v[0][:, :T + 1], "V cache")


def _lin_layout(V):   # [heads,R,Dh] -> nn.Linear weight [heads*Dh, R]
    h, r, d = V.shape
    return V.transpose(1, 2).reshape(h * d, r).contiguous()


# the one-kernel form (short caches, 1 / 2 / 4 query heads per kv head, deep and plain) and the three-launch form
# (2^17 (head, key) pairs and more: pair, grouped and single-head score kernels)
@pytest.mark.parametrize("B,H,Hk,L,S,Rk,Rv,nsplit", [(1, 32, 32, 512, 560, 1024, 1024, None), (2, 8, 2, 100, 128, 72, 40, 3),
                                                    (2, 16, 4, 333, 400, 1664, 1664, 4), (2, 8, 4, 700, 720, 136, 264, 2),
                                                    (4, 32, 32, 8200, 8200, 192, 200, 2), (4, 32, 8, 8200, 8200, 128, 64, 3), (12, 3, 3, 4000, 4000, 64, 64, 2)])
def test_rank_space_decode_attention(B, H, Hk, L, S, Rk, Rv, nsplit):
    from flashsvd_amd.kernels import rank_decode as RD
    Dh = 128
    cos, sin = O.rope_tables(S, Dh, dtype=FP16)
    q = rand_fp16(B, H, Dh, seed=1)
    Pk, Pv = rand_fp16(B, S, Rk, seed=2), rand_fp16(B, S, Rv, seed=3)
    Vk, Vv = rand_fp16(Hk, Rk, Dh, std=Rk ** -0.5, seed=4), rand_fp16(Hk, Rv, Dh, std=Rv ** -0.5, seed=5)
    lens = torch.tensor([max(1, min(L, S) - 17 * b) for b in range(B)], dtype=torch.int32)
    out = RD.rank_decode(q.cuda(), Pk.cuda(), Pv.cuda(), _lin_layout(Vk).cuda(), _lin_layout(Vv).cuda(), cos.cuda(), sin.cuda(),
                         lens.cuda(), num_kv_heads=Hk, nsplit=nsplit)
    for b in (0, B - 1):
        n = int(lens[b])
        close(out[b:b + 1], O.rank_decode_attn(q[b:b + 1], Pk[b:b + 1, :n], Pv[b:b + 1, :n], Vk, Vv, cos[:n], sin[:n]), f"b={b} n={n}")


def test_model_rank_cache_greedy_in_float16():
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.runtime.cache import FlashSVDLegacySparseKVCache
    mw = O.make_model(d=256, n_heads=2, n_kv_heads=2, head_dim=128, ffn=512, attn_rank=64, mlp_rank=96, n_layers=2,
                      vocab=500, dtype=FP16, seed=5, std=0.05)
    prompt = torch.randint(0, 500, (1, 21), generator=torch.Generator().manual_seed(4))
    n_new = 8
    ref_tok, ref_hid, ref_cache = O.greedy_decode(mw, prompt, n_new, "rank", return_hidden=True)
    model = model_from_oracle(mw)
    cache = FlashSVDLegacySparseKVCache(model.config, max_batch_size=1, max_cache_len=40, device="cuda", dtype=FP16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(21))
    close(cache.key_cache[0][:, :21], ref_cache.pk[0][:, :21], "Pk cache layer 0")
    # the rank path rounds at other points than the oracle's (fp32 K rebuild, V applied in rank space): hidden states
    # are held to three times the float16 bar, tokens are teacher-forced
    assert_close_bf16(out.hidden_states[:, -1], ref_hid[:, 0], "prefill hidden", abs_tol=1.5e-2, rel_tol=7.5e-3)
    same = int(torch.equal(out.logits[:, -1].float().argmax(-1, keepdim=True).cpu(), ref_tok[:, :1]))
    dec = GraphedDecoder(model, cache, 1)
    dec.set_state(ref_tok[:, :1].cuda(), 21)
    for s in range(1, n_new):
        nxt = dec.eager_step().clone().cpu()
        assert_close_bf16(dec.hidden, ref_hid[:, s], f"hidden step {s}", abs_tol=1.5e-2, rel_tol=7.5e-3)
        same += int(torch.equal(nxt, ref_tok[:, s:s + 1]))
        dec.tokens.copy_(ref_tok[:, s:s + 1])
    assert same >= n_new - 1, f"only {same}/{n_new} teacher-forced tokens identical"


def test_generate_text_after_the_float16_cast():
    """The reference's own sequence: cast_model_for_inference(dtype="fp16"), then generate_text (scripts/demo_support/api.py:128-165,
    238-322); the decode driver hands a float16 model to the per-operator engine."""
    from flashsvd_amd import api

    class Tok:
        pad_token_id, eos_token_id, eos_token, pad_token = 0, None, "<eos>", "<pad>"

        def __call__(self, text, return_tensors="pt", add_special_tokens=False):
            return {"input_ids": torch.tensor([[1, 5, 7, 11, 13]], dtype=torch.long)}

        def decode(self, ids, skip_special_tokens=False):
            return " ".join(str(int(i)) for i in ids)

    mw32, _ = O.config_c1(torch.float32)
    mw16 = O.hold_weights_as(mw32, FP16)
    mw16.embed, mw16.norm = mw32.embed.to(FP16), mw32.norm.to(FP16)
    for b16, b32 in zip(mw16.blocks, mw32.blocks):
        b16.ln1, b16.ln2 = b32.ln1.to(FP16), b32.ln2.to(FP16)
    ref = O.greedy_decode(mw16, torch.tensor([[1, 5, 7, 11, 13]]), 6)
    model = api.cast_model_for_inference(model_from_oracle(mw32), dtype="fp16", device="cuda")
    assert next(model.parameters()).dtype == FP16
    api.configure_runtime("flashsvd")
    for graph in (False, True):
        res = api.generate_text(model, Tok(), prompt="x", max_new_tokens=6, device="cuda", use_graph=graph)
        assert res["completion_ids"] == ref[0].tolist()
    out = api.decode_kvcache_eval(model, prompt_len=16, new_tokens=4, warmup=2, batch_size=2)
    assert out["new_tokens"] == 4 and out["decode_tok_s"] > 0 and out["flashsvd_dense_cache"]


@pytest.mark.parametrize("composed", [False, True], ids=["ten_phase", "composed"])
def test_persistent_step_in_float16_teacher_forced_against_oracle(composed):
    """The resident step over a float16 model (every GEMV phase carries FSVD_WBITS_FP16): a 3-layer GQA model of
    head_dim 128, the oracle's tokens fed back, hidden states and logits against the oracle in float16 at the
    multi-layer bound (three times the float16 bar), tokens tie-aware; then free-running against the per-operator
    engine on the same model."""
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import PersistentDecoder
    mw = O.make_model(d=1024, n_heads=8, n_kv_heads=4, head_dim=128, ffn=2048, attn_rank=256, mlp_rank=384,
                      n_layers=3, vocab=2048, dtype=FP16, seed=3)
    prompt = torch.randint(0, 2048, (1, 37), generator=torch.Generator().manual_seed(5))
    n_new, Lp = 12, 37
    model = model_from_oracle(mw)
    ref_tok, ref_hid, _, ref_logits = O.greedy_decode(mw, prompt, n_new, "dense", return_logits=True)

    def prefill():
        cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 4, device="cuda", dtype=FP16)
        out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp))
        return cache, out.logits[:, -1].float().argmax(-1, keepdim=True)

    cache, tok0 = prefill()
    assert int(tok0) == int(ref_tok[0, 0])
    dec = PersistentDecoder(model, cache, composed=composed)
    assert dec.dtype == FP16 and dec.composed == composed and dec.logits.dtype == FP16
    n_equal = 0
    for s_ in range(1, n_new):
        dec.set_state(ref_tok[:, s_ - 1], Lp + s_ - 1)
        dec.step(1)
        g, o = int(dec.tokens()[0]), int(ref_tok[0, s_])
        m = float(ref_hid[:, s_].float().abs().max())
        assert_close_bf16(dec.hidden()[None].cpu(), ref_hid[:, s_], f"hidden state at step {s_}",
                          abs_tol=3 * (5e-3 if m < 2.0 else 2.0 * m * 2.0 ** -10), rel_tol=7.5e-3)
        rl = ref_logits[0, s_].float()
        if g != o:    # only where the oracle itself holds the two candidates within float16 resolution of the hidden states
            assert float(rl[o] - rl[g]) <= 5e-3 * float(rl.abs().max()), f"step {s_}: token {g} vs oracle {o}"
        n_equal += int(g == o)
    assert n_equal >= n_new - 3
    # free-running: the resident step and the per-operator engine from the same prompt
    cache_p, tok_p = prefill()
    pdec = PersistentDecoder(model, cache_p, composed=composed)
    pdec.set_state(tok_p, Lp)
    pdec.step(n_new - 1)
    cache_g, tok_g = prefill()
    gdec = GraphedDecoder(model, cache_g, 1)
    gdec.set_state(tok_g, Lp)
    toks_g = torch.cat([gdec.eager_step().reshape(-1).cpu() for _ in range(n_new - 1)])
    same = int((pdec.tokens().cpu() == toks_g).sum())
    if composed:
        assert same >= n_new - 3, f"composed form: {same}/{n_new - 1} tokens equal to the per-operator engine"
    else:
        assert same == n_new - 1, f"resident step {pdec.tokens().tolist()} vs per-operator engine {toks_g.tolist()}"


def test_persistent_step_refuses_mixed_types():
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import PersistentDecoder
    mw, _ = O.config_c1(FP16)
    model = model_from_oracle(mw)
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="KV cache of the model's type"):
        PersistentDecoder(model, cache)


# ---------------------------------------------------------------------------------------------------------------------
# group-wise int4 factors under float16 activations: the nibble patterns become float16 values 16 + n
# ---------------------------------------------------------------------------------------------------------------------
def _quant(N, K, group, sym=False, seed=0):
    return O.quantize_weight(rand_fp16(N, K, std=0.05, seed=seed).float(), bits=4, group_size=group, sym=sym)


def _ulp_check_f16(got, ref64, what, ulps=1.0):
    """|got - ref| within ``ulps`` float16 steps at the magnitude of each reference value (the step at 1/32 of the largest
    value for anything smaller: fp32 accumulation noise does not shrink with the result)."""
    got, ref = got.double().cpu(), ref64
    floor = float(ref.abs().max()) / 32.0
    step = torch.clamp(ref.abs(), min=floor).log2().floor().exp2() * 2.0 ** -10
    bad = (got - ref).abs() > ulps * step
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} values off by more than {ulps} ulp; worst " \
                                f"{float(((got - ref).abs() / step).max()):.2f} ulp"


@pytest.mark.parametrize("B,N,K,group", [(1, 4096, 1024, 128), (1, 1536, 11008, 128), (3, 1000, 512, 32), (4, 300, 256, -1),
                                         (7, 520, 1024, 128)])
def test_linear_q4(ops, B, N, K, group):
    """Against the module's forward in float16 (weights rounded to float16 first) at the float16 bar, and against the
    un-rounded sum_k x_k * s * (q - z) in float64, which is what the kernel adds up, within one float16 ulp."""
    qw, sc, zr = _quant(N, K, group, seed=N + K)
    x = rand_fp16(B, K, seed=1)
    got = ops.linear_q4(x.cuda(), qw.cuda(), sc.cuda(), zr.cuda(), group_size=group)
    close(got, O.quant_linear(x, qw, sc, zr, group_size=group), f"linear_q4 {B}x{N}x{K} g{group}")
    w64 = O.dequantize_weight(qw, sc, zr, in_features=K, group_size=group, dtype=torch.float64)
    _ulp_check_f16(got, x.double() @ w64.t(), f"linear_q4 closed form {B}x{N}x{K}")


def test_linear_q4_symmetric_bias_norm_residual(ops):
    B, N, K, group = 2, 768, 1024, 128
    qw, sc, zr = _quant(N, K, group, sym=True, seed=5)
    x, bias, res = rand_fp16(B, K, seed=2), rand_fp16(N, seed=3), rand_fp16(B, N, seed=6)
    nw = (1 + rand_fp16(K, std=0.1, seed=4).float()).to(FP16)
    out = torch.zeros(B, 2 * N, dtype=FP16, device="cuda")
    ops.linear_q4(x.cuda(), qw.cuda(), sc.cuda(), zr.cuda(), group_size=group, bias=bias.cuda(), norm_weight=nw.cuda(), eps=1e-5,
                  residual=res.cuda(), out=out[:, N:])
    ref = (res.float() + O.quant_linear(O.rms_norm(x, nw, 1e-5), qw, sc, zr, bias, group_size=group).float()).to(FP16)
    close(out[:, N:], ref, "q4 linear with norm, bias, residual")
    assert float(out[:, :N].abs().max()) == 0.0


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("B,D,R", [(1, 11008, 1536), (2, 1376, 256)])
def test_swiglu_q4(ops, mode, B, D, R):
    gq, gs, gz = _quant(D, R, 128, seed=1)
    uq, us, uz = _quant(D, R, 128, seed=2)
    p = rand_fp16(B, 2 * R, seed=3)
    got = ops.swiglu_linear_q4(p.cuda(), (gq.cuda(), gs.cuda(), gz.cuda()), (uq.cuda(), us.cuda(), uz.cuda()), up_off=R,
                               group_size=128, mode=mode)
    wg = O.dequantize_weight(gq, gs, gz, in_features=R, group_size=128, dtype=FP16).float()
    wu = O.dequantize_weight(uq, us, uz, in_features=R, group_size=128, dtype=FP16).float()
    g, u = p[:, :R].float() @ wg.t(), p[:, R:].float() @ wu.t()
    if mode == 0:
        g, u = g.to(FP16), u.to(FP16)
        ref = torch.nn.functional.silu(g.float()).to(FP16) * u
    else:
        ref = ((g * torch.sigmoid(g)) * u).to(FP16)
    close(got, ref, f"swiglu_q4 mode {mode}")


def test_dequant_q4_is_bit_exact_in_float16(ops):
    for N, K, group in ((64, 1024, 128), (33, 200, 40), (5, 7, -1), (16, 96, 32)):
        qw, sc, zr = _quant(N, K, group, seed=K)
        got = ops.dequant_q4(qw.cuda(), sc.cuda(), zr.cuda(), in_features=K, group_size=group, dtype=FP16)
        assert got.dtype == FP16
        assert torch.equal(got.cpu(), O.dequantize_weight(qw, sc, zr, in_features=K, group_size=group, dtype=FP16)), (N, K, group)
    with pytest.raises(ValueError, match="bfloat16 or torch.float16"):
        ops.dequant_q4(qw.cuda(), sc.cuda(), zr.cuda(), in_features=K, group_size=group, dtype=torch.float32)


def test_quantized_float16_model_decodes_like_the_oracle_on_dequantized_weights(monkeypatch):
    """Every factor linear of a small float16 model quantised to int4: prompt pass and teacher-forced decode through the
    per-operator path and through the resident step (phases with FSVD_WBITS_Q4_FP16) against the oracle on the
    dequantised float16 weights, at the multi-layer bound."""
    from flashsvd_amd import _lib
    from flashsvd_amd import quant as Q
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import PersistentDecoder, make_persistent_decoder
    mw = O.make_model(d=1024, n_heads=8, n_kv_heads=4, head_dim=128, ffn=2048, attn_rank=256, mlp_rank=512,
                      n_layers=2, vocab=2048, dtype=FP16, seed=7)
    model = model_from_oracle(mw)
    n = Q.replace_linears_with_packed_quant_inplace(model, module_names=Q.factor_linear_names(model), bits=4, group_size=128, sym=False)
    assert n == 28
    for blk, layer in zip(mw.blocks, model.model.layers):
        for name in ("q", "k", "v", "o"):
            for f in ("u", "v"):
                setattr(blk, f"{name}_{f}", getattr(layer.self_attn, f"{name}_{f}_proj").dequantize(dtype=FP16).cpu())
        for name in ("gate", "up", "down"):
            for f in ("u", "v"):
                setattr(blk, f"{name}_{f}", getattr(layer.mlp, f"{name}_{f}_proj").dequantize(dtype=FP16).cpu())
    prompt = torch.randint(0, 2048, (1, 19), generator=torch.Generator().manual_seed(8))
    n_new, Lp = 6, 19
    ref_tok, ref_hid, _ = O.greedy_decode(mw, prompt, n_new, "dense", return_hidden=True)

    def bar(r):
        m = float(r.abs().max())
        return dict(abs_tol=3 * (5e-3 if m < 2.0 else 2.0 * m * 2.0 ** -10), rel_tol=7.5e-3)

    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 4, device="cuda", dtype=FP16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp))
    r0 = ref_hid[:, 0].float()
    assert out.hidden_states.dtype == FP16
    assert_close_bf16(out.hidden_states[:, -1], r0, "prompt pass hidden state", **bar(r0))
    for s in range(1, n_new):
        pos = torch.full((1,), Lp + s - 1, dtype=torch.int32, device="cuda")
        _, h = model.decode_step(ref_tok[:, s - 1:s].cuda(), cache, pos, return_hidden=True)
        r = ref_hid[:, s].float()
        assert_close_bf16(h, r, f"decode hidden state {s}", **bar(r))
    monkeypatch.setenv("FLASHSVD_AMD_DECODE_ENGINE", "auto")
    cache2 = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 4, device="cuda", dtype=FP16)
    model(prompt.cuda(), past_key_values=cache2, cache_position=torch.arange(Lp))
    dec = make_persistent_decoder(model, cache2, 1)
    assert isinstance(dec, PersistentDecoder) and dec.dtype == FP16
    wb = {int(ph.wbits) for ph in dec.host_phases if int(ph.type) == 1}
    assert wb == {_lib.WBITS_Q4_FP16, _lib.WBITS_FP16}, wb
    for s in range(1, n_new):
        dec.set_state(ref_tok[:, s - 1], Lp + s - 1)
        dec.step(1)
        dec.check()
        r = ref_hid[:, s].float()
        assert_close_bf16(dec.hidden()[None].cpu(), r, f"resident step, hidden state {s}", **bar(r))
    kb = bar(cache.key_cache[1].float().cpu())
    assert_close_bf16(cache2.key_cache[1][:, :Lp + n_new - 1], cache.key_cache[1][:, :Lp + n_new - 1].cpu(),
                      "K rows of layer 1 vs the per-operator path", **kb)
