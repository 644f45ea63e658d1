"""Group-wise int4 projections (fsvd_linear_q4, fsvd_swiglu_linear_q4, fsvd_dequant_q4) against the CPU oracle.

Two comparisons per case: the oracle's module forward (weights rounded to bf16 before the product, the reference's
own arithmetic) within the decode path's tolerance, and the un-rounded closed form sum_k x_k * s * (q - z) in float64,
which is what the kernel adds up, within one bf16 ulp."""
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, rand_bf16

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _quant(N, K, group, sym=False, seed=0):
    w = rand_bf16(N, K, std=0.05, seed=seed).float()
    return O.quantize_weight(w, bits=4, group_size=group, sym=sym)


def _closed_form(x, qw, sc, zr, group, K):
    w = O.dequantize_weight(qw, sc, zr, in_features=K, group_size=group, dtype=torch.float64)
    return x.double() @ w.t()


def _ulp_check(got, ref64, what, ulps=1.0):
    """|got - ref| within ``ulps`` bf16 steps at the magnitude of each reference value; values below 1/32 of the
    largest one are held to the step at that floor instead (fp32 accumulation noise does not shrink with the result)."""
    got, ref = got.double().cpu(), ref64
    floor = float(ref.abs().max()) / 32.0
    step = torch.clamp(ref.abs(), min=floor).log2().floor().exp2() * 2.0 ** -7
    bad = (got - ref).abs() > ulps * step
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} values off by more than {ulps} ulp; worst " \
                                f"{float(((got - ref).abs() / step).max()):.2f} ulp"


@pytest.mark.parametrize("B,N,K,group", [(1, 4096, 1024, 128), (1, 1024, 4096, 128), (1, 1536, 11008, 128), (3, 1000, 512, 32),
                                         (4, 300, 256, -1), (1, 4096, 1536, 64), (2, 8, 768, 256), (7, 520, 1024, 128)])
def test_linear_q4(B, N, K, group):
    from flashsvd_amd import hip_ops
    qw, sc, zr = _quant(N, K, group, seed=N + K)
    x = rand_bf16(B, K, seed=1)
    got = hip_ops.linear_q4(x.cuda(), qw.cuda(), sc.cuda(), zr.cuda(), group_size=group)
    ref = O.quant_linear(x, qw, sc, zr, group_size=group)
    assert_close_bf16(got, ref, f"linear_q4 {B}x{N}x{K} g{group}", **bounds(ref))
    _ulp_check(got, _closed_form(x, qw, sc, zr, group, K), f"linear_q4 closed form {B}x{N}x{K}")


def test_linear_q4_symmetric_bias_norm_residual_strided_out():
    from flashsvd_amd import hip_ops
    B, N, K, group = 2, 768, 1024, 128
    qw, sc, zr = _quant(N, K, group, sym=True, seed=5)
    assert int(zr.min()) == int(zr.max()) == 8
    x, bias, nw, res = rand_bf16(B, K, seed=2), rand_bf16(N, seed=3), (1 + rand_bf16(K, std=0.1, seed=4).float()).to(BF16), rand_bf16(B, N, seed=6)
    out = torch.zeros(B, 2 * N, dtype=BF16, device="cuda")
    hip_ops.linear_q4(x.cuda(), qw.cuda(), sc.cuda(), zr.cuda(), group_size=group, bias=bias.cuda(), norm_weight=nw.cuda(), eps=1e-5,
                      residual=res.cuda(), out=out[:, N:])
    xn = O.rms_norm(x, nw, 1e-5)
    ref = (res.float() + O.quant_linear(xn, qw, sc, zr, bias, group_size=group).float()).to(BF16)
    assert_close_bf16(out[:, N:], ref, "q4 linear with norm, bias, residual", **bounds(ref))
    assert float(out[:, :N].abs().max()) == 0.0                               # the other half of the buffer is untouched


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("B,D,R", [(1, 11008, 1536), (2, 1376, 256)])
def test_swiglu_q4(mode, B, D, R):
    from flashsvd_amd import hip_ops
    gq, gs, gz = _quant(D, R, 128, seed=1)
    uq, us, uz = _quant(D, R, 128, seed=2)
    p = rand_bf16(B, 2 * R, seed=3)
    got = hip_ops.swiglu_linear_q4(p.cuda(), (gq.cuda(), gs.cuda(), gz.cuda()), (uq.cuda(), us.cuda(), uz.cuda()), up_off=R,
                                   group_size=128, mode=mode)
    wg = O.dequantize_weight(gq, gs, gz, in_features=R, group_size=128, dtype=BF16).float()
    wu = O.dequantize_weight(uq, us, uz, in_features=R, group_size=128, dtype=BF16).float()
    g, u = p[:, :R].float() @ wg.t(), p[:, R:].float() @ wu.t()
    if mode == 0:
        g, u = g.to(BF16), u.to(BF16)
        ref = (torch.nn.functional.silu(g) * u)
    else:
        ref = ((g * torch.sigmoid(g)) * u).to(BF16)
    assert_close_bf16(got, ref, f"swiglu_q4 mode {mode}", **bounds(ref))


def test_dequant_q4_is_bit_exact():
    from flashsvd_amd import hip_ops
    for N, K, group in ((64, 1024, 128), (33, 200, 40), (5, 7, -1), (16, 96, 32)):
        qw, sc, zr = _quant(N, K, group, seed=K)
        got = hip_ops.dequant_q4(qw.cuda(), sc.cuda(), zr.cuda(), in_features=K, group_size=group)
        ref = O.dequantize_weight(qw, sc, zr, in_features=K, group_size=group, dtype=BF16)
        assert torch.equal(got.cpu(), ref), (N, K, group)


def test_q4_argument_checks():
    from flashsvd_amd import hip_ops
    from flashsvd_amd._lib import FlashSVDHipError
    qw, sc, zr = _quant(16, 384, 128)
    with pytest.raises(FlashSVDHipError, match="multiple of 256"):
        hip_ops.linear_q4(rand_bf16(1, 384).cuda(), qw.cuda(), sc.cuda(), zr.cuda(), group_size=128)
    qw, sc, zr = _quant(16, 512, 96)
    with pytest.raises(FlashSVDHipError, match="power of two"):
        hip_ops.linear_q4(rand_bf16(1, 512).cuda(), qw.cuda(), sc.cuda(), zr.cuda(), group_size=96)
    qw, sc, zr = _quant(16, 512, 128)
    with pytest.raises(TypeError, match="uint8 weights"):
        hip_ops.linear_q4(rand_bf16(1, 512).cuda(), qw.cuda().to(torch.int8), sc.cuda(), zr.cuda(), group_size=128)
    with pytest.raises(ValueError, match="scales / zeros"):
        hip_ops.linear_q4(rand_bf16(1, 512).cuda(), qw.cuda(), sc.cuda()[:, :2], zr.cuda()[:, :2], group_size=128)


def test_quantized_model_decodes_like_the_oracle_on_dequantized_weights(monkeypatch):
    """Every factor linear of a small model quantised to int4: prefill + teacher-forced decode through the per-kernel
    path and through the persistent step against the oracle run on the dequantised (bf16) weights."""
    from flashsvd_amd import quant as Q
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import PersistentDecoder, make_persistent_decoder
    from tests.util import model_from_oracle
    mw = O.make_model(d=1024, n_heads=8, n_kv_heads=4, head_dim=128, ffn=2048, attn_rank=256, mlp_rank=512,
                      n_layers=2, vocab=2048, dtype=BF16, seed=7)
    model = model_from_oracle(mw)
    n = Q.replace_linears_with_packed_quant_inplace(model, module_names=Q.factor_linear_names(model), bits=4, group_size=128, sym=False)
    assert n == 28
    for blk, layer in zip(mw.blocks, model.model.layers):                      # the oracle gets the dequantised factors
        for name in ("q", "k", "v", "o"):
            for f in ("u", "v"):
                setattr(blk, f"{name}_{f}", getattr(layer.self_attn, f"{name}_{f}_proj").dequantize(dtype=BF16).cpu())
        for name in ("gate", "up", "down"):
            for f in ("u", "v"):
                setattr(blk, f"{name}_{f}", getattr(layer.mlp, f"{name}_{f}_proj").dequantize(dtype=BF16).cpu())
    prompt = torch.randint(0, 2048, (1, 19), generator=torch.Generator().manual_seed(8))
    n_new, Lp = 6, 19
    ref_tok, ref_hid, _ = O.greedy_decode(mw, prompt, n_new, "dense", return_hidden=True)
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 4, device="cuda", dtype=BF16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp))
    r0 = ref_hid[:, 0].float()
    assert_close_bf16(out.hidden_states[:, -1], r0, "prefill hidden state", abs_tol=3 * bounds(r0)["abs_tol"], rel_tol=3e-2)
    for s in range(1, n_new):
        pos = torch.full((1,), Lp + s - 1, dtype=torch.int32, device="cuda")
        _, h = model.decode_step(ref_tok[:, s - 1:s].cuda(), cache, pos, return_hidden=True)
        r = ref_hid[:, s].float()
        assert_close_bf16(h, r, f"decode hidden state {s}", abs_tol=3 * bounds(r)["abs_tol"], rel_tol=3e-2)
    # the persistent step streams the same int4 factors (phases with wbits == 4): teacher-forced against the same oracle,
    # and against the per-kernel path on the hidden state of every step
    monkeypatch.setenv("FLASHSVD_AMD_DECODE_ENGINE", "auto")
    cache2 = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 4, device="cuda", dtype=BF16)
    model(prompt.cuda(), past_key_values=cache2, cache_position=torch.arange(Lp))
    dec = make_persistent_decoder(model, cache2, 1)
    assert isinstance(dec, PersistentDecoder)
    assert any(int(ph.wbits) == 4 for ph in dec.host_phases)
    for s in range(1, n_new):
        dec.set_state(ref_tok[:, s - 1], Lp + s - 1)
        dec.step(1)
        dec.check()
        r = ref_hid[:, s].float()
        assert_close_bf16(dec.hidden()[None].cpu(), r, f"persistent step, hidden state {s}", abs_tol=3 * bounds(r)["abs_tol"], rel_tol=3e-2)
    assert_close_bf16(cache2.key_cache[1][:, :Lp + n_new - 1], cache.key_cache[1][:, :Lp + n_new - 1].cpu(), "K rows of layer 1 vs the per-kernel path",
                      abs_tol=3 * bounds(cache.key_cache[1].float().cpu())["abs_tol"], rel_tol=3e-2)


def test_persistent_step_rejects_int4_layers_it_cannot_stream():
    """A layer that mixes int4 and bf16 factors is refused at construction (the driver then takes the per-kernel engine)."""
    from flashsvd_amd import quant as Q
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import PersistentDecoder
    from tests.util import model_from_oracle
    mw = O.make_model(d=1024, n_heads=8, n_kv_heads=4, head_dim=128, ffn=2048, attn_rank=256, mlp_rank=512,
                      n_layers=1, vocab=2048, dtype=BF16, seed=7)
    model = model_from_oracle(mw)
    names = [n for n in Q.factor_linear_names(model) if "down_u_proj" not in n]
    Q.replace_linears_with_packed_quant_inplace(model, module_names=names, bits=4, group_size=128, sym=False)
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=32, device="cuda", dtype=BF16)
    with pytest.raises(ValueError, match="mixes int4"):
        PersistentDecoder(model, cache)
