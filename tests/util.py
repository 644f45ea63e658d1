"""Helpers shared by the GPU parity tests."""
import torch

ABS_TOL = 2e-2   # max-abs tolerance on bf16 outputs (the acceptance bar of the decode path)
REL_TOL = 1e-2   # max |a-b| / max |ref|


def rand_bf16(*shape, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


def assert_close_bf16(got, ref, what="", abs_tol=ABS_TOL, rel_tol=REL_TOL):
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = (got - ref).abs().max().item()
    scale = ref.abs().max().item()
    rel = err / max(scale, 1e-30)
    assert err <= abs_tol and rel <= rel_tol, f"{what}: max-abs {err:.4g} (tol {abs_tol}) max-rel {rel:.4g} (tol {rel_tol})"
    return err, rel


def load_oracle_weights(model, mw, device="cuda"):
    """Copy an oracle ModelWeights (CPU, seeded) into a flashsvd_amd SVDLlamaForCausalLM on ``device``."""
    from flashsvd_amd import llama
    model = llama.materialize(model, device, mw.embed.dtype)
    with torch.no_grad():
        model.model.embed_tokens.weight.copy_(mw.embed)
        model.lm_head.weight.copy_(mw.lm_head)
        model.model.norm.weight.copy_(mw.norm)
        for layer, b in zip(model.model.layers, mw.blocks):
            a, m = layer.self_attn, layer.mlp
            for name in ("q", "k", "v", "o"):
                getattr(a, f"{name}_v_proj").weight.copy_(getattr(b, f"{name}_v"))
                getattr(a, f"{name}_u_proj").weight.copy_(getattr(b, f"{name}_u"))
            for name in ("gate", "up", "down"):
                getattr(m, f"{name}_v_proj").weight.copy_(getattr(b, f"{name}_v"))
                getattr(m, f"{name}_u_proj").weight.copy_(getattr(b, f"{name}_u"))
            layer.input_layernorm.weight.copy_(b.ln1)
            layer.post_attention_layernorm.weight.copy_(b.ln2)
    return model


def model_from_oracle(mw, device="cuda"):
    from flashsvd_amd import llama
    meta = mw.meta
    model = llama.build_model(hidden_size=meta["d"], num_heads=mw.n_heads, num_kv_heads=mw.n_kv_heads,
                              head_dim=mw.head_dim, intermediate_size=meta["ffn"], num_layers=meta["n_layers"],
                              vocab_size=meta["vocab"], attn_rank=meta["attn_rank"], mlp_rank=meta["mlp_rank"],
                              rope_theta=mw.rope_theta, rms_norm_eps=mw.eps)
    return load_oracle_weights(model, mw, device)


def bounds(ref):
    """(abs_tol, rel_tol): 2e-2 / 1e-2, except that where max|ref| >= 2 one bf16 ulp already exceeds
    1.5e-2, so the absolute bound becomes two ulps at max|ref|."""
    m = float(ref.float().abs().max())
    return dict(abs_tol=2e-2 if m < 2.0 else 2.0 * m * 2.0 ** -7, rel_tol=1e-2)
