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
