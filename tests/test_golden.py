"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py).
CPU: the oracle still reproduces them.  GPU: the HIP path is checked against the stored numbers
directly, with no oracle in the loop."""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds

G = Path(__file__).resolve().parent / "golden"
BF16 = torch.bfloat16


def _load(name):
    return np.load(G / name, allow_pickle=False)


@pytest.mark.parametrize("dtype,name", [(torch.float32, "config1_fp32.npz"), (BF16, "config1_bf16.npz")])
def test_oracle_reproduces_config1(dtype, name):
    z = _load(name)
    mw, prompt = O.config_c1(dtype)
    assert np.array_equal(prompt.numpy(), z["prompt"])
    tok, hid, cache, logits = O.greedy_decode(mw, prompt, 16, "dense", return_logits=True)
    margins = z["logit_top2"][:, 0] - z["logit_top2"][:, 1]
    # tokens must match wherever the stored top-2 margin is not a near-tie for this dtype
    eps = 1e-4 if dtype == torch.float32 else 2e-2
    for s in range(16):
        if margins[s] > eps:
            assert int(tok[0, s]) == int(z["tokens"][0, s]), f"token {s}"
        else:
            break   # later steps were generated after a near-tie
    tol = dict(atol=2e-4, rtol=1e-3) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    assert np.allclose(hid[0, :1].float().numpy(), z["hidden_last"][:1], **tol)
    assert np.allclose(cache.k[0][0, [0, 64, 127]].float().numpy(), z["k_cache_rows"][:3], **tol)


def test_oracle_reproduces_small_kernels():
    z = _load("kernels_small.npz")
    t = lambda k: torch.from_numpy(z[k]).to(BF16)
    y = O.dual_split_mlp(t("mlp_PUp"), t("mlp_PGate"), t("mlp_GateU"), t("mlp_UpU"), t("mlp_DownV"), t("mlp_DownU"), t("mlp_b2"))
    assert np.allclose(y.float().numpy(), z["mlp_Y_v2"], atol=2e-2, rtol=1e-2)
    Q, K, V = O.reconstruct_qkv_token_shared_hetero(t("rec_Pq"), t("rec_Pk"), t("rec_Pv"), t("rec_Vq"), t("rec_Vk"), t("rec_Vv"))
    assert np.allclose(K.float().numpy(), z["rec_K"], atol=2e-2, rtol=1e-2)


@pytest.mark.gpu
def test_gpu_matches_config1_bf16_fixture():
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from tests.util import model_from_oracle
    z = _load("config1_bf16.npz")
    mw, prompt = O.config_c1(BF16)      # only the seeded weights come from here, no oracle compute
    model = model_from_oracle(mw)
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=150, device="cuda", dtype=BF16)
    out = model(torch.from_numpy(z["prompt"]).cuda(), past_key_values=cache, cache_position=torch.arange(128))
    tok = out.logits[:, -1].float().argmax(-1, keepdim=True)
    toks, hid = [int(tok)], [out.hidden_states[0, -1].float().cpu()]
    dec = GraphedDecoder(model, cache, 1)
    dec.set_state(tok, 128)
    dec.capture()
    for _ in range(15):
        toks.append(int(dec.step()))
        hid.append(dec.hidden[0].float().cpu())
    assert toks == z["tokens"][0].tolist()
    for s in range(16):
        assert_close_bf16(hid[s], torch.from_numpy(z["hidden_last"][s]), f"hidden {s}")
    assert_close_bf16(cache.key_cache[0][0, [0, 64, 127, 130]], torch.from_numpy(z["k_cache_rows"]), "K rows")
    assert_close_bf16(cache.value_cache[0][0, [0, 64, 127, 130]], torch.from_numpy(z["v_cache_rows"]), "V rows")


@pytest.mark.gpu
def test_gpu_matches_small_kernel_fixtures():
    import flashsvd_amd.kernels as K
    from flashsvd_amd.kernels import rank_decode as RD
    z = _load("kernels_small.npz")
    t = lambda k: torch.from_numpy(z[k]).to(BF16).cuda()
    args = [t("mlp_" + k) for k in ("PUp", "PGate", "GateU", "UpU", "DownV", "DownU", "b2")]
    for fn, key in ((K.flashsvd_mlp_dual_split_triton_v2, "mlp_Y_v2"), (K.flashsvd_mlp_dual_split_triton_v3, "mlp_Y_v3")):
        ref = torch.from_numpy(z[key])
        assert_close_bf16(fn(*args), ref, key, **bounds(ref))
    Q, Kk, V = K.reconstruct_qkv_token_shared_hetero(*[t("rec_" + k) for k in ("Pq", "Pk", "Pv", "Vq", "Vk", "Vv")])
    for got, key in ((Q, "rec_Q"), (Kk, "rec_K"), (V, "rec_V")):
        ref = torch.from_numpy(z[key])
        assert_close_bf16(got, ref, key, **bounds(ref))
    cos, sin = O.rope_tables(40, 128, dtype=BF16)
    lin = lambda Vb: Vb.transpose(1, 2).reshape(-1, Vb.shape[1]).contiguous()
    out = RD.rank_decode(t("rank_q"), t("rank_Pk"), t("rank_Pv"), lin(t("rank_Vk")), lin(t("rank_Vv")), cos.cuda(), sin.cuda(),
                         torch.tensor([33], dtype=torch.int32).cuda(), num_kv_heads=2)
    ref = torch.from_numpy(z["rank_out"])
    assert_close_bf16(out, ref, "rank decode", **bounds(ref))
