#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ from the CPU oracle (oracle/flashsvd_oracle.py).

The reference checkout holds no golden vectors for this path (its checks are print-only GPU
scripts), so these fixtures pin the oracle's own outputs: they catch a later change of the
oracle, of the seeded weight generation or of the GPU kernels against numbers that no longer
depend on either.  Header of every file: what was drawn, in which order, with which seed.

    python tests/golden/make_fixtures.py        # rewrites config1_*.npz and kernels_small.npz
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import flashsvd_oracle as O  # noqa: E402

OUT = Path(__file__).resolve().parent
HEADER = ("weights: oracle.make_model draw order under torch.Generator().manual_seed(0): embed; per layer q_v,q_u,k_v,"
          "k_u,v_v,v_u,o_v,o_u,gate_v,gate_u,up_v,up_u,down_v,down_u; lm_head (separate, untied); N(0,0.02) fp32 then "
          "cast; RMSNorm weights 1, final norm present, eps 1e-6, rope theta 10000. prompt: 128 ids from "
          "torch.randint(0,32000) under manual_seed(1). greedy: prefill token + 15 decode forwards.")


def f32(t):
    return t.detach().float().numpy()


def config1(dtype, name):
    mw, prompt = O.config_c1(dtype)
    tok, hid, cache, logits = O.greedy_decode(mw, prompt, 16, "dense", return_logits=True)
    top2 = logits.float().topk(2, dim=-1).values
    np.savez_compressed(OUT / name, header=np.array(HEADER), prompt=prompt.numpy(), tokens=tok.numpy(), hidden_last=f32(hid[0]),
                        logit_top2=f32(top2[0]), k_cache_rows=f32(cache.k[0][0, [0, 64, 127, 130]]),
                        v_cache_rows=f32(cache.v[0][0, [0, 64, 127, 130]]))


def kernels_small():
    g = torch.Generator().manual_seed(42)

    def rn(*s, std=1.0):
        return (torch.randn(*s, generator=g) * std).to(torch.bfloat16)
    d = {}
    # dual-split MLP, reference operand layouts
    PUp, PGate = rn(2, 1, 24), rn(2, 1, 24)
    GateU, UpU, DownV, DownU, b2 = rn(24, 80, std=0.2), rn(24, 80, std=0.2), rn(80, 24, std=0.2), rn(24, 32, std=0.2), rn(32, std=0.1)
    for k, v in dict(PUp=PUp, PGate=PGate, GateU=GateU, UpU=UpU, DownV=DownV, DownU=DownU, b2=b2).items():
        d["mlp_" + k] = f32(v)
    d["mlp_Y_v2"] = f32(O.dual_split_mlp(PUp, PGate, GateU, UpU, DownV, DownU, b2))
    d["mlp_Y_v3"] = f32(O.dual_split_mlp_v3(PUp, PGate, GateU, UpU, DownV, DownU, b2, BD=128, BR2=24))
    # reconstruct, shared coefficients, hetero ranks
    Pq, Pk, Pv = rn(2, 16), rn(2, 24), rn(2, 8)
    Vq, Vk, Vv = rn(4, 16, 64, std=0.2), rn(2, 24, 64, std=0.2), rn(2, 8, 64, std=0.2)
    Q, K, V = O.reconstruct_qkv_token_shared_hetero(Pq, Pk, Pv, Vq, Vk, Vv)
    for k, v in dict(Pq=Pq, Pk=Pk, Pv=Pv, Vq=Vq, Vk=Vk, Vv=Vv, Q=Q, K=K, V=V).items():
        d["rec_" + k] = f32(v)
    # rank-space decode, head_dim 128
    cos, sin = O.rope_tables(40, 128, dtype=torch.bfloat16)
    q, Pkc, Pvc = rn(1, 4, 128), rn(1, 40, 16), rn(1, 40, 16)
    Bk, Bv = rn(2, 16, 128, std=0.25), rn(2, 16, 128, std=0.25)
    out = O.rank_decode_attn(q, Pkc[:, :33], Pvc[:, :33], Bk, Bv, cos[:33], sin[:33])
    for k, v in dict(q=q, Pk=Pkc, Pv=Pvc, Vk=Bk, Vv=Bv, out=out).items():
        d["rank_" + k] = f32(v)
    d["header"] = np.array("bf16 values stored as float32; torch.Generator().manual_seed(42), drawn in the order of this file's code")
    np.savez_compressed(OUT / "kernels_small.npz", **d)


if __name__ == "__main__":
    config1(torch.float32, "config1_fp32.npz")
    config1(torch.bfloat16, "config1_bf16.npz")
    kernels_small()
    for f in sorted(OUT.glob("*.npz")):
        print(f.name, f.stat().st_size, "bytes")
