#!/usr/bin/env python3
"""Decode benchmark of the low-rank Llama path on one MI355X.

Workload (the configuration the headline metric is quoted on): a 32-layer Llama-2-7B-shaped
low-rank model (d 4096, 32x128 heads, ffn 11008, attention rank 1024, MLP rank 1536, vocab
32000, ~0.5 parameter ratio), bf16, random-init factors N(0, 0.02), batch 1, random-token prompt
of 512, greedy decode with the whole step captured as one HIP graph.

A "step" is one decoded token (one graph replay).  Protocol follows the reference's
decode_kvcache_eval (utils/evaluator.py:486-522): prefill, W untimed warm-up tokens, then exactly
K timed tokens between two device synchronisations.

Prints ONE JSON line.  `roofline` describes the dominant kernel (gate/up u-projection + SwiGLU,
67.6 MB of factor bytes per launch), timed live with events around graph replays that launch it
once per layer over all 32 layers' weights.  `cpu_baseline` is the CPU oracle (fp32, the reference's
CPU precision) timed on this host on a 2-layer sample and scaled to 32 layers.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

CFG = dict(hidden_size=4096, num_heads=32, num_kv_heads=32, head_dim=128, intermediate_size=11008,
           num_layers=32, vocab_size=32000, attn_rank=1024, mlp_rank=1536)
PROMPT_LEN = 512
HBM_PEAK_GBS = 8000.0


def _parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=CFG["num_layers"], help="debug only: fewer layers => INVALID as a headline number")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense bf16 comparator leg")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--kernel-breakdown", action="store_true", help="also time every kernel type of the step")
    ap.add_argument("--no-composed", dest="composed", action="store_false",
                    help="skip the leg that times the persistent step in its composed form (rank projections folded into the "
                         "u-factor phases, products with the hidden state streamed as leading phases); the form is opt-in in the "
                         "library (FLASHSVD_AMD_STEP_COMPOSED=1) because it moves rounding points, and is never the headline value")
    ap.add_argument("--composed", dest="composed", action="store_true", help=argparse.SUPPRESS)   # the old spelling; now the default
    ap.add_argument("--no-stress", action="store_true", help="skip the stress configuration's whole-model pass in the default line")
    ap.add_argument("--no-kernel-configs", action="store_true",
                    help="skip the kernel-level configurations (for profiler runs: their launches share kernel names with the step's)")
    ap.add_argument("--kernel-configs-only", action="store_true",
                    help="only the kernel-level configurations (attention block, MLP at 1 / 8 / 32 rows): the run to trace per kernel")
    ap.add_argument("--engine", choices=["persistent", "graph", "both"], default="both",
                    help="persistent: one resident kernel per token (fsvd_decode_step); graph: one HIP graph of the "
                         "per-operator kernels per token; both: time both, the headline value is the persistent step")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only time the prompt pass (matrix-core kernels): W untimed and K timed passes over a 512-token prompt")
    ap.add_argument("--stress", action="store_true",
                    help="time the attention kernels of the stress configuration per layer (attention rank 1664: rank-space decode "
                         "at batch 16 x context 4096, prompt attention path at 8 x 2048) and print their own JSON line")
    ap.add_argument("--quant", action="store_true",
                    help="the same model with every factor quantised to group-wise int4 (group 128): decode tok/s of both engines "
                         "and the bytes that cross HBM per token, as its own JSON line")
    ap.add_argument("--fp16", action="store_true",
                    help="the same model held in float16: warm prompt pass and decode tok/s of both engines")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 256 MiB device copy 10 times (the known-size kernel that FETCH_SIZE / WRITE_SIZE "
                         "counters are scaled against) and exit")
    return ap.parse_args()


def _median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def time_graph_ms(graph, reps: int, warm: int = 3) -> float:
    """Median over `reps` of the event time of one replay (events on the current stream)."""
    import torch
    for _ in range(warm):
        graph.replay()
    torch.cuda.synchronize()
    out = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1))
    return _median(out)


def per_layer_kernel_us(fn_per_layer, n_layers: int, reps: int = 10) -> float:
    """Capture `fn_per_layer(i)` for i in range(n_layers) (cold weights for every launch) into a
    graph and return the average microseconds per launch, launch gaps included."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n_layers):
            fn_per_layer(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(n_layers):
            fn_per_layer(i)
    # subtract the replay's fixed cost measured on an empty-ish graph of one launch? no: keep it in (conservative)
    return time_graph_ms(g, reps) * 1000.0 / n_layers


def kernel_configs(model, cache, dec, n_layers: int) -> dict:
    """The two kernel-level configurations of the benchmark contract, per CALL (all launches of the block replayed
    from a graph over every layer's cold weights, launch gaps included): one low-rank attention block at the 7B shape
    (rank projection, q/k/v expansion + RoPE + cache append, attention over the cached context, output projection) and
    one low-rank SwiGLU MLP for 1, 8 and 32 rows."""
    import torch
    L = model.model.layers
    d = CFG["hidden_size"]
    out = {}
    x = torch.randn(1, d, device="cuda").to(torch.bfloat16)
    pos = torch.full((1,), PROMPT_LEN, dtype=torch.int32, device="cuda")

    def attn(i):
        n1 = L[i].input_layernorm
        return L[i].self_attn.decode_token(x, cache, pos, norm_weight=n1.weight, eps=n1.variance_epsilon, residual=x,
                                           rope=dec.rope, attn_ws=dec.attn_ws, nsplit=dec.nsplit)
    us = per_layer_kernel_us(attn, n_layers)
    nb = 8 * d * CFG["attn_rank"] * 2 + 2 * PROMPT_LEN * CFG["num_heads"] * CFG["head_dim"] * 2 + 2 * d * 2 * 2
    out["attention_block_bs1_ctx512"] = {"us_per_call": us, "bytes_per_call": nb, "GB/s": nb / us / 1e3, "frac_of_peak": nb / us / 1e3 / HBM_PEAK_GBS}
    # the same block over a rank-space cache (coefficients Pk / Pv of 512 tokens, K and V rebuilt in the kernel)
    from flashsvd_amd.runtime.cache import FlashSVDLegacySparseKVCache
    Ra = CFG["attn_rank"]
    rcache = FlashSVDLegacySparseKVCache(model.config, max_batch_size=1, max_cache_len=PROMPT_LEN + 8, device="cuda", dtype=torch.bfloat16)
    for i in range(n_layers):
        rcache.ensure_layer_ranks(i, Ra, Ra)
        rcache.key_cache[i][:, :PROMPT_LEN].normal_(0.0, 1.0)
        rcache.value_cache[i][:, :PROMPT_LEN].normal_(0.0, 1.0)

    def attn_rank(i):
        n1 = L[i].input_layernorm
        return L[i].self_attn.decode_token(x, rcache, pos, norm_weight=n1.weight, eps=n1.variance_epsilon, residual=x, rope=dec.rope)
    us = per_layer_kernel_us(attn_rank, n_layers)
    nb = 8 * d * Ra * 2 + 2 * PROMPT_LEN * Ra * 2 + 2 * Ra * 2 + 2 * d * 2 * 2
    out["attention_block_bs1_ctx512_rank_kv"] = {"us_per_call": us, "bytes_per_call": nb, "GB/s": nb / us / 1e3, "frac_of_peak": nb / us / 1e3 / HBM_PEAK_GBS,
                                                 "rebuild_GFLOP": 2 * PROMPT_LEN * Ra * CFG["num_kv_heads"] * CFG["head_dim"] / 1e9}
    del rcache
    for B in (1, 8, 32):
        xb = torch.randn(B, d, device="cuda").to(torch.bfloat16)

        def mlp(i, xb=xb):
            n2 = L[i].post_attention_layernorm
            return L[i].mlp.run(xb, norm_weight=n2.weight, eps=n2.variance_epsilon, residual=xb)
        us = per_layer_kernel_us(mlp, n_layers)
        nb = 3 * (d + CFG["intermediate_size"]) * CFG["mlp_rank"] * 2 + B * 2 * d * 2
        out[f"swiglu_mlp_bs{B}"] = {"us_per_call": us, "bytes_per_call": nb, "GB/s": nb / us / 1e3, "frac_of_peak": nb / us / 1e3 / HBM_PEAK_GBS}
    # the same two blocks as short phase lists of the resident step kernel (embedding row -> the block's phases, one launch
    # per call, hand-off between phases inside the kernel): 8 layers' weights in rotation, launches queued back to back
    from flashsvd_amd.step import PersistentDecoder
    nrot = min(8, n_layers)
    nb_attn = out["attention_block_bs1_ctx512"]["bytes_per_call"]
    nb_mlp = out["swiglu_mlp_bs1"]["bytes_per_call"]
    for part, key, nb in (("attention", "attention_block_bs1_ctx512_resident_step", nb_attn), ("mlp", "swiglu_mlp_bs1_resident_step", nb_mlp)):
        decs = [PersistentDecoder(model, cache, part=part, layer=i, max_new_tokens=8) for i in range(nrot)]
        for dd in decs:
            dd.set_state(1234, PROMPT_LEN)
            dd.step(2)
        torch.cuda.synchronize()
        reps = 40
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for dd in decs:
                dd.step(1)
        e1.record()
        torch.cuda.synchronize()
        for dd in decs:
            dd.check()
        us = e0.elapsed_time(e1) * 1e3 / (reps * nrot)
        out[key] = {"us_per_call": us, "bytes_per_call": nb, "GB/s": nb / us / 1e3, "frac_of_peak": nb / us / 1e3 / HBM_PEAK_GBS,
                    "phases": len(decs[0].phase_names())}
        del decs
    # the operators under the reference's own names and operand layouts (x @ W): flashsvd_mlp_dual_split_triton_v2 on
    # PUp / PGate [B,1,R], GateU / UpU [R,D], DownV [D,R], DownU [R,d], and reconstruct_qkv_token_shared on the split of a
    # packed coefficient row and bases [H,R,Dh]; operands of 8 layers in rotation (1.1 GB: nothing comes from a cache)
    from flashsvd_amd.kernels import dual_split as DS, densekv_reconstruct as DR
    nref = min(8, n_layers)
    R, Ra, H, Dh = CFG["mlp_rank"], CFG["attn_rank"], CFG["num_heads"], CFG["head_dim"]
    refw = []
    for i in range(nref):
        m, a = L[i].mlp, L[i].self_attn
        refw.append(dict(GateU=m.gate_u_proj.weight.t().contiguous(), UpU=m.up_u_proj.weight.t().contiguous(),
                         DownV=m.down_v_proj.weight.t().contiguous(), DownU=m.down_u_proj.weight.t().contiguous(),
                         Vq=a.q_u_proj.weight.view(H, Dh, Ra).transpose(1, 2).contiguous(),
                         Vk=a.k_u_proj.weight.view(H, Dh, Ra).transpose(1, 2).contiguous(),
                         Vv=a.v_u_proj.weight.view(H, Dh, Ra).transpose(1, 2).contiguous()))
    twin_note = ("bf16 v2-type calls stream cached nn.Linear-layout twins of GateU / UpU / DownV / DownU (a second copy of each operand, "
                 "built at the first call and kept while the operand lives); the *_xw_kernel entry is the same call on the "
                 "operands as given (x @ W kernel, FLASHSVD_AMD_REFERENCE_LAYOUT_FAST=0)")
    for B in (1, 8):
        pcat = torch.randn(B, 1, 2 * R, device="cuda").to(torch.bfloat16)          # [PGate | PUp] of one rank projection

        def ref_mlp(i, pcat=pcat):
            w = refw[i % nref]
            return DS.flashsvd_mlp_dual_split_triton_v2(pcat[..., R:], pcat[..., :R], w["GateU"], w["UpU"], w["DownV"], w["DownU"])
        nb = 3 * CFG["intermediate_size"] * R * 2 + d * R * 2 + B * (2 * R + d) * 2
        for nm, fast in ((f"reference_layout_mlp_dual_split_v2_bs{B}", "1"), (f"reference_layout_mlp_dual_split_v2_xw_kernel_bs{B}", "0")):
            keep = os.environ.get("FLASHSVD_AMD_REFERENCE_LAYOUT_FAST")
            os.environ["FLASHSVD_AMD_REFERENCE_LAYOUT_FAST"] = fast
            try:
                us = per_layer_kernel_us(ref_mlp, n_layers)
            finally:
                if keep is None:
                    os.environ.pop("FLASHSVD_AMD_REFERENCE_LAYOUT_FAST", None)
                else:
                    os.environ["FLASHSVD_AMD_REFERENCE_LAYOUT_FAST"] = keep
            out[nm] = {"us_per_call": us, "bytes_per_call": nb, "GB/s": nb / us / 1e3, "frac_of_peak": nb / us / 1e3 / HBM_PEAK_GBS,
                       "operands": "cached transposed twins (warm)" if fast == "1" else "as given (x @ W)"}
    out["reference_layout_note"] = twin_note
    packed = torch.randn(1, 3 * Ra, device="cuda").to(torch.bfloat16)

    def ref_rec(i):
        w = refw[i % nref]
        return DR.reconstruct_qkv_token_shared(packed[:, :Ra], packed[:, Ra:2 * Ra], packed[:, 2 * Ra:], w["Vq"], w["Vk"], w["Vv"])
    us = per_layer_kernel_us(ref_rec, n_layers)
    nb = 3 * H * Dh * Ra * 2 + 3 * Ra * 2 + 3 * H * Dh * 2
    out["reference_layout_reconstruct_qkv_token_shared"] = {"us_per_call": us, "bytes_per_call": nb, "GB/s": nb / us / 1e3,
                                                            "frac_of_peak": nb / us / 1e3 / HBM_PEAK_GBS}
    del refw
    # the dense-cache attention kernel alone at a serving shape (batch 16 over 4096 cached tokens, 32 heads): the cache
    # rows are its algorithmic bytes; two caches in rotation (2.1 GB) so that nothing comes from a cache
    from flashsvd_amd import hip_ops
    Bs, ctx, Hk = 16, 4096, CFG["num_kv_heads"]
    kcs = [torch.randn(Bs, ctx + 8, Hk, Dh, device="cuda").to(torch.bfloat16) for _ in range(2)]
    vcs = [torch.randn(Bs, ctx + 8, Hk, Dh, device="cuda").to(torch.bfloat16) for _ in range(2)]
    qb = torch.randn(Bs, H, Dh, device="cuda").to(torch.bfloat16)
    lens = torch.full((Bs,), ctx, dtype=torch.int32, device="cuda")
    ob = torch.empty(Bs, H, Dh, device="cuda", dtype=torch.bfloat16)
    ws = hip_ops.attn_workspace(Bs, H, Dh, 4, "cuda")

    def dense_attn(i):
        return hip_ops.attn_decode_densekv(qb, kcs[i % 2], vcs[i % 2], lens, nsplit=4, workspace=ws, out=ob)
    us = per_layer_kernel_us(dense_attn, 8)
    nb = 2 * Bs * ctx * Hk * Dh * 2
    out["dense_kv_attention_b16_ctx4096"] = {"us_per_call": us, "bytes_per_call": nb, "GB/s": nb / us / 1e3, "frac_of_peak": nb / us / 1e3 / HBM_PEAK_GBS}
    del kcs, vcs
    return out


def kernel_legs(model, cache, dec):
    """name -> (launch closure over layer index, algorithmic bytes per launch)."""
    import torch
    from flashsvd_amd import hip_ops
    L = model.model.layers
    dev = "cuda"
    d, R, Ra, D = CFG["hidden_size"], CFG["mlp_rank"], CFG["attn_rank"], CFG["intermediate_size"]
    H, Dh = CFG["num_heads"], CFG["head_dim"]
    bf = torch.bfloat16
    x = torch.randn(1, d, device=dev).to(bf)
    p_attn = torch.randn(1, 3 * Ra, device=dev).to(bf)
    a_in = torch.randn(1, H * Dh, device=dev).to(bf)
    po = torch.randn(1, Ra, device=dev).to(bf)
    p_mlp = torch.randn(1, 2 * R, device=dev).to(bf)
    h = torch.randn(1, D, device=dev).to(bf)
    s = torch.randn(1, R, device=dev).to(bf)
    q = torch.randn(1, H, Dh, device=dev).to(bf)
    pos = dec.positions
    outs = dict(p_attn=torch.empty_like(p_attn), q=torch.empty_like(q), a=torch.empty(1, H, Dh, device=dev, dtype=bf),
                po=torch.empty_like(po), x=torch.empty_like(x), p_mlp=torch.empty_like(p_mlp), h=torch.empty_like(h),
                s=torch.empty_like(s))
    for l in L:
        l.self_attn._ensure_runtime_state()
        l.mlp._ensure_runtime_state()
    n_ctx = PROMPT_LEN
    legs = {
        "attn_rank_proj(norm+[q_v;k_v;v_v])": (
            lambda i: hip_ops.linear(x, L[i].self_attn._packed_qkv_v, norm_weight=L[i].input_layernorm.weight, out=outs["p_attn"]),
            3 * Ra * d * 2 + d * 2 + 3 * Ra * 2),
        "attn_qkv_u+rope+append": (
            lambda i: hip_ops.qkv_rope_append(p_attn, L[i].self_attn.q_u_proj.weight, L[i].self_attn.k_u_proj.weight,
                                              L[i].self_attn.v_u_proj.weight, dec.rope[0], dec.rope[1], pos,
                                              cache.key_cache[i], cache.value_cache[i], num_heads=H, num_kv_heads=H,
                                              head_dim=Dh, q_out=outs["q"]),
            3 * H * Dh * Ra * 2 + 3 * Ra * 2 + 3 * H * Dh * 2),
        "attn_decode_densekv(L=%d)" % n_ctx: (
            lambda i: hip_ops.attn_decode_densekv(q, cache.key_cache[i], cache.value_cache[i], pos, seqlen_add=1,
                                                  nsplit=dec.nsplit, workspace=dec.attn_ws, out=outs["a"]),
            2 * (n_ctx + 1) * H * Dh * 2 + 2 * H * Dh * 2),
        "attn_o_v": (lambda i: hip_ops.linear(a_in, L[i].self_attn.o_v_proj.weight, out=outs["po"]), Ra * H * Dh * 2 + H * Dh * 2 + Ra * 2),
        "attn_o_u+residual": (lambda i: hip_ops.linear(po, L[i].self_attn.o_u_proj.weight, residual=x, out=outs["x"]), d * Ra * 2 + Ra * 2 + 2 * d * 2),
        "mlp_rank_proj(norm+[gate_v;up_v])": (
            lambda i: hip_ops.linear(x, L[i].mlp._packed_gu_v, norm_weight=L[i].post_attention_layernorm.weight, out=outs["p_mlp"]),
            2 * R * d * 2 + d * 2 + 2 * R * 2),
        "mlp_gate_up_u+swiglu": (
            lambda i: hip_ops.swiglu_linear(p_mlp, L[i].mlp.gate_u_proj.weight, L[i].mlp.up_u_proj.weight, up_off=R, out=outs["h"]),
            2 * D * R * 2 + 2 * R * 2 + D * 2),
        "mlp_down_v": (lambda i: hip_ops.linear(h, L[i].mlp.down_v_proj.weight, out=outs["s"]), R * D * 2 + D * 2 + R * 2),
        "mlp_down_u+residual": (lambda i: hip_ops.linear(s, L[i].mlp.down_u_proj.weight, residual=x, out=outs["x"]), d * R * 2 + R * 2 + 2 * d * 2),
    }
    return legs


def run_lowrank(args, dtype=None):
    import torch
    from flashsvd_amd import llama
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache

    dtype = dtype or torch.bfloat16
    cfg = dict(CFG, num_layers=args.layers)
    model = llama.materialize(llama.build_model(**cfg), "cuda", dtype, seed=0)
    B = 1
    max_len = PROMPT_LEN + args.warmup + args.steps + 8
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=B, max_cache_len=max_len, device="cuda", dtype=dtype)
    prompt = torch.randint(0, cfg["vocab_size"], (B, PROMPT_LEN), generator=torch.Generator().manual_seed(1)).cuda()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = model(prompt, past_key_values=cache, cache_position=torch.arange(PROMPT_LEN), logits_to_keep=1)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    tok = out.logits[:, -1].float().argmax(-1, keepdim=True)
    res = dict(prefill_s=t_prefill)
    # the first pass pays one-time set-up (weight packing, tables, kernel attributes): time warm passes as well
    reps = args.steps if args.prefill_only else 2
    scratch = FlashSVDV15DenseKVCache(model.config, max_batch_size=B, max_cache_len=max_len, device="cuda", dtype=dtype)
    for _ in range(args.warmup if args.prefill_only else 1):
        model(prompt, past_key_values=scratch, cache_position=torch.arange(PROMPT_LEN), logits_to_keep=1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        model(prompt, past_key_values=scratch, cache_position=torch.arange(PROMPT_LEN), logits_to_keep=1)
    torch.cuda.synchronize()
    t_warm = (time.perf_counter() - t0) / reps
    del scratch
    d, D, Ra, Rm, H, Dh = (CFG[k] for k in ("hidden_size", "intermediate_size", "attn_rank", "mlp_rank", "num_heads", "head_dim"))
    proj_flop = 2.0 * PROMPT_LEN * (8 * d * Ra + 3 * (d + D) * Rm)                    # every factor once per token
    attn_flop = 2.0 * 2 * H * Dh * PROMPT_LEN * (PROMPT_LEN + 1) / 2                   # causal QK^T and PV
    flop = args.layers * (proj_flop + attn_flop) + 2.0 * d * CFG["vocab_size"]
    res["prefill"] = dict(prompt_len=PROMPT_LEN, warm_s=t_warm, tok_s=PROMPT_LEN / t_warm, flop=flop,
                          TFLOPs=flop / t_warm / 1e12, frac_of_bf16_mfma_peak=flop / t_warm / 2.5e15, cold_s=t_prefill)
    if args.prefill_only:
        return res
    dec = GraphedDecoder(model, cache, B)
    dec.set_state(tok, PROMPT_LEN)
    if args.kernel_configs_only:
        res["kernel_configs"] = kernel_configs(model, cache, dec, args.layers)
        return res
    if args.engine in ("graph", "both"):
        dec.capture()
        for _ in range(args.warmup):
            dec.step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            dec.step()
        torch.cuda.synchronize()
        t_decode = time.perf_counter() - t1
        res["graph"] = dict(tok_s=B * args.steps / t_decode, ms_per_step=t_decode * 1000.0 / args.steps)
    if args.engine in ("persistent", "both"):
        from flashsvd_amd.step import PersistentDecoder
        cache._seen_tokens = PROMPT_LEN
        pdec = PersistentDecoder(model, cache)
        pdec.set_state(tok, PROMPT_LEN)
        pdec.step(args.warmup)
        pdec.check()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        e0.record()
        pdec.step(args.steps)
        e1.record()
        torch.cuda.synchronize()
        t_decode = time.perf_counter() - t1
        pdec.check()
        res["persistent"] = dict(tok_s=B * args.steps / t_decode, ms_per_step=t_decode * 1000.0 / args.steps,
                                 kernel_us_per_launch=e0.elapsed_time(e1) * 1000.0 / args.steps,
                                 workgroups=pdec.nwg, last_token=int(pdec.tokens()[-1]))
        # where the launch's time goes, from inside the kernel: per phase kind (averaged over layers and 8 workgroups)
        # wait for the input | weight stream | epilogue and publication, microseconds
        prof = pdec.phase_profile(32)
        res["persistent"]["phase_profile_us"] = {k: {m: round(x, 2) for m, x in v.items()} for k, v in prof.items()}
        pdec.check()
        del pdec
        if args.composed:
            # the same step with the rank projections folded into the u-factor phases (PersistentDecoder(composed=True)):
            # eight hand-offs per layer instead of ten, 6 % more bytes; reported beside the default form, never as the headline
            # value (its rank coefficients come from unrounded sums: closer to exact arithmetic, but not the reference's roundings)
            scratch_c = FlashSVDV15DenseKVCache(model.config, max_batch_size=B, max_cache_len=max_len, device="cuda", dtype=dtype)
            model(prompt, past_key_values=scratch_c, cache_position=torch.arange(PROMPT_LEN), logits_to_keep=1)
            cdec = PersistentDecoder(model, scratch_c, composed=True)
            cdec.set_state(tok, PROMPT_LEN)
            cdec.step(args.warmup)
            cdec.check()
            torch.cuda.synchronize()
            e0.record()
            cdec.step(args.steps)
            e1.record()
            torch.cuda.synchronize()
            cdec.check()
            us_c = e0.elapsed_time(e1) * 1000.0 / args.steps
            prof = cdec.phase_profile(32)
            res["persistent_composed"] = dict(tok_s=1e6 / us_c, kernel_us_per_launch=us_c, phases=cdec.nph, leading_phases=bool(cdec.leading),
                                              traffic=_traffic("decode_step_kernel_composed"),   # measured HBM bytes per launch (1.08x the token's algorithmic bytes: the composed blocks)
                                              last_token=int(cdec.tokens()[-1]),
                                              phase_profile_us={k: {m: round(x, 2) for m, x in v.items()} for k, v in prof.items()})
            del cdec, scratch_c
    best = res.get("persistent") or res["graph"]
    res["tok_s"], res["ms_per_step"] = best["tok_s"], best["ms_per_step"]
    if dtype != torch.bfloat16:
        return res
    if not args.no_kernel_configs:
        res["kernel_configs"] = kernel_configs(model, cache, dec, args.layers)
    legs = kernel_legs(model, cache, dec)
    name = "mlp_gate_up_u+swiglu"
    fn, nbytes = legs[name]
    us = per_layer_kernel_us(fn, args.layers)
    res["roofline"] = {"kernel": "swiglu_kernel (" + name + ")", "bound": "hbm", "achieved": nbytes / us / 1e3,
                       "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / us / 1e3 / HBM_PEAK_GBS,
                       "traffic": _traffic("swiglu_kernel"), "bytes_per_launch": nbytes, "us_per_launch": us}
    if args.kernel_breakdown:
        kb = {}
        for nm, (f, nb) in legs.items():
            u = per_layer_kernel_us(f, args.layers)
            kb[nm] = {"us": round(u, 3), "bytes": nb, "GB/s": round(nb / u / 1e3, 1), "frac": round(nb / u / 1e3 / HBM_PEAK_GBS, 4)}
        res["kernels"] = kb
        tot_b = sum(v["bytes"] for v in kb.values())
        tot_u = sum(v["us"] for v in kb.values())
        res["layer_sum"] = {"us": round(tot_u, 2), "bytes": tot_b, "GB/s": round(tot_b / tot_u / 1e3, 1)}
    # whole-step effective bandwidth: every factor byte + lm_head + KV read once per token
    n_ctx = PROMPT_LEN + args.warmup + args.steps // 2
    per_layer = 8 * CFG["hidden_size"] * CFG["attn_rank"] * 2 + 3 * (CFG["hidden_size"] + CFG["intermediate_size"]) * CFG["mlp_rank"] * 2
    step_bytes = args.layers * (per_layer + 2 * n_ctx * CFG["num_heads"] * CFG["head_dim"] * 2) + CFG["vocab_size"] * CFG["hidden_size"] * 2
    res["step_bytes"] = step_bytes
    res["step_GBs"] = step_bytes / (res["ms_per_step"] * 1e-3) / 1e9
    if "persistent" in res:
        # the resident step kernel is the dominant (only) kernel of the token: its algorithmic bytes are the
        # step's — every factor, the lm_head and the KV rows read once — over its event-timed launch duration
        us_launch = res["persistent"]["kernel_us_per_launch"]
        res["swiglu_roofline"] = res["roofline"]
        res["roofline"] = {"kernel": "decode_step_kernel (whole token: 32 layers + lm_head + argmax)", "bound": "hbm",
                           "achieved": step_bytes / us_launch / 1e3, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": step_bytes / us_launch / 1e3 / HBM_PEAK_GBS, "traffic": _traffic("decode_step_kernel"),
                           "bytes_per_launch": step_bytes, "us_per_launch": us_launch}
    del dec, cache, model
    torch.cuda.empty_cache()
    return res


def _traffic(kernel: str):
    """HBM bytes per launch from the committed rocprofv3 --pmc summaries, if present."""
    f = ROOT / "profiles" / "hbm_traffic.json"
    try:
        return json.loads(f.read_text())[kernel]["traffic_bytes_per_launch"]
    except Exception:
        return None


def run_dense(args):
    """Same model shape with dense bf16 weights, vendor GEMV (torch.matmul -> hipBLASLt) for the
    projections, torch ops for norm/rotary/SwiGLU, the same HIP decode-attention kernel, whole step
    captured as one graph.  This is the "same model run as dense bf16 on the same GPU" comparator."""
    import torch
    import torch.nn.functional as F
    from flashsvd_amd import hip_ops
    from types import SimpleNamespace
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    d, H, Dh, D, V, NL = CFG["hidden_size"], CFG["num_heads"], CFG["head_dim"], CFG["intermediate_size"], CFG["vocab_size"], args.layers
    bf = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(0)

    def rn(*s):
        return (torch.randn(*s, generator=gen, device="cuda") * 0.02).to(bf)

    layers = [dict(wqkv=rn(3 * d, d), wo=rn(d, d), wgu=rn(2 * D, d), wd=rn(d, D), n1=torch.ones(d, device="cuda", dtype=bf),
                   n2=torch.ones(d, device="cuda", dtype=bf)) for _ in range(NL)]
    embed, head, nf = rn(V, d), rn(V, d), torch.ones(d, device="cuda", dtype=bf)
    max_len = PROMPT_LEN + args.warmup + args.steps + 8
    cfg = SimpleNamespace(num_hidden_layers=NL, rope_theta=10000.0)
    cache = FlashSVDV15DenseKVCache(cfg, max_batch_size=1, max_cache_len=max_len, device="cuda", dtype=bf)
    for i in range(NL):
        cache._ensure_layer_spec(i, h=H, dh=Dh)
        cache.key_cache[i][:, :PROMPT_LEN].normal_()
        cache.value_cache[i][:, :PROMPT_LEN].normal_()
    cos, sin = cache.get_rope_tables(seqlen=max_len, head_dim=Dh, device="cuda", dtype=bf)
    nsplit = hip_ops.pick_nsplit(max_len, 1, H, Dh)
    ws = hip_ops.attn_workspace(1, H, Dh, nsplit, "cuda")
    tokens = torch.zeros(1, 1, dtype=torch.long, device="cuda")
    positions = torch.full((1,), PROMPT_LEN, dtype=torch.int32, device="cuda")

    def rms(x, w):
        x32 = x.float()
        return w * (x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + 1e-6)).to(bf)

    def step():
        x = embed[tokens[:, 0]]
        for i, L in enumerate(layers):
            qkv = F.linear(rms(x, L["n1"]), L["wqkv"]).view(1, 3, H, Dh)
            c, s = cos[positions.long()][:, None], sin[positions.long()][:, None]
            q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]

            def rot(t):
                t0, t1 = t[..., :Dh // 2], t[..., Dh // 2:]
                return torch.cat([t0 * c - t1 * s, t1 * c + t0 * s], -1)
            a = hip_ops.attn_decode_densekv(rot(q).contiguous(), cache.key_cache[i], cache.value_cache[i], positions,
                                            k_new=rot(k).contiguous(), v_new=v.contiguous(), nsplit=nsplit, workspace=ws)
            x = x + F.linear(a.view(1, d), L["wo"])
            gu = F.linear(rms(x, L["n2"]), L["wgu"])
            x = x + F.linear(F.silu(gu[:, :D]) * gu[:, D:], L["wd"])
        logits = F.linear(rms(x, nf), head)
        tokens.copy_(logits.argmax(-1, keepdim=True))
        positions.add_(1)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
            positions.fill_(PROMPT_LEN)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    positions.fill_(PROMPT_LEN)
    for _ in range(args.warmup):
        g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        g.replay()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return dict(tok_s=args.steps / dt, ms_per_step=dt * 1000.0 / args.steps)


def run_dense_step(args):
    """The same 7B shape with DENSE bf16 weights through this build's own engine: the resident step kernel walking
    [q;k;v] projection -> attention -> merge -> o projection -> gate/up pair + SwiGLU -> down projection per layer
    (flashsvd_amd.step.DenseStepDecoder).  Same kernel, same hand-off and attention phase as the low-rank step: the
    like-for-like comparator for "the same model run as dense bf16 on the same GPU"."""
    import torch
    from types import SimpleNamespace
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import DenseStepDecoder
    d, H, Dh, D, V, NL = CFG["hidden_size"], CFG["num_heads"], CFG["head_dim"], CFG["intermediate_size"], CFG["vocab_size"], args.layers
    bf = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(0)

    def rn(*s):
        return (torch.randn(*s, generator=gen, device="cuda") * 0.02).to(bf)

    ones = torch.ones(d, device="cuda", dtype=bf)
    layers = [dict(wqkv=rn(3 * d, d), wo=rn(d, d), wg=rn(D, d), wu=rn(D, d), wd=rn(d, D), n1=ones, n2=ones) for _ in range(NL)]
    embed, head = rn(V, d), rn(V, d)
    max_len = PROMPT_LEN + args.warmup + args.steps + 8
    cache = FlashSVDV15DenseKVCache(SimpleNamespace(num_hidden_layers=NL, rope_theta=10000.0), max_batch_size=1,
                                    max_cache_len=max_len, device="cuda", dtype=bf)
    for i in range(NL):
        cache._ensure_layer_spec(i, h=H, dh=Dh)
        cache.key_cache[i][:, :PROMPT_LEN].normal_()
        cache.value_cache[i][:, :PROMPT_LEN].normal_()
    cache._seen_tokens = PROMPT_LEN
    dec = DenseStepDecoder(embed=embed, layers=layers, norm=ones, lm_head=head, cache=cache, num_heads=H, num_kv_heads=H,
                           head_dim=Dh, max_new_tokens=args.warmup + args.steps + 4)
    dec.set_state(1, PROMPT_LEN)
    dec.step(args.warmup)
    dec.check()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    dec.step(args.steps)
    e1.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    dec.check()
    n_ctx = PROMPT_LEN + args.warmup + args.steps // 2
    step_bytes = NL * ((4 * d * d + 3 * d * D) * 2 + 2 * n_ctx * H * Dh * 2) + V * d * 2
    us = e0.elapsed_time(e1) * 1000.0 / args.steps
    res = dict(tok_s=args.steps / dt, ms_per_step=dt * 1000.0 / args.steps, kernel_us_per_launch=us, bytes_per_token=step_bytes,
               **{"GB/s": step_bytes / us / 1e3, "frac_of_peak": step_bytes / us / 1e3 / HBM_PEAK_GBS})
    del dec, cache, layers, embed, head
    torch.cuda.empty_cache()
    return res


def run_stress():
    """Stress configuration of the 7B shape at parameter ratio ~0.8 (attention rank 1664), one layer's attention kernels:
    decode at batch 16 over a 4096-token rank-space cache (K rebuilt in-kernel), and the prompt path at 8 x 2048 tokens
    (q / k / v head expansion + RoPE + causal attention).  Matrix-core bound: flop / time against the bf16 peak."""
    import torch
    from flashsvd_amd import hip_ops
    from flashsvd_amd.kernels.rank_decode import rank_decode

    def timed(fn, reps=5, warm=2):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e-3 / reps

    g = torch.Generator(device="cuda").manual_seed(0)
    rnd = lambda *shape, std=1.0: (torch.randn(*shape, device="cuda", generator=g) * std).to(torch.bfloat16)
    B, H, Hk, Dh, R, ctx = 16, 32, 32, 128, 1664, 4096
    S = ctx + 4
    q, pk, pv = rnd(B, H, Dh), rnd(B, S, R, std=0.5), rnd(B, S, R, std=0.5)
    ku, vu = rnd(Hk * Dh, R, std=R ** -0.5), rnd(Hk * Dh, R, std=R ** -0.5)
    ang = torch.arange(S, device="cuda", dtype=torch.float32)[:, None] * (1.0 / 10000.0 ** (torch.arange(0, Dh // 2, device="cuda").float() / (Dh // 2)))
    cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)     # half tables [S, Dh/2]
    lens = torch.full((B,), ctx, dtype=torch.int32, device="cuda")
    out = torch.empty(B, H, Dh, device="cuda", dtype=torch.bfloat16)
    t_dec = timed(lambda: rank_decode(q, pk, pv, ku, vu, cos, sin, lens, num_kv_heads=Hk, rotate_q=True, out=out), reps=20, warm=5)
    flop_dec = 2.0 * B * ctx * R * Hk * Dh + 2.0 * B * H * ctx * R
    cache_bytes = 2 * B * ctx * R * 2
    del pk, pv
    Bp, T = 8, 2048
    p = rnd(Bp, T, 3 * R, std=0.5)
    qu = rnd(H * Dh, R, std=R ** -0.5)
    kc = torch.zeros(Bp, T, Hk, Dh, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    qb = torch.empty(Bp, T, H, Dh, device="cuda", dtype=torch.bfloat16)
    ob = torch.empty_like(qb)
    pos0 = torch.zeros(Bp, dtype=torch.int32, device="cuda")

    def expand():
        hip_ops.lowrank_expand_heads(p[..., :R], qu, num_heads=H, head_dim=Dh, out=qb, cos=cos, sin=sin, positions=pos0)
        hip_ops.lowrank_expand_heads(p[..., R:2 * R], ku, num_heads=Hk, head_dim=Dh, out=kc, cos=cos, sin=sin, positions=pos0, dst_by_position=True)
        hip_ops.lowrank_expand_heads(p[..., 2 * R:], vu, num_heads=Hk, head_dim=Dh, out=vc, positions=pos0, dst_by_position=True)

    t_exp = timed(expand, reps=3, warm=1)
    t_att = timed(lambda: hip_ops.attn_prefill(qb, kc, vc, q_pos0=pos0, causal=True, out=ob), reps=3, warm=1)
    flop_exp = 3 * 2.0 * Bp * T * R * H * Dh
    flop_att = 2 * 2.0 * Bp * H * Dh * T * (T + 1) / 2
    peak = 2500e12
    return {
        "rank_space_decode_attention_b16_ctx4096_r1664": {
            "ms_per_layer": t_dec * 1e3, "flop": flop_dec, "TFLOPs": flop_dec / t_dec / 1e12, "frac_of_bf16_mfma_peak": flop_dec / t_dec / peak,
            "cache_bytes": cache_bytes, "cache_GB/s": cache_bytes / t_dec / 1e9},
        "prompt_attention_path_8x2048_r1664": {
            "expand_qkv_ms": t_exp * 1e3, "expand_TFLOPs": flop_exp / t_exp / 1e12, "attention_ms": t_att * 1e3,
            "attention_TFLOPs": flop_att / t_att / 1e12, "ms_per_layer": (t_exp + t_att) * 1e3,
            "frac_of_bf16_mfma_peak": (flop_exp + flop_att) / (t_exp + t_att) / peak},
    }


def run_stress_model(steps: int = 8, warmup: int = 2, layers: int = 32):
    """The stress configuration as one model: the 7B shape at parameter ratio ~0.8 (attention rank 1664, MLP rank 2432),
    bf16.  Leg 1: prefill of 8 prompts x 2048 tokens into the rank-space cache.  Leg 2: greedy decode at batch 16 over
    a 4096-token context held in rank space (the prompt is prefilled for real, 16 x 4096 tokens, untimed), K rebuilt
    in-kernel, one HIP graph per token.  Both legs are matrix-core bound at these sizes, so each reports flop / time
    against the dense bf16 peak next to its token rate; `attention_share` prices the rank-space attention kernels alone
    (their per-layer time, measured separately, x layers / step time)."""
    import torch
    from flashsvd_amd import llama
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.runtime.cache import FlashSVDLegacySparseKVCache
    R, RM, ctx, Bd, Bp, Tp = 1664, 2432, 4096, 16, 8, 2048
    cfg = dict(CFG, attn_rank=R, mlp_rank=RM, num_layers=int(layers), max_position_embeddings=ctx + 64)
    d, H, Dh, D, V, L = cfg["hidden_size"], cfg["num_heads"], cfg["head_dim"], cfg["intermediate_size"], cfg["vocab_size"], int(layers)
    def say(msg):                       # progress on stderr: the legs take tens of seconds
        print(f"[stress] {msg}", file=sys.stderr, flush=True)

    model = llama.materialize(llama.build_model(**cfg), "cuda", torch.bfloat16, seed=0)
    model.eval()
    say(f"model of {L} layers on the device")
    gen = torch.Generator().manual_seed(11)
    peak = 2500e12
    lin_flop_tok = 2.0 * (8 * d * R + 3 * (d + D) * RM)          # factor products per token per layer

    # ---- leg 1: prefill 8 x 2048.  The prompt pass rebuilds q and the context's K / V from the rank coefficients into
    # temporaries and attends over them; the heads can be taken in groups sized by a byte budget (default 1 GiB: all heads
    # at once at this shape), and the same pass with a 64 MiB budget is timed beside it: what the temporaries cost in
    # memory, and what the grouping costs in time.  (The reference's kernel rebuilds K / V tiles per query tile inside its
    # attention loop and writes none.)
    from flashsvd_amd import hip_ops as _ops
    ids = torch.randint(0, V, (Bp, Tp), generator=gen).cuda()
    legs = {}
    saved_budget = os.environ.get("FLASHSVD_AMD_PREFILL_TEMP_BYTES")
    for name, budget in (("default", None), ("head_groups_64MiB", str(64 << 20))):
        if budget is None:
            os.environ.pop("FLASHSVD_AMD_PREFILL_TEMP_BYTES", None)
        else:
            os.environ["FLASHSVD_AMD_PREFILL_TEMP_BYTES"] = budget
        times = []
        with torch.no_grad():
            for it in range(3):
                cache = FlashSVDLegacySparseKVCache(model.config, max_batch_size=Bp, max_cache_len=Tp + 8, device="cuda", dtype=torch.bfloat16)
                for li in range(L):             # the cache sizes a layer at its first use: do it before the measurement
                    cache.ensure_layer_ranks(li, R, R)
                torch.cuda.synchronize()
                torch.cuda.reset_peak_memory_stats()
                resident = torch.cuda.memory_allocated()
                t0 = time.perf_counter()
                out = model(ids, past_key_values=cache, cache_position=torch.arange(Tp), logits_to_keep=1)
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                transient = torch.cuda.max_memory_allocated() - resident
                say(f"prefill {Bp} x {Tp} ({name}): {times[-1]:.3f} s")
                del cache, out
        gk = _ops.prefill_head_groups(Bp, Tp, Tp, H, H, Dh)   # under the budget of this leg
        legs[name] = {"s": min(times[1:]), "cold_s": times[0], "transient_bytes_peak": int(transient), "kv_heads_per_pass": gk,
                      "qkv_temporaries_bytes": 3 * Bp * Tp * gk * Dh * 2}
    if saved_budget is None:
        os.environ.pop("FLASHSVD_AMD_PREFILL_TEMP_BYTES", None)
    else:
        os.environ["FLASHSVD_AMD_PREFILL_TEMP_BYTES"] = saved_budget
    t_pre = legs["default"]["s"]
    attn_flop_pre = 3 * 2.0 * Bp * Tp * R * H * Dh + 2 * 2.0 * Bp * H * Dh * Tp * (Tp + 1) / 2     # head expansion + causal attention
    flop_pre = L * (Bp * Tp * lin_flop_tok + attn_flop_pre) + 2.0 * Bp * d * V
    prefill = {"batch": Bp, "prompt_len": Tp, "s": t_pre, "cold_s": legs["default"]["cold_s"], "tok_s": Bp * Tp / t_pre, "flop": flop_pre,
               "TFLOPs": flop_pre / t_pre / 1e12, "frac_of_bf16_mfma_peak": flop_pre / t_pre / peak,
               "transient_bytes_peak": legs["default"]["transient_bytes_peak"],
               "kv_heads_per_pass": legs["default"]["kv_heads_per_pass"],
               "qkv_temporaries_bytes": legs["default"]["qkv_temporaries_bytes"],
               "head_groups_64MiB": legs["head_groups_64MiB"],
               "rank_cache_bytes_per_layer": 2 * Bp * (Tp + 8) * R * 2}

    # ---- leg 2: decode at batch 16, context 4096, rank-space cache
    ids = torch.randint(0, V, (Bd, ctx), generator=gen).cuda()
    cache = FlashSVDLegacySparseKVCache(model.config, max_batch_size=Bd, max_cache_len=ctx + steps + warmup + 8, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        out = model(ids, past_key_values=cache, cache_position=torch.arange(ctx), logits_to_keep=1)
    tok = out.logits[:, -1].float().argmax(-1, keepdim=True)
    del out
    torch.cuda.synchronize()
    say(f"context of {Bd} x {ctx} tokens prefilled into the rank-space cache")
    dec = GraphedDecoder(model, cache, Bd)
    dec.set_state(tok, ctx)
    dec.capture()
    say("decode step captured")
    for _ in range(warmup):
        dec.step()
    torch.cuda.synchronize()
    say("timing the decode steps")
    t0 = time.perf_counter()
    for _ in range(steps):
        dec.step()
    torch.cuda.synchronize()
    t_step = (time.perf_counter() - t0) / steps
    attn_flop_dec = 2.0 * Bd * ctx * R * H * Dh + 2.0 * Bd * H * ctx * R + 2.0 * Bd * H * R * Dh     # K rebuild, rank-space PV, expansion
    flop_step = L * (Bd * lin_flop_tok + attn_flop_dec) + 2.0 * Bd * d * V
    cache_bytes = L * 2 * Bd * ctx * R * 2
    weight_bytes = L * 2 * (8 * d * R + 3 * (d + D) * RM) + 2 * d * V
    decode = {"batch": Bd, "context": ctx, "steps": steps, "ms_per_step": t_step * 1e3, "tok_s": Bd / t_step, "flop_per_step": flop_step,
              "TFLOPs": flop_step / t_step / 1e12, "frac_of_bf16_mfma_peak": flop_step / t_step / peak,
              "attention_flop_per_layer": attn_flop_dec, "bytes_per_step": cache_bytes + weight_bytes,
              "GB/s": (cache_bytes + weight_bytes) / t_step / 1e9, "engine": "per-operator HIP graph", "kv_cache": "rank space (FlashSVDLegacySparseKVCache)"}
    del dec, cache, model
    torch.cuda.empty_cache()
    return {"model": f"{L}-layer 7B shape, attention rank {R}, MLP rank {RM}", "prefill": prefill, "decode": decode}


def run_quant(args, dtype=None):
    """Config 4 with every factor linear as group-wise int4 (PackedQuantLinear, group 128, asymmetric): the persistent step
    streams the packed nibbles (int4 phases), the per-operator graph uses fsvd_linear_q4 / fsvd_swiglu_linear_q4.
    ``dtype``: the type of the activations, the lm_head and the cache (bf16, or float16 with --fp16)."""
    import os
    import torch
    from flashsvd_amd import api, llama, quant as Q
    cfg = dict(CFG, num_layers=args.layers)
    model = llama.materialize(llama.build_model(**cfg), "cuda", dtype or torch.bfloat16, seed=0)
    n = Q.replace_linears_with_packed_quant_inplace(model, module_names=Q.factor_linear_names(model), bits=4, group_size=128, sym=False)
    torch.cuda.empty_cache()
    wbytes = 0
    for m in model.modules():
        if isinstance(m, Q.PackedQuantLinear):
            wbytes += m.qweight.numel() + 2 * m.scales.numel() + 2 * m.zeros.numel()
    head = model.lm_head.weight.numel() * 2
    mid = PROMPT_LEN + args.warmup + args.steps // 2
    kv = 2 * args.layers * mid * cfg["num_kv_heads"] * cfg["head_dim"] * 2
    step_bytes = wbytes + head + kv
    res = {"modules": n, "resident_GB": torch.cuda.memory_allocated() / 1e9, "bytes_per_token": step_bytes}
    keep = os.environ.get("FLASHSVD_AMD_DECODE_ENGINE")
    try:
        for eng in ("persistent", "graph"):
            os.environ["FLASHSVD_AMD_DECODE_ENGINE"] = eng
            r = api.decode_kvcache_eval(model, prompt_len=PROMPT_LEN, new_tokens=args.steps, warmup=args.warmup)
            res[eng] = {"tok_s": r["decode_tok_s"], "ms_per_step": 1e3 / r["decode_tok_s"],
                        "GB/s": step_bytes * r["decode_tok_s"] / 1e9, "frac_of_peak": step_bytes * r["decode_tok_s"] / 1e9 / HBM_PEAK_GBS}
    finally:
        if keep is None:
            os.environ.pop("FLASHSVD_AMD_DECODE_ENGINE", None)
        else:
            os.environ["FLASHSVD_AMD_DECODE_ENGINE"] = keep
    return res


def run_cpu_baseline():
    """The CPU oracle in fp32 (the precision of the reference's CPU path, scripts/demo_support/api.py:128-143,161-165) on
    the host cores of this box, every leg a bounded sample:
      value      the headline shape: 2 of the 32 layers + final norm + lm_head at context 512, 5 timed greedy tokens,
                 per-layer time scaled to 32 layers;
      legs.C1    configuration 1 whole: one block of d 512, prompt 128, then 16 greedy decode steps;
      legs.K2    one attention block call (norm, q / k / v factor pairs, rotation, cache append, attention over 513 keys,
                 o factor pair, residual) at the 7B shape, batch 1;
      legs.K3    one SwiGLU MLP call (three factor pairs) at the 7B shape for 1, 8 and 32 rows."""
    import torch
    from oracle import flashsvd_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    n_s = 2
    mw = O.make_model(d=CFG["hidden_size"], n_heads=CFG["num_heads"], n_kv_heads=CFG["num_kv_heads"], head_dim=CFG["head_dim"],
                      ffn=CFG["intermediate_size"], attn_rank=CFG["attn_rank"], mlp_rank=CFG["mlp_rank"], n_layers=n_s,
                      vocab=CFG["vocab_size"], dtype=torch.float32, seed=0)
    prompt = torch.randint(0, CFG["vocab_size"], (1, PROMPT_LEN), generator=torch.Generator().manual_seed(1))
    n_new = 6
    cache = O.DenseCache(mw, 1, PROMPT_LEN + 16, torch.float32)
    cos, sin = O.rope_tables(PROMPT_LEN + 16, mw.head_dim, mw.rope_theta, torch.float32)
    logits = O.model_forward(mw, prompt, 0, cache, cos, sin)
    tok = logits[:, -1].argmax(-1, keepdim=True)
    t_layers = t_head = 0.0
    for s in range(n_new):
        t0 = time.perf_counter()
        x = mw.embed[tok]
        for li in range(n_s):
            x = O.block_forward(mw, li, x, PROMPT_LEN + s, cache, cos, sin)
        t1 = time.perf_counter()
        logits = O.lin(O.rms_norm(x[:, -1:], mw.norm, mw.eps), mw.lm_head)
        tok = logits[:, -1].argmax(-1, keepdim=True)
        t2 = time.perf_counter()
        if s > 0:  # first token warms the allocator
            t_layers += t1 - t0
            t_head += t2 - t1
    per_tok = (t_layers / n_s * CFG["num_layers"] + t_head) / (n_new - 1)

    def med_ms(fn, reps):
        fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return _median(ts) * 1e3

    legs = {}
    # K2: the attention half of a block (the oracle's block_forward up to its first residual), one token at position 512
    bw, H, Hk, Dh = mw.blocks[0], mw.n_heads, mw.n_kv_heads, mw.head_dim
    pos = PROMPT_LEN
    xk = torch.randn(1, 1, CFG["hidden_size"], generator=torch.Generator().manual_seed(2))

    def attention_block():
        h1 = O.rms_norm(xk, bw.ln1, mw.eps)
        c, s_ = cos[pos:pos + 1][None, :, None, :], sin[pos:pos + 1][None, :, None, :]
        q = O.apply_rope(O.lowrank_pair(h1, bw.q_v, bw.q_u).reshape(1, 1, H, Dh), c, s_)
        cache.k[0][:1, pos:pos + 1] = O.apply_rope(O.lowrank_pair(h1, bw.k_v, bw.k_u).reshape(1, 1, Hk, Dh), c, s_)
        cache.v[0][:1, pos:pos + 1] = O.lowrank_pair(h1, bw.v_v, bw.v_u).reshape(1, 1, Hk, Dh)
        a = O._attend(q, cache.k[0][:1, :pos + 1], cache.v[0][:1, :pos + 1], pos)
        return xk + O.lowrank_pair(a, bw.o_v, bw.o_u)
    legs["K2_attention_block_bs1_ctx512"] = {"ms_per_call": med_ms(attention_block, 10)}
    # K3: the oracle's mlp_forward on RMS-normalised N(0,1) rows
    for B in (1, 8, 32):
        h2 = O.rms_norm(torch.randn(B, 1, CFG["hidden_size"], generator=torch.Generator().manual_seed(3)), bw.ln2, mw.eps)
        legs[f"K3_swiglu_mlp_bs{B}"] = {"ms_per_call": med_ms(lambda: O.mlp_forward(bw, h2), 10)}
    del mw, cache
    # C1 on its own protocol: prefill 128, then 16 greedy decode steps
    mw1, p1 = O.config_c1(torch.float32)
    runs = []
    for _ in range(3):
        c1 = O.DenseCache(mw1, 1, 128 + 20, torch.float32)
        cs1, sn1 = O.rope_tables(128 + 20, mw1.head_dim, mw1.rope_theta, torch.float32)
        t0 = time.perf_counter()
        tk = O.model_forward(mw1, p1, 0, c1, cs1, sn1)[:, -1].argmax(-1, keepdim=True)
        t1 = time.perf_counter()
        for s in range(16):
            tk = O.model_forward(mw1, tk, 128 + s, c1, cs1, sn1)[:, -1].argmax(-1, keepdim=True)
        t2 = time.perf_counter()
        runs.append((t1 - t0, (t2 - t1) / 16))
    pre, dec = _median([r[0] for r in runs]), _median([r[1] for r in runs])
    legs["C1_one_block_d512_prompt128_16steps"] = {"prefill_ms": pre * 1e3, "decode_ms_per_token": dec * 1e3, "decode_tok_s": 1.0 / dec}
    return {"value": 1.0 / per_tok, "unit": "tok/s", "cores": int(torch.get_num_threads()), "kind": "port",
            "sample": f"CPU oracle fp32, {n_s} of 32 layers + lm_head, context {PROMPT_LEN}-{PROMPT_LEN + n_new - 1}, {n_new - 1} timed greedy tokens, "
                      f"per-layer time x32 + head time ({per_tok * 1e3:.1f} ms/token)",
            "legs": legs}


def main():
    args = _parse()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); no multi-GPU path exists", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.calibrate_copy:
        n = 256 << 20
        src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch device copy", "bytes_read": n, "bytes_written": n, "launches": 10}))
        return
    from flashsvd_amd import _lib
    _lib.load()
    if args.quant:
        q = run_quant(args, torch.float16 if args.fp16 else None)
        act = "fp16" if args.fp16 else "bf16"
        print(json.dumps({"metric": "decode tok/s, 7B-shape rank-0.5 bs1, int4 factors (group 128)", "value": q["persistent"]["tok_s"], "unit": "tok/s",
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": f"int4 weights, {act} activations, fp32 sums",
                          "data": "synthetic", "quant": q}))
        return
    if args.stress:
        kern = run_stress()
        print("[stress] attention kernels timed", file=sys.stderr, flush=True)
        mp = run_stress_model(steps=max(2, min(args.steps, 8)), warmup=max(1, min(args.warmup, 2)), layers=args.layers)
        t_att = kern["rank_space_decode_attention_b16_ctx4096_r1664"]["ms_per_layer"]
        mp["decode"]["attention_share"] = t_att * args.layers / mp["decode"]["ms_per_step"]
        mp["decode"]["attention_kernel_frac_of_bf16_mfma_peak"] = kern["rank_space_decode_attention_b16_ctx4096_r1664"]["frac_of_bf16_mfma_peak"]
        print(json.dumps({"metric": "stress decode tok/s, 7B-shape rank-0.8, batch 16, context 4096, rank-space cache", "value": mp["decode"]["tok_s"],
                          "unit": "tok/s", "n_gpus": 1, "steps": mp["decode"]["steps"], "dtype": "bf16", "data": "synthetic",
                          "config": {"workload": mp["model"] + "; prefill 8 x 2048, then decode batch 16 at context 4096", "layers": args.layers},
                          "model_pass": mp, "kernels": kern}))
        return
    if args.fp16:
        lr = run_lowrank(args, torch.float16)
        line = {"metric": "decode tok/s, 7B-shape rank-0.5 bs1, float16", "value": lr["tok_s"], "unit": "tok/s", "n_gpus": 1,
                "steps": args.steps, "warmup": args.warmup, "ms_per_step": lr["ms_per_step"], "dtype": "fp16", "data": "synthetic",
                "prefill": lr["prefill"]}
        for k in ("persistent", "persistent_composed", "graph"):
            if k in lr:
                line[k if k != "graph" else "per_operator_graph"] = {m: v for m, v in lr[k].items() if m != "phase_profile_us"}
        print(json.dumps(line))
        return
    lr = run_lowrank(args)
    if args.kernel_configs_only:
        print(json.dumps({"metric": "kernel-level configurations, 7B shape rank 0.5: microseconds per call", "unit": "us", "n_gpus": 1,
                          "dtype": "bf16", "data": "synthetic", "layers": args.layers, "kernel_configs": lr["kernel_configs"]}))
        return
    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s, 7B-shape rank-0.5 bs1 prompt 512", "value": lr["prefill"]["tok_s"], "unit": "tok/s",
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": "bf16", "data": "synthetic",
                          "prefill": lr["prefill"]}))
        return
    line = {
        "metric": "decode tok/s, 7B-shape rank-0.5 bs1", "value": lr["tok_s"], "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": lr["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "32-layer Llama-2-7B-shaped low-rank decode (attn rank 1024, MLP rank 1536, vocab 32000), "
                               "bs1, prompt 512, greedy, " + ("one resident kernel launch per token" if "persistent" in lr
                                                              else "whole step in one HIP graph"), "layers": args.layers,
                   "prompt_len": PROMPT_LEN, "batch": 1, "kv_cache": "dense"},
        "roofline": lr["roofline"],
        "step_hbm": {"bytes_per_token": lr["step_bytes"], "GB/s": lr["step_GBs"], "frac_of_peak": lr["step_GBs"] / HBM_PEAK_GBS},
        "prefill_s": lr["prefill_s"],
        "prefill": lr["prefill"],
        "kernel_configs": lr.get("kernel_configs"),
    }
    for k in ("persistent", "persistent_composed", "graph", "swiglu_roofline"):
        if k in lr:
            line[k if k != "graph" else "per_operator_graph"] = lr[k]
    if "kernels" in lr:
        line["kernels"] = lr["kernels"]
        line["layer_sum"] = lr["layer_sum"]
    if not args.no_dense:
        # two dense-bf16 comparators of the same shape on the same GPU; the speed-up is quoted against the FASTER one
        ds = run_dense_step(args)
        dn = run_dense(args)
        best = max(ds["tok_s"], dn["tok_s"])
        line["dense_bf16"] = {
            "tok_s": best, "ms_per_step": 1e3 / best, "speedup_lowrank_vs_dense": lr["tok_s"] / best,
            "comparator": "resident step kernel over dense weights" if ds["tok_s"] >= dn["tok_s"] else "torch.matmul graph",
            "resident_step": dict(ds, how="same shape, dense bf16 weights, this build's resident step kernel (q;k;v projection, attention, "
                                          "o projection, gate/up pair + SwiGLU, down projection per layer), one launch per token"),
            "torch_graph": dict(dn, how="same shape, dense bf16 weights, torch.matmul (hipBLASLt) projections, torch elementwise ops, "
                                        "same attention kernel, one HIP graph per token"),
            "bandwidth_ratio_dense_over_lowrank": ds["bytes_per_token"] / lr["step_bytes"]}
        if "persistent_composed" in lr:
            line["dense_bf16"]["speedup_composed_form_vs_dense"] = lr["persistent_composed"]["tok_s"] / best
    if not args.no_stress and args.layers == CFG["num_layers"]:
        # the stress configuration (rank ratio ~0.8) as one model: prefill 8 x 2048, decode batch 16 at context 4096 over the
        # rank-space cache; `bench.py --stress` prints the same with the attention kernels timed alone
        try:
            line["stress_rank08"] = run_stress_model(steps=4, warmup=1, layers=args.layers)
        except Exception as exc:      # the headline line must not be lost to a failure of a side leg
            line["stress_rank08"] = {"error": f"{type(exc).__name__}: {exc}"}
    line["cpu_baseline"] = None if args.no_cpu else run_cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
