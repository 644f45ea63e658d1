"""The headline configuration at full depth on its own protocol: 32 layers of the 7B shape (attention rank 1024,
MLP rank 1536), bf16, prompt 512, 32 greedy tokens, both decode engines (one resident launch per token; one HIP
graph of per-operator kernels per token).

What "as accurate as the reference" means at this depth.  The bf16 oracle and the GPU paths round to bf16 at the
same points and differ only in the order of their fp32 sums, i.e. in an occasional last-bit flip at a rounding, and
32 layers of N(0, 0.02) factors amplify such flips: two CORRECT bf16 runs end a few per cent apart.  The yardstick is
therefore an exact run — the same stored weights and rotation tables, fp32 activations, no rounding between operators
(fp32 accumulation noise is four orders of magnitude below one bf16 rounding) — and the requirement is that a GPU
path is no further from it than the bf16 oracle itself is, within 1.5x (a wrong rounding point, a dropped term or
a stale value fails this; summation order does not).  Per layer, fed the oracle's own layer input and cache
(teacher forcing), the stated 1e-2 tolerance holds for all 32 layers.

Tokens.  With E = max |oracle logits - exact logits| at a step and the GPU logits within 1.5 E of the exact ones,
the GPU token MUST equal the oracle's whenever the oracle's top-2 margin exceeds 5 E (decisive steps); at the other
steps a different token is accepted only among candidates the oracle holds within that same margin.  The test prints
how many of the 32 steps are decisive and how many tokens are identical.
"""
import pytest
import torch
from types import SimpleNamespace

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, model_from_oracle

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
LP, N_NEW = 512, 32
FACTOR = 1.5          # a GPU path may be this much further from the exact run than the bf16 oracle is
# Measured on this model and prompt (the sums run in a fixed order, so the figures repeat from run to run): tokens
# identical to the oracle's out of the steps judged, and the worst distance to the exact run in units of the bf16
# oracle's own.  The floors sit just below the measurements, so that a regression of either shows.
TOKEN_FLOOR = {"per-operator graph": 28, "persistent step": 27, "persistent step, composed form": 27}
WORST_RATIO = 1.45


def _rel(a, ref):
    a, ref = a.double().flatten(), ref.double().flatten()
    return float((a - ref).abs().max() / ref.abs().max()), float(((a - ref).pow(2).mean() / ref.pow(2).mean()).sqrt())


@pytest.fixture(scope="module")
def deep():
    print("building the 32-layer model and running the oracle (bf16 and exact) ...", flush=True)
    mw = O.make_model(d=4096, n_heads=32, n_kv_heads=32, head_dim=128, ffn=11008, attn_rank=1024, mlp_rank=1536,
                      n_layers=32, vocab=32000, dtype=BF16, seed=0)
    model = model_from_oracle(mw)
    mwf = O.hold_weights_as(mw, torch.float32)
    del mw
    prompt = torch.randint(0, 32000, (1, LP), generator=torch.Generator().manual_seed(1))
    trace = []
    ref_tok, ref_hid, ref_cache, ref_logits = O.greedy_decode(mwf, prompt, N_NEW, "dense", return_logits=True, layer_trace=trace)
    # the exact run follows the oracle's tokens, so that step s of both runs is the same question
    _, x_hid, _, x_logits = O.greedy_decode(mwf, prompt, N_NEW, "dense", return_logits=True, act_dtype=torch.float32, forced=ref_tok)
    print("oracle done", flush=True)
    return SimpleNamespace(model=model, mwf=mwf, prompt=prompt, trace=trace, ref_tok=ref_tok, ref_hid=ref_hid, ref_cache=ref_cache,
                           ref_logits=ref_logits.float(), x_hid=x_hid, x_logits=x_logits.float())


def _prefill(model, prompt, extra):
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    Lp = prompt.shape[1]
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + extra, device="cuda", dtype=BF16)
    out = model(prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp), logits_to_keep=1)
    return cache, out


def _judge_step(d, s, hid, logits, what):
    """One teacher-forced step of one engine against the exact run; returns (decisive, identical)."""
    e_o, r_o = _rel(d.ref_hid[:, s], d.x_hid[:, s])
    e_g, r_g = _rel(hid, d.x_hid[:, s])
    assert torch.isfinite(hid.float()).all()
    assert e_g <= FACTOR * e_o + 1e-3 and r_g <= FACTOR * r_o + 1e-4, \
        f"{what} step {s}: hidden state {e_g:.4f} (rms {r_g:.4f}) from the exact run, the bf16 oracle {e_o:.4f} (rms {r_o:.4f})"
    lx, lo, lg = d.x_logits[0, s], d.ref_logits[0, s], logits.float().flatten().cpu()
    E = float((lo - lx).abs().max())
    Eg = float((lg - lx).abs().max())
    assert Eg <= FACTOR * E + 1e-3 * float(lx.abs().max()), f"{what} step {s}: logits {Eg:.4f} from the exact run, the bf16 oracle {E:.4f}"
    top2 = torch.topk(lo, 2).values
    margin = float(top2[0] - top2[1])
    o, g = int(d.ref_tok[0, s]), int(lg.argmax())
    decisive = margin > 5.0 * E
    if decisive:
        assert g == o, f"{what} step {s}: token {g} vs oracle {o} although the oracle's margin {margin:.4f} exceeds 5 x {E:.4f}"
    elif g != o:
        gap = float(lo[o] - lo[g])
        assert gap <= 2.0 * (E + Eg), f"{what} step {s}: token {g} vs oracle {o}, oracle logit gap {gap:.4f} beyond the measured error {E:.4f} / {Eg:.4f}"
    return decisive, g == o, e_o, e_g


def test_config4_protocol_both_engines_against_the_exact_run(deep):
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.step import PersistentDecoder
    d, model = deep, deep.model
    stats = {}
    # ---- per-operator kernels, one HIP graph per token, teacher-forced with the oracle's tokens
    cache, out = _prefill(model, d.prompt, N_NEW + 4)
    rows = [_judge_step(d, 0, out.hidden_states[:, -1].cpu(), out.logits[:, -1], "prompt pass")]
    dec = GraphedDecoder(model, cache, 1)
    dec.set_state(d.ref_tok[:, :1].cuda(), LP)
    dec.capture()
    for s in range(1, N_NEW):
        dec.step()
        rows.append(_judge_step(d, s, dec.hidden.cpu(), dec.logits[:, -1], "per-operator graph"))
        dec.tokens.copy_(d.ref_tok[:, s:s + 1])
    stats["per-operator graph"] = rows
    # ---- the persistent step
    cache_p, _ = _prefill(model, d.prompt, N_NEW + 4)
    pdec = PersistentDecoder(model, cache_p)
    rows = []
    for s in range(1, N_NEW):
        pdec.set_state(d.ref_tok[:, s - 1], LP + s - 1)
        pdec.step(1)
        pdec.check()
        rows.append(_judge_step(d, s, pdec.hidden()[None].cpu(), pdec.logits, "persistent step"))
    stats["persistent step"] = rows
    # ---- the persistent step in its composed form (rank projections folded into the u-factor phases)
    del pdec, cache_p
    cache_c, _ = _prefill(model, d.prompt, N_NEW + 4)
    cdec = PersistentDecoder(model, cache_c, composed=True)
    assert cdec.composed
    rows = []
    for s in range(1, N_NEW):
        cdec.set_state(d.ref_tok[:, s - 1], LP + s - 1)
        cdec.step(1)
        cdec.check()
        rows.append(_judge_step(d, s, cdec.hidden()[None].cpu(), cdec.logits, "persistent step, composed form"))
    stats["persistent step, composed form"] = rows
    del cdec, cache_c
    for nm, rows in stats.items():
        n_dec, n_same = sum(r[0] for r in rows), sum(r[1] for r in rows)
        worst = max(r[3] / max(r[2], 1e-9) for r in rows)
        print(f"{nm}: {len(rows)} steps, {n_dec} decisive (all identical), {n_same} tokens identical to the oracle's, "
              f"distance to the exact run at most {worst:.2f} x the bf16 oracle's "
              f"(oracle {min(r[2] for r in rows):.4f}-{max(r[2] for r in rows):.4f}, gpu {min(r[3] for r in rows):.4f}-{max(r[3] for r in rows):.4f})",
              flush=True)
        assert n_same >= TOKEN_FLOOR[nm], f"{nm}: only {n_same} of {len(rows)} tokens equal the oracle's (floor {TOKEN_FLOOR[nm]})"
        assert worst <= WORST_RATIO, f"{nm}: {worst:.2f} x the bf16 oracle's distance to the exact run (bound {WORST_RATIO})"


def test_config4_free_running_tokens_until_the_first_near_tie(deep):
    """Greedy decoding on its own tokens (no teacher): 32 tokens per engine, identical to the oracle's up to the first
    step whose top-2 margin in the oracle is inside the measured bf16-vs-exact error."""
    from flashsvd_amd.graphs import GraphedDecoder
    from flashsvd_amd.step import PersistentDecoder
    d, model = deep, deep.model
    E = [(float((d.ref_logits[0, s] - d.x_logits[0, s]).abs().max())) for s in range(N_NEW)]
    margins = [float(torch.topk(d.ref_logits[0, s], 2).values.diff().abs()) for s in range(N_NEW)]
    for engine in ("persistent", "graph"):
        cache, out = _prefill(model, d.prompt, N_NEW + 4)
        tok0 = out.logits[:, -1].float().argmax(-1, keepdim=True)
        if engine == "persistent":
            dec = PersistentDecoder(model, cache)
            dec.set_state(tok0, LP)
            dec.step(N_NEW - 1)
            toks = [int(tok0)] + dec.tokens().cpu().tolist()
        else:
            dec = GraphedDecoder(model, cache, 1)
            dec.set_state(tok0, LP)
            dec.capture()
            toks = [int(tok0)] + [int(dec.step()) for _ in range(N_NEW - 1)]
        ref = d.ref_tok[0].tolist()
        same = next((s for s in range(N_NEW) if toks[s] != ref[s]), N_NEW)
        print(f"{engine}: first {same} of {N_NEW} free-running tokens identical to the oracle's", flush=True)
        if same < N_NEW:
            assert margins[same] <= 5.0 * E[same], \
                f"{engine}: token {toks[same]} vs {ref[same]} at step {same} where the oracle's margin {margins[same]:.4f} exceeds 5 x {E[same]:.4f}"


def test_all_32_layers_teacher_forced_one_token(deep):
    """Every layer on the oracle's own layer input and the oracle's own cache rows, one decode token at position 512:
    the 1e-2 tolerance against the bf16 oracle, and no further from the exact layer output than the oracle is, for
    the per-operator kernels and for the persistent step (run as a one-layer phase list)."""
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    from flashsvd_amd.step import PersistentDecoder
    d, model = deep, deep.model
    cfg = model.config
    Hk, Dh, dm = 32, 128, 4096
    cos, sin = O.rope_tables(LP + N_NEW + 4, Dh, dtype=BF16)
    step_in = d.trace[0]                       # inputs of the 32 blocks (+ final output) at position LP
    gc = FlashSVDV15DenseKVCache(cfg, max_batch_size=1, max_cache_len=LP + 8, device="cuda", dtype=BF16)
    cfg1 = SimpleNamespace(**{**vars(cfg), "num_hidden_layers": 1})
    pos = torch.full((1,), LP, dtype=torch.int32, device="cuda")
    worst = {"per-operator": 0.0, "persistent": 0.0}
    for li in range(32):
        x, y_ref = step_in[li], step_in[li + 1]                  # [1, 1, d] bf16
        # exact output of this layer on the same input and the same (bf16-valued) cache rows
        xc = O.DenseCache.__new__(O.DenseCache)
        xc.k = [None] * 32
        xc.v = [None] * 32
        xc.k[li], xc.v[li] = d.ref_cache.k[li].float().clone(), d.ref_cache.v[li].float().clone()
        y_x = O.block_forward(d.mwf, li, x.float(), LP, xc, cos, sin)
        e_o, r_o = _rel(y_ref, y_x)
        # per-operator kernels
        gc._ensure_layer_spec(li, h=Hk, dh=Dh)
        gc.key_cache[li][:, :LP].copy_(d.ref_cache.k[li][:, :LP])
        gc.value_cache[li][:, :LP].copy_(d.ref_cache.v[li][:, :LP])
        y_k = model.model.layers[li].decode_token(x[:, 0].cuda(), gc, pos).cpu()
        # persistent step over a one-layer list: the "embedding table" is the layer input, token 0
        sub = SimpleNamespace(config=cfg1, lm_head=model.lm_head,
                              model=SimpleNamespace(layers=[model.model.layers[li]], norm=model.model.norm,
                                                    embed_tokens=SimpleNamespace(weight=x[0].cuda().contiguous())))
        c1 = FlashSVDV15DenseKVCache(cfg1, max_batch_size=1, max_cache_len=LP + 8, device="cuda", dtype=BF16)
        c1._ensure_layer_spec(0, h=Hk, dh=Dh)
        c1.key_cache[0][:, :LP].copy_(d.ref_cache.k[li][:, :LP])
        c1.value_cache[0][:, :LP].copy_(d.ref_cache.v[li][:, :LP])
        pdec = PersistentDecoder(sub, c1, max_new_tokens=4)
        pdec.set_state(0, LP)
        pdec.step(1)
        pdec.check()
        y_p = pdec.hidden()[None].cpu()
        for nm, y in (("per-operator", y_k), ("persistent", y_p)):
            assert_close_bf16(y.reshape(1, dm), y_ref.reshape(1, dm), f"layer {li} {nm} vs the bf16 oracle", **bounds(y_ref))
            e_g, r_g = _rel(y, y_x)
            worst[nm] = max(worst[nm], e_g / max(e_o, 1e-9))
            assert e_g <= FACTOR * e_o + 1e-4 and r_g <= FACTOR * r_o + 1e-5, \
                f"layer {li} {nm}: {e_g:.5f} (rms {r_g:.5f}) from the exact layer output, the bf16 oracle {e_o:.5f} (rms {r_o:.5f})"
        # the appended cache row equals the oracle's
        assert_close_bf16(gc.key_cache[li][:, LP], d.ref_cache.k[li][:, LP], f"layer {li} appended K row", abs_tol=float("inf"))
        assert_close_bf16(c1.value_cache[0][:, LP], d.ref_cache.v[li][:, LP], f"layer {li} appended V row (persistent)", abs_tol=float("inf"))
        del pdec, c1, sub
    print(f"32 layers teacher-forced: distance to the exact output at most {worst['per-operator']:.2f} x (per-operator) / "
          f"{worst['persistent']:.2f} x (persistent) the bf16 oracle's", flush=True)
