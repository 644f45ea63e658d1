"""Greedy batch-1 decoding with ONE persistent launch per token (C ABI: fsvd_decode_step).

The per-token module walk of the reference (utils/evaluator.py:39-82 ``_manual_llama_decode_step``,
scripts/demo_support/api.py:238-322) issues ~10 dependent kernels per layer; at batch 1 each of them
is a few microseconds of weight streaming behind a launch gap of the same size.  Here the whole step
is a list of phases handed to one kernel that keeps one workgroup per compute unit resident, passes
activations between workgroups through tagged vectors and keeps the weight stream of the next phase
in flight while it waits (flashsvd_amd/csrc/decode_step.hip).  Token id, position and the tag epoch
live on the device, so N tokens are N launches without host synchronisation.

Arithmetic and rounding points are those of the stand-alone kernels (hip_ops.linear,
swiglu_linear, qkv_rope_append, attn_decode_densekv); only fp32 summation order differs.
"""
from __future__ import annotations

import ctypes
import math
import os

import torch

from . import _lib
from ._lib import (EP_F32, EP_LOGITS, EP_RESID, EP_STORE, EP_SWIGLU, PF_LEAD, PF_NOWAIT, PF_SPLIT, PF_STAGE2, PH_ARGMAX, PH_ATTN, PH_EMBED,
                   PH_GEMV, PH_MERGE, Phase, TagBuf)
from .runtime.cache import FlashSVDV15DenseKVCache


class DecodeStepError(RuntimeError):
    """The persistent step gave up waiting for a hand-off (state.err != 0)."""


def _tb(t: torch.Tensor, uses: int, use: int) -> TagBuf:
    return TagBuf(t.data_ptr(), int(uses), int(use))


class PersistentDecoder:
    """``PersistentDecoder(model, cache)`` then ``set_state(token, position)``, ``step(n)``, ``tokens()``.

    Requirements (checked): batch 1, one 16-bit type throughout (bfloat16 or float16;
    weights, norms, embedding and cache alike), dense KV cache, head_dim 128, hidden and intermediate sizes that are
    multiples of 128, and a device whose compute-unit count is a multiple of the number of heads.  Factor ranks are free
    for 16-bit factors (unequal q / k / v ranks, ranks that are not multiples of 128 or smaller than the workgroup count are served
    from zero-padded copies made once, at the cost of their memory); int4 layers need equal q / k / v ranks and row
    lengths that are multiples of 256.  Models outside these limits decode through ``graphs.GraphedDecoder``.
    """

    def __init__(self, model, cache, *, mode: int | None = None, max_new_tokens: int = 4096, part: str = "model",
                 layer: int = 0, composed: bool | None = None):
        """``part``: "model" (the whole token), or — for timing one block through the same machinery — "attention"
        (embedding row -> the attention half of layer ``layer``, ending at its residual add) or "mlp" (embedding row ->
        the MLP half of that layer).  A part has no argmax phase: token and position stay where ``set_state`` put them.

        ``composed`` (default: FLASHSVD_AMD_STEP_COMPOSED, off) selects the composed form of a bf16 layer, see
        ``_composed_layers``; the default ten-phase form follows the module walk one projection per phase."""
        from .llama import _packed_rows, mlp_rounding_mode
        if part not in ("model", "attention", "mlp"):
            raise ValueError(f"part must be 'model', 'attention' or 'mlp', got {part!r}")
        self.part = part
        layer_index = int(layer)
        if not isinstance(cache, FlashSVDV15DenseKVCache):
            raise TypeError("PersistentDecoder needs a FlashSVDV15DenseKVCache")
        lib = _lib.load()
        self.lib = lib
        self.model, self.cache = model, cache
        inner = model.model
        cfg = model.config
        dev = model.lm_head.weight.device
        # one 16-bit element type for the whole step, named by the lm_head: bfloat16 or float16.
        # The kernel reinterprets every buffer it is pointed at as bits of that type (int4 factors aside):
        # anything else is refused here, so that the driver falls back to the per-operator engine instead of decoding garbage
        edt = model.lm_head.weight.dtype
        if edt not in (torch.bfloat16, torch.float16):
            raise ValueError(f"PersistentDecoder computes in bfloat16 or float16, the model is {edt}")
        self.dtype = edt
        if getattr(cache, "_dtype", edt) != edt:
            raise ValueError(f"PersistentDecoder needs a KV cache of the model's type {edt}, got {cache._dtype} "
                             f"(FlashSVDV15DenseKVCache defaults to float16: pass dtype={edt})")
        if inner.embed_tokens.weight.dtype != edt or inner.norm.weight.dtype != edt:
            raise ValueError(f"PersistentDecoder needs the embedding table and final norm in the model's type {edt}")
        layers = list(inner.layers) if part == "model" else [inner.layers[layer_index]]
        for li, layer in enumerate(layers):
            for nm, p_ in layer.named_parameters():
                if p_.is_floating_point() and p_.dtype != edt:
                    raise ValueError(f"PersistentDecoder needs weights of one type ({edt}); layer {li} {nm} is {p_.dtype}")
        self.nwg = int(lib.fsvd_decode_step_workgroups())
        if self.nwg <= 0:
            raise RuntimeError((lib.fsvd_last_error() or b"").decode() or "fsvd_decode_step_workgroups: cannot query the device")
        H = int(cfg.num_attention_heads)
        Hk = int(getattr(cfg, "num_key_value_heads", H))
        Dh = int(getattr(cfg, "head_dim", None) or cfg.hidden_size // H)
        d = int(cfg.hidden_size)
        L = len(layers)
        V = int(model.lm_head.weight.shape[0])
        if self.nwg % H != 0:
            raise ValueError(f"{self.nwg} workgroups are not a multiple of {H} heads")
        nsplit = self.nwg // H
        S = int(cache.max_cache_len)
        mode = mlp_rounding_mode() if mode is None else int(mode)
        self.H, self.Hk, self.Dh, self.d, self.L, self.V, self.S, self.nsplit = H, Hk, Dh, d, L, V, S, nsplit

        def tagged(n):  # uint32 words: tag << 16 | bf16
            return torch.zeros(n, dtype=torch.int32, device=dev)

        def tagged64(n):
            return torch.zeros(n, dtype=torch.int64, device=dev)

        from .quant import PackedQuantLinear, is_quantized, pack_quant_rows
        # a layer is either all bf16 factors or all group-wise int4 factors (PackedQuantLinear, no bias, K % 256 == 0)
        layer_q4 = []
        for li, layer in enumerate(layers):
            mods = [*layer.self_attn._factor_modules(), *layer.mlp._factor_modules()]
            if not is_quantized(*mods):
                layer_q4.append(False)
                continue
            for m in mods:
                if not isinstance(m, PackedQuantLinear) or m.bits != 4 or m.bias is not None or m.in_features % 256 != 0:
                    raise ValueError(f"PersistentDecoder: layer {li} mixes int4 and other factors, or holds an int4 factor "
                                     "with a bias or a row length that is not a multiple of 256")
                gs = int(m.group_size)
                if gs < m.in_features and (gs < 32 or gs & (gs - 1)):
                    raise ValueError(f"PersistentDecoder: int4 group size {gs} is not a power of two >= 32")
            layer_q4.append(True)
        # Ranks may differ from layer to layer and, for bf16 factors, between q, k and v: the kernel wants one rank per
        # row group, a multiple of 128 (a lane group covers 128 elements of a row) and at least one row per workgroup,
        # so factors that do not fit are copied once into zero-padded twins (zero rows / columns contribute nothing:
        # results are bit-identical to the unpadded product).  int4 factors are streamed as stored and must fit as they are.
        def rank_up(r: int) -> int:
            return max((int(r) + 127) // 128 * 128, (self.nwg + 127) // 128 * 128)

        ranks, padded = [], []
        for li, layer in enumerate(layers):
            at, mlp = layer.self_attn, layer.mlp
            rq, rk, rv = at._qkv_rank_tuple()
            rm = int(mlp.gate_v_proj.out_features)
            if int(mlp.up_v_proj.out_features) != rm:
                raise ValueError(f"PersistentDecoder needs equal gate/up ranks in layer {li}")
            ro, rd = int(at.o_v_proj.out_features), int(mlp.down_v_proj.out_features)
            if layer_q4[li]:
                if not (rq == rk == rv):
                    raise ValueError(f"PersistentDecoder needs equal q/k/v ranks in an int4 layer (layer {li}: {rq}/{rk}/{rv})")
                ranks.append((rq, ro, rm, rd))
                padded.append(None)
                continue
            Rq, Ro, Rm, Rd = rank_up(max(rq, rk, rv)), rank_up(ro), rank_up(rm), rank_up(rd)
            ranks.append((Rq, Ro, Rm, Rd))
            padded.append(dict(qkv=not (rq == rk == rv == Rq), o=ro != Ro, gu=rm != Rm, d=rd != Rd))
        if not ranks:
            raise ValueError("PersistentDecoder needs at least one layer")
        Rq, Ro, Rm, Rd = (max(r[i] for r in ranks) for i in range(4))
        D = int(layers[0].mlp.gate_u_proj.out_features)
        self.XA, self.XB = tagged(d), tagged(d)
        self.P, self.QKV = tagged(3 * Rq), tagged((H + 2 * Hk) * Dh)
        self.PART, self.A = tagged64(H * nsplit * (Dh + 2)), tagged(H * Dh)
        self.PO, self.PM, self.HB, self.SB = tagged(Ro), tagged(2 * Rm), tagged(D), tagged(Rd)
        self.CAND = tagged64(self.nwg)
        self.logits = torch.zeros(V, dtype=edt, device=dev)
        self.token_log = torch.zeros(int(max_new_tokens), dtype=torch.int64, device=dev)
        self.state = torch.zeros(8, dtype=torch.int32, device=dev)   # fsvd_step_state
        self.rope = cache.get_rope_tables(seqlen=S, head_dim=Dh, device=dev, dtype=edt)
        cos, sin = self.rope
        self._keep = []   # tensors whose storage the phase list points into

        ph: list[Phase] = []
        names: list[str] = []

        def sz_words(scales, zeros):
            """uint32 [N, G]: fp16 scale bits in the low half, zero point + c in the high half (what a piece needs in one
            load); c = 128 in a bf16 step, 16 in a float16 one: the value a nibble's bit pattern is offset by."""
            if scales.dtype != torch.float16:
                raise ValueError(f"int4 scales must be float16, got {scales.dtype}")
            c = 16 if edt == torch.float16 else 128
            zmin, zmax = int(zeros.min()), int(zeros.max())
            if zmin < -c or zmax > 65535 - c:
                raise ValueError(f"int4 zero points {zmin}..{zmax} do not fit the unsigned 16-bit field of the packed "
                                 f"scale | zero word (zero + {c})")
            lo = scales.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
            hi = (zeros.to(torch.int32) + c) << 16
            return (lo | hi).contiguous()

        def pad_rows(w, n):       # zero rows below: outputs that are zero
            out_ = torch.zeros(n, w.shape[1], dtype=edt, device=dev)
            out_[:w.shape[0]] = w.data
            return out_

        def pad_cols(w, n):       # zero columns to the right: inputs that are multiplied by zero
            out_ = torch.zeros(w.shape[0], n, dtype=edt, device=dev)
            out_[:, :w.shape[1]] = w.data
            return out_

        def gemv(name, W, N, K, inp, out, *, nmat=1, norm=None, eps=0.0, epi=EP_STORE, aux=None, plain=None, groups=None, q4=None,
                 flags=0, in_off=0, in2=None, in2_len=0, in2_off=0, rows0=0, aux2=None, out1=None):
            p = Phase()
            p.type, p.epilogue, p.N, p.K, p.nmat, p.mode = PH_GEMV, epi, N, K, nmat, mode
            if edt == torch.float16:
                p.wbits = _lib.WBITS_FP16     # in every GEMV phase: the step's element type
            if groups is not None:          # rows are q | k | v heads, each group reads its own K-long input
                p.H, p.Hk, p.Dh = groups
            if q4 is not None:              # W holds (qweight, scales, zeros) triples; q4 = group size
                gs = min(int(q4), K)
                p.wbits, p.gshift = (_lib.WBITS_Q4_FP16 if edt == torch.float16 else 4), int(math.log2(gs // 32))
                for i, (qw, sc, zr) in enumerate(W):
                    G = (K + gs - 1) // gs
                    if tuple(qw.shape) != (N, K // 2) or not qw.is_contiguous() or tuple(sc.shape) != (N, G) or tuple(zr.shape) != (N, G):
                        raise ValueError(f"int4 factor {tuple(qw.shape)} / {tuple(sc.shape)} does not match [{N},{K}] in groups of {gs}")
                    sz = sz_words(sc, zr)
                    p.W[i], p.qsz[i], p.ldg = qw.data_ptr(), sz.data_ptr(), G
                    self._keep += [qw, sz]
                W = ()
            for i, w in enumerate(W):
                if tuple(w.shape) != (N, K) or not w.is_contiguous():
                    raise ValueError(f"weight {tuple(w.shape)} is not a contiguous [{N},{K}] matrix")
                p.W[i] = w.data_ptr()
                self._keep.append(w)
            if norm is not None:
                p.norm_w, p.fparam = norm.data_ptr(), float(eps)
                self._keep.append(norm)
            elif flags & PF_STAGE2:
                p.fparam = float(eps)
            p.flags, p.in_off = int(flags), int(in_off)
            if flags & PF_STAGE2:
                p.in2, p.in2_len, p.in2_off = in2, int(in2_len), int(in2_off)
            if flags & PF_SPLIT:
                p.rows0 = int(rows0)
            if inp is not None:
                p.inp = inp
            if out is not None:
                p.out0 = out
            if aux is not None:
                p.aux0 = aux
            if aux2 is not None:
                p.aux2 = aux2
            if out1 is not None:
                p.out1 = out1
            if plain is not None:
                p.plain_out = plain.data_ptr()
            ph.append(p)
            names.append(name)

        def attention(l, lc):
            kc, vc = cache.key_cache[lc][0], cache.value_cache[lc][0]    # [S, Hk, Dh]
            a = Phase()
            a.type, a.H, a.Hk, a.Dh, a.S, a.nsplit = PH_ATTN, H, Hk, Dh, S, nsplit
            a.fparam = 1.0 / math.sqrt(Dh)
            a.cos, a.sin, a.rope_len = cos.data_ptr(), sin.data_ptr(), int(cos.shape[0])
            a.k_cache, a.v_cache, a.sc_s, a.sc_h = kc.data_ptr(), vc.data_ptr(), kc.stride(0), kc.stride(1)
            a.inp, a.out0 = _tb(self.QKV, L, l), _tb(self.PART, L, l)
            ph.append(a)
            names.append("attn")
            m = Phase()
            m.type, m.H, m.Dh, m.nsplit = PH_MERGE, H, Dh, nsplit
            m.inp, m.out0 = _tb(self.PART, L, l), _tb(self.A, L, l)
            ph.append(m)
            names.append("attn_merge")

        def bf16_weights(l):
            """The nine matrices of a bf16 layer as the kernel streams them: [q_v; k_v; v_v], [q_u; k_u; v_u], o_v, o_u,
            [gate_v; up_v], gate_u, up_u, down_v, down_u, zero-padded to the layer's working ranks where needed."""
            layer = layers[l]
            at, mlp = layer.self_attn, layer.mlp
            rq, ro, rm, rd = ranks[l]
            if padded[l]["qkv"]:
                # unequal or unaligned q / k / v ranks: [q_v; k_v; v_v] with each block padded to rq rows, and the head bases
                # with their columns padded to rq
                aq, ak, av = at._qkv_rank_tuple()
                pv = torch.zeros(3 * rq, d, dtype=edt, device=dev)
                qu = torch.zeros((H + 2 * Hk) * Dh, rq, dtype=edt, device=dev)
                for i, (m_v, m_u, r_, row0, rows) in enumerate(((at.q_v_proj, at.q_u_proj, aq, 0, H * Dh), (at.k_v_proj, at.k_u_proj, ak, H * Dh, Hk * Dh),
                                                                (at.v_v_proj, at.v_u_proj, av, (H + Hk) * Dh, Hk * Dh))):
                    pv[i * rq:i * rq + r_] = m_v.weight.data
                    qu[row0:row0 + rows, :r_] = m_u.weight.data
            else:
                pv = at._packed_qkv_v
                # the three module weights become views of one buffer
                qu = _packed_rows([at.q_u_proj, at.k_u_proj, at.v_u_proj])
            w_ov, w_ou = at.o_v_proj.weight, at.o_u_proj.weight
            if padded[l]["o"]:
                w_ov, w_ou = pad_rows(w_ov, ro), pad_cols(w_ou, ro)
            w_guv, w_gu, w_uu = mlp._packed_gu_v, mlp.gate_u_proj.weight, mlp.up_u_proj.weight
            if padded[l]["gu"]:
                am = int(mlp.gate_v_proj.out_features)
                w_guv = torch.zeros(2 * rm, d, dtype=edt, device=dev)
                w_guv[:am] = mlp.gate_v_proj.weight.data
                w_guv[rm:rm + am] = mlp.up_v_proj.weight.data
                w_gu, w_uu = pad_cols(w_gu, rm), pad_cols(w_uu, rm)
            w_dv, w_du = mlp.down_v_proj.weight, mlp.down_u_proj.weight
            if padded[l]["d"]:
                w_dv, w_du = pad_rows(w_dv, rd), pad_cols(w_du, rd)
            return dict(qkv_v=pv, qkv_u=qu, o_v=w_ov, o_u=w_ou, gu_v=w_guv, gate_u=w_gu, up_u=w_uu, down_v=w_dv, down_u=w_du)

        e = Phase()
        e.type, e.N = PH_EMBED, d
        emb = inner.embed_tokens.weight
        e.K = int(emb.shape[0])          # rows of the table: the kernel refuses a token outside it
        if tuple(emb.shape)[1] != d or not emb.is_contiguous():
            raise ValueError("embedding table must be a contiguous [V, hidden] matrix")
        e.W[0] = emb.data_ptr()
        e.out0 = _tb(self.XB, L, 0) if part == "mlp" else _tb(self.XA, L + 1, 0)     # an MLP part starts at the mid-layer state
        ph.append(e)
        names.append("embed")
        for layer in layers:
            layer.self_attn._ensure_runtime_state()
            layer.mlp._ensure_runtime_state()
        if composed is None:
            composed = os.getenv("FLASHSVD_AMD_STEP_COMPOSED", "0").strip().lower() in ("1", "true", "on", "yes")
        # the composed form is for whole bf16 models whose two-vector stagings fit one round of loads
        in2_off_a = (3 * Rq + 127) // 128 * 128
        in2_off_m = (2 * Rm + 127) // 128 * 128

        def slots(n_sums):
            return (n_sums // 2 + 511) // 512 + (d // 4 + 511) // 512

        self.composed = bool(composed) and part == "model" and not any(layer_q4) and max(slots(3 * Rq), slots(2 * Rm)) <= 8 \
            and max(in2_off_a, in2_off_m) + d <= 16384 and d + max(3 * Rq, 2 * Rm) <= 64 * self.nwg
        # The products with the hidden state as leading phases (streamed in front of o_v / down_v): the hidden state
        # must stay in the staging area until then, i.e. behind everything staged in between, and a workgroup's share of
        # each product must fill whole windows of loads
        lead_off_a = (max(3 * Rq, H * Dh, 3 * Dh) + 127) // 128 * 128
        lead_off_m = (max(2 * Rm, D) + 127) // 128 * 128
        want_lead = os.getenv("FLASHSVD_AMD_STEP_LEAD", "1").strip().lower() in ("1", "true", "on", "yes")
        self.leading = self.composed and want_lead and max(lead_off_a, lead_off_m) + d <= 16384 and all(
            n % self.nwg == 0 and n // self.nwg <= 64 and ((n // self.nwg) * (d // 8)) % 2048 == 0
            for r in ranks for n in (3 * r[0], 2 * r[2]))
        if self.leading:
            in2_off_a, in2_off_m = lead_off_a, lead_off_m
        if self.composed:
            self._composed_layers(layers, ranks, bf16_weights, gemv, attention, in2_off_a, in2_off_m)
        for l, layer in enumerate(layers):
            if self.composed:
                break
            at, mlp = layer.self_attn, layer.mlp
            rq, ro, rm, rd = ranks[l]
            lc = l if part == "model" else layer_index                    # the layer's index in the cache
            cache._ensure_layer_spec(lc, h=Hk, dh=Dh)
            n1, n2 = layer.input_layernorm, layer.post_attention_layernorm
            xin, xmid, xout = _tb(self.XA, L + 1, l), _tb(self.XB, L, l), _tb(self.XA, L + 1, l + 1)
            q4 = layer_q4[l]

            def triple(*mods):
                """(qweight, scales, zeros) of one int4 module, or of several stacked row-wise into one stream."""
                if len(mods) == 1:
                    m = mods[0]
                    return (m.qweight, m.scales, m.zeros), int(m.group_size)
                pk = pack_quant_rows(mods)
                if pk is None:
                    raise ValueError(f"PersistentDecoder: int4 factors of layer {l} cannot share a stream (group sizes differ)")
                return pk, int(mods[0].group_size)

            bw = None if q4 else bf16_weights(l)
            if part == "mlp":
                pass
            elif q4:
                w, gs = triple(at.q_v_proj, at.k_v_proj, at.v_v_proj)
                gemv("attn_rank_proj", [w], 3 * rq, d, xin, _tb(self.P, L, l), norm=n1.weight, eps=n1.variance_epsilon, q4=gs)
                w, gs = triple(at.q_u_proj, at.k_u_proj, at.v_u_proj)
                gemv("qkv_u", [w], (H + 2 * Hk) * Dh, rq, _tb(self.P, L, l), _tb(self.QKV, L, l), groups=(H, Hk, Dh), q4=gs)
            else:
                gemv("attn_rank_proj", [bw["qkv_v"]], 3 * rq, d, xin, _tb(self.P, L, l), norm=n1.weight, eps=n1.variance_epsilon)
                # q, k, v head expansion as one GEMV over the row-packed [q_u; k_u; v_u]; RoPE and the cache append
                # happen in the attention phase
                gemv("qkv_u", [bw["qkv_u"]], (H + 2 * Hk) * Dh, rq, _tb(self.P, L, l), _tb(self.QKV, L, l), groups=(H, Hk, Dh))
            if part != "mlp":
                attention(l, lc)
                if q4:
                    w, gs = triple(at.o_v_proj)
                    gemv("o_v", [w], ro, H * Dh, _tb(self.A, L, l), _tb(self.PO, L, l), q4=gs)
                    w, gs = triple(at.o_u_proj)
                    gemv("o_u", [w], d, ro, _tb(self.PO, L, l), xmid, epi=EP_RESID, aux=xin, q4=gs)
                else:
                    gemv("o_v", [bw["o_v"]], ro, H * Dh, _tb(self.A, L, l), _tb(self.PO, L, l))
                    gemv("o_u", [bw["o_u"]], d, ro, _tb(self.PO, L, l), xmid, epi=EP_RESID, aux=xin)
            if part == "attention":
                pass
            elif q4:
                w, gs = triple(mlp.gate_v_proj, mlp.up_v_proj)
                gemv("mlp_rank_proj", [w], 2 * rm, d, xmid, _tb(self.PM, L, l), norm=n2.weight, eps=n2.variance_epsilon, q4=gs)
                (wg, gs), (wu, gs2) = triple(mlp.gate_u_proj), triple(mlp.up_u_proj)
                if gs != gs2:
                    raise ValueError(f"PersistentDecoder: gate_u / up_u of layer {l} use different int4 group sizes")
                gemv("swiglu", [wg, wu], D, rm, _tb(self.PM, L, l), _tb(self.HB, L, l), nmat=2, epi=EP_SWIGLU, q4=gs)
                w, gs = triple(mlp.down_v_proj)
                gemv("down_v", [w], rd, D, _tb(self.HB, L, l), _tb(self.SB, L, l), q4=gs)
                w, gs = triple(mlp.down_u_proj)
                gemv("down_u", [w], d, rd, _tb(self.SB, L, l), xout, epi=EP_RESID, aux=xmid, q4=gs)
            else:
                gemv("mlp_rank_proj", [bw["gu_v"]], 2 * rm, d, xmid, _tb(self.PM, L, l), norm=n2.weight, eps=n2.variance_epsilon)
                gemv("swiglu", [bw["gate_u"], bw["up_u"]], D, rm, _tb(self.PM, L, l), _tb(self.HB, L, l), nmat=2, epi=EP_SWIGLU)
                gemv("down_v", [bw["down_v"]], rd, D, _tb(self.HB, L, l), _tb(self.SB, L, l))
                gemv("down_u", [bw["down_u"]], d, rd, _tb(self.SB, L, l), xout, epi=EP_RESID, aux=xmid)
            cache._layer_initialized[lc] = True
        if part == "model":
            fn = inner.norm
            gemv("lm_head", [model.lm_head.weight], V, d, _tb(self.XA, L + 1, L), _tb(self.CAND, 1, 0), norm=fn.weight,
                 eps=fn.variance_epsilon, epi=EP_LOGITS, plain=self.logits)
            g = Phase()
            g.type = PH_ARGMAX
            g.inp = _tb(self.CAND, 1, 0)
            g.plain_out = self.token_log.data_ptr()
            ph.append(g)
            names.append("argmax")
        self._names = names

        self._finish(ph, dev)

    def _composed_layers(self, layers, ranks, bf16_weights, gemv, attention, off_a, off_m) -> None:
        """The eight-phase form of a bf16 layer.

        RMSNorm is a scalar behind a product once its weight vector is folded into the matrix (W' = W diag(w)), and a
        product with a hidden state that is itself ``x + U t`` splits as ``W' x + (W' U) t``.  So the two rank
        projections of a layer leave the critical path: ``[gate_v; up_v]' x`` is taken (as unrounded fp32 sums) right
        behind the q / k / v expansion, from the copy of x that phase has staged, and the o_u phase streams
        ``[o_u; [gate_v; up_v]' o_u]`` — its first rows give the new hidden state, the others complete the sums, which the
        SwiGLU phase scales by 1 / rms of that state while staging them; the same with down_u and the NEXT layer's
        ``[q_v; k_v; v_v]'``, whose product with the mid-layer state rides behind the SwiGLU pair.  Per layer: ten
        hand-offs become eight and the two composed blocks add 6 % to the layer's bytes.

        Where the two moved products (25 MB each at the 7B shape) run: as *leading phases* (``self.leading``) when a
        workgroup's share of each fills whole windows of loads and the staging area can keep the hidden state that long -
        ``[gate_v; up_v]' x`` is then streamed in front of o_v and the next layer's ``[q_v; k_v; v_v]' x2`` in front of
        down_v, in iterations that neither poll nor publish (the sums wait in the workgroup's partial buffer and leave
        with o_v's / down_v's), so that o_v / down_v poll for their input when it has long been published; otherwise as
        phases of their own behind the expansion and behind the pair (the older arrangement, FLASHSVD_AMD_STEP_LEAD=0
        forces it).  Same sums, same bits.

        Arithmetic: the hidden states take the same roundings as in the ten-phase form; the rank coefficients are formed
        from the unrounded residual sum and rounded once (the ten-phase form rounds the hidden state, the normalised
        state and its product with the norm weight first), and the composed blocks ``W' U`` are products in fp32 of the
        stored factors, rounded to bf16 once.
        """
        dev = self.XA.device
        H, Hk, Dh, d, L = self.H, self.Hk, self.Dh, self.d, self.L
        D = int(layers[0].mlp.gate_u_proj.out_features)
        Rq = max(r[0] for r in ranks)
        Rm = max(r[2] for r in ranks)

        def tagged64(n):
            return torch.zeros(n, dtype=torch.int64, device=dev)

        self.PRAW, self.G0, self.PMRAW, self.Q0 = tagged64(3 * Rq), tagged64(2 * Rm), tagged64(2 * Rm), tagged64(3 * Rq)
        nq0 = max(L - 1, 1)

        def folded(w, norm):
            """W diag(norm) in fp32; as a bf16 matrix it is W itself when the norm weights are all one."""
            nw = norm.weight.data.float()
            wf = w.data.float() * nw[None, :]
            return wf, (w if bool((nw == 1).all()) else wf.to(self.dtype).contiguous())

        bw = [bf16_weights(l) for l in range(L)]
        fq = [folded(bw[l]["qkv_v"], layers[l].input_layernorm) for l in range(L)]
        for l, layer in enumerate(layers):
            rq, ro, rm, rd = ranks[l]
            n1, n2 = layer.input_layernorm, layer.post_attention_layernorm
            self.cache._ensure_layer_spec(l, h=Hk, dh=Dh)
            xin, xmid, xout = _tb(self.XA, L + 1, l), _tb(self.XB, L, l), _tb(self.XA, L + 1, l + 1)
            w = bw[l]
            gu32, gu16 = folded(w["gu_v"], n2)
            # [o_u; [gate_v; up_v]' o_u] and [down_u; [q_v; k_v; v_v]'(next layer) down_u]: one stream each
            cat_o = torch.cat([w["o_u"].data, (gu32 @ w["o_u"].data.float()).to(self.dtype)]).contiguous()
            if l == 0:
                gemv("attn_rank_proj", [fq[0][1]], 3 * rq, d, xin, None, epi=EP_F32, out1=_tb(self.PRAW, L, 0))
            gemv("qkv_u", [w["qkv_u"]], (H + 2 * Hk) * Dh, rq, _tb(self.PRAW, L, l), _tb(self.QKV, L, l), groups=(H, Hk, Dh),
                 flags=PF_STAGE2, eps=n1.variance_epsilon, in2=xin, in2_len=d, in2_off=off_a)
            if not self.leading:
                gemv("mlp_rank_x", [gu16], 2 * rm, d, None, None, epi=EP_F32, flags=PF_NOWAIT, in_off=off_a, out1=_tb(self.G0, L, l))
            attention(l, l)
            if self.leading:
                gemv("mlp_rank_x", [gu16], 2 * rm, d, None, None, epi=EP_F32, flags=PF_NOWAIT | PF_LEAD, in_off=off_a,
                     out1=_tb(self.G0, L, l))
            gemv("o_v", [w["o_v"]], ro, H * Dh, _tb(self.A, L, l), _tb(self.PO, L, l))
            gemv("o_u+mlp_rank", [cat_o], d + 2 * rm, ro, _tb(self.PO, L, l), xmid, epi=EP_RESID, aux=xin, flags=PF_SPLIT, rows0=d,
                 aux2=_tb(self.G0, L, l), out1=_tb(self.PMRAW, L, l))
            gemv("swiglu", [w["gate_u"], w["up_u"]], D, rm, _tb(self.PMRAW, L, l), _tb(self.HB, L, l), nmat=2, epi=EP_SWIGLU,
                 flags=PF_STAGE2, eps=n2.variance_epsilon, in2=xmid, in2_len=d, in2_off=off_m)
            if l + 1 < L:
                rq_n = ranks[l + 1][0]
                gemv("attn_rank_x", [fq[l + 1][1]], 3 * rq_n, d, None, None, epi=EP_F32,
                     flags=PF_NOWAIT | (PF_LEAD if self.leading else 0), in_off=off_m, out1=_tb(self.Q0, nq0, l))
            gemv("down_v", [w["down_v"]], rd, D, _tb(self.HB, L, l), _tb(self.SB, L, l))
            if l + 1 < L:
                cat_d = torch.cat([w["down_u"].data, (fq[l + 1][0] @ w["down_u"].data.float()).to(self.dtype)]).contiguous()
                gemv("down_u+attn_rank", [cat_d], d + 3 * rq_n, rd, _tb(self.SB, L, l), xout, epi=EP_RESID, aux=xmid, flags=PF_SPLIT,
                     rows0=d, aux2=_tb(self.Q0, nq0, l), out1=_tb(self.PRAW, L, l + 1))
            else:
                gemv("down_u", [w["down_u"]], d, rd, _tb(self.SB, L, l), xout, epi=EP_RESID, aux=xmid)
            self.cache._layer_initialized[l] = True
            fq[l] = None      # the fp32 copies are only needed while the blocks are composed

    def _finish(self, ph, dev) -> None:
        """Derived fields, host-side validation, upload of the phase list."""
        lib = self.lib
        self.nph = len(ph)
        self.host_phases = (Phase * self.nph)(*ph)
        _lib.check("fsvd_decode_step_prepare", lib.fsvd_decode_step_prepare(ctypes.addressof(self.host_phases), self.nph, self.nwg))
        # reject a model the kernel cannot run here, not at the first step (the driver then takes the other engine)
        _lib.check("fsvd_decode_step_validate", lib.fsvd_decode_step_validate(ctypes.addressof(self.host_phases), self.nph, self.nwg))
        raw = bytes(self.host_phases)
        self.dev_phases = torch.frombuffer(bytearray(raw), dtype=torch.uint8).to(dev)
        self._validated = False
        self._host_pos = 0
        self._host_steps = 0

    # ------------------------------------------------------------------ state
    def set_state(self, token, position: int) -> None:
        """Next input token and its position (= number of keys already in the cache)."""
        if position < 0 or position >= self.S:
            raise IndexError(f"decode position {position} outside the cache (max {self.S})")
        tok = int(token.reshape(-1)[0].item()) if torch.is_tensor(token) else int(token)
        st = self.state
        st[2] = int(position)
        st[3] = 0
        st.view(torch.int64)[2] = tok
        self._host_pos = int(position)
        self._host_steps = 0

    def step(self, n: int = 1) -> None:
        """Decode ``n`` tokens greedily (asynchronous; read them with ``tokens()``).  A part ("attention" / "mlp") runs its
        phases ``n`` times at the position of ``set_state``: nothing advances."""
        if getattr(self, "part", "model") != "model":
            stream = torch.cuda.current_stream().cuda_stream
            for _ in range(int(n)):
                rc = self.lib.fsvd_decode_step(self.dev_phases.data_ptr(), ctypes.addressof(self.host_phases), self.nph,
                                               self.state.data_ptr(), 0 if self._validated else 1, stream)
                _lib.check("fsvd_decode_step", rc)
                self._validated = True
            return
        if self._host_pos + n > self.S:
            raise IndexError(f"decode position {self._host_pos + n - 1} outside the cache (max {self.S})")
        if self._host_steps + n > self.token_log.numel():
            raise IndexError(f"token log holds {self.token_log.numel()} tokens")
        stream = torch.cuda.current_stream().cuda_stream
        for _ in range(int(n)):
            rc = self.lib.fsvd_decode_step(self.dev_phases.data_ptr(), ctypes.addressof(self.host_phases), self.nph,
                                           self.state.data_ptr(), 0 if self._validated else 1, stream)
            _lib.check("fsvd_decode_step", rc)
            self._validated = True
        self._host_pos += int(n)
        self._host_steps += int(n)
        self.cache._seen_tokens += int(n)

    def phase_names(self) -> list:
        return list(self._names)

    def trace_step(self, wg_stride: int = 32) -> torch.Tensor:
        """Run ONE step with per-phase time stamps; returns int64 [workgroups/stride, phases, 4] in
        microseconds relative to the earliest stamp (0 entered, 1 input staged, 2 weights consumed,
        3 epilogue done).  The step counts like any other (token, position and cache advance)."""
        if not self._validated:
            raise RuntimeError("run step() once before tracing")
        if self._host_pos + 1 > self.S or self._host_steps + 1 > self.token_log.numel():
            raise IndexError("no room for another step")
        nt = (self.nwg + wg_stride - 1) // wg_stride
        buf = torch.zeros(nt * self.nph * 4, dtype=torch.int64, device=self.state.device)
        rc = self.lib.fsvd_decode_step_trace(self.dev_phases.data_ptr(), ctypes.addressof(self.host_phases), self.nph,
                                             self.state.data_ptr(), buf.data_ptr(),
                                             buf.numel(), int(wg_stride), torch.cuda.current_stream().cuda_stream)
        _lib.check("fsvd_decode_step_trace", rc)
        self._host_pos += 1
        self._host_steps += 1
        self.cache._seen_tokens += 1
        self.check()
        t = buf.view(nt, self.nph, 4).cpu()
        t0 = t[t > 0].min()
        return (t - t0).clamp_min(0).float() / 100.0

    def check(self) -> None:
        """Synchronise and raise if a step reported an error: a hand-off that never arrived (time-out), an input token
        outside the embedding table, or logits none of which compares (all NaN: there is no greedy token)."""
        st = self.state.cpu()
        if int(st[1]) != 0:
            p = int(st[1]) - 1
            names = self.phase_names() if hasattr(self, "phase_names") else []
            what = f" ({names[p]})" if 0 <= p < len(names) else ""
            raise DecodeStepError(f"decode step failed in phase {p}{what} (workgroup {int(st[6])}): time-out of a hand-off, "
                                  "token outside the embedding table, or no comparable logit; clear with reset_error() "
                                  "after finding the cause")

    def reset_error(self) -> None:
        """Clear a time-out.  The failed step left half-written vectors that carry its tags, so the
        epoch moves on and every tag of the next step differs from them."""
        self.state[1] = 0
        self.state[0] += 1

    def set_spin_limit(self, polls: int) -> None:
        """Polls before a workgroup gives up waiting (0 = default, about a second)."""
        self.state[7] = int(polls)

    def tokens(self) -> torch.Tensor:
        """Tokens generated since ``set_state`` (synchronises)."""
        self.check()
        return self.token_log[: self._host_steps].clone()

    def hidden(self) -> torch.Tensor:
        """Final-layer hidden state of the last step in the step's element type, [hidden] (part "attention": the state after the attention
        half's residual add; part "mlp": after the MLP half's)."""
        buf = self.XB if getattr(self, "part", "model") == "attention" else self.XA
        if getattr(self, "dtype", torch.bfloat16) == torch.float16:
            return (buf & 0xFFFF).to(torch.int16).view(torch.float16)
        return ((buf & 0xFFFF) << 16).view(torch.float32).to(torch.bfloat16)


    # ------------------------------------------------------------------ GraphedDecoder-compatible face
    def step_token(self) -> torch.Tensor:
        """One token; returns the device tensor [1, 1] that holds the next token id (no synchronisation)."""
        self.step(1)
        return self.state.view(torch.int64)[2].reshape(1, 1)

    def phase_profile(self, wg_stride: int = 32) -> dict:
        """Per-phase microseconds of one traced step, averaged over layers and traced workgroups:
        {phase name: {"wait": input wait, "stream": weight stream, "publish": epilogue, "total": ...}}."""
        t = self.trace_step(wg_stride)
        names = self.phase_names()
        acc: dict = {}
        for p, nm in enumerate(names):
            e, s_, c, d_ = (t[:, p, k] for k in range(4))
            staged = torch.where(s_ > 0, s_, e)
            row = acc.setdefault(nm, {"wait": 0.0, "stream": 0.0, "publish": 0.0, "total": 0.0, "n": 0})
            row["wait"] += float((staged - e).mean())
            row["stream"] += float((c - staged).mean())
            row["publish"] += float((d_ - c).mean())
            row["total"] += float((d_ - e).mean())
            row["n"] += 1
        return {k: {m: v[m] / v["n"] for m in ("wait", "stream", "publish", "total")} for k, v in acc.items()}


class DenseStepDecoder(PersistentDecoder):
    """The same resident step over DENSE bf16 Llama weights: per layer [q; k; v] projection (RMSNorm fused) -> attention
    -> merge -> o projection (+ residual) -> gate / up pair (RMSNorm fused, SwiGLU, both matrices over one input) ->
    down projection (+ residual), then final norm + lm_head + argmax.  It exists as the like-for-like comparator of the
    low-rank step ("the same model run as dense bf16 on the same GPU"): same kernel, same hand-off, same attention
    phase, only the weight streams differ.

    ``layers``: one dict per layer with ``wqkv`` [(H + 2*Hk)*Dh, d], ``wo`` [d, H*Dh], ``wg``, ``wu`` [D, d],
    ``wd`` [d, D], ``n1``, ``n2`` [d] (bf16, contiguous, on the cache's device)."""

    PHASE_NAMES = ("embed", "qkv", "attn", "attn_merge", "o", "gate_up", "down")

    def __init__(self, *, embed, layers, norm, lm_head, cache, num_heads: int, num_kv_heads: int, head_dim: int,
                 eps: float = 1e-6, mode: int = 0, max_new_tokens: int = 4096):
        if not isinstance(cache, FlashSVDV15DenseKVCache) or getattr(cache, "_dtype", None) != torch.bfloat16:
            raise TypeError("DenseStepDecoder needs a bfloat16 FlashSVDV15DenseKVCache")
        lib = _lib.load()
        self.lib, self.cache, self.model = lib, cache, None
        dev = lm_head.device
        self.nwg = int(lib.fsvd_decode_step_workgroups())
        H, Hk, Dh = int(num_heads), int(num_kv_heads), int(head_dim)
        V, d = lm_head.shape
        L = len(layers)
        D = int(layers[0]["wg"].shape[0])
        if self.nwg <= 0 or self.nwg % H != 0:
            raise ValueError(f"{self.nwg} workgroups are not a multiple of {H} heads")
        nsplit = self.nwg // H
        S = int(cache.max_cache_len)
        self.H, self.Hk, self.Dh, self.d, self.L, self.V, self.S, self.nsplit = H, Hk, Dh, d, L, V, S, nsplit
        for t in (embed, norm, lm_head, *(w for lw in layers for w in lw.values())):
            if t.dtype != torch.bfloat16 or not t.is_contiguous() or t.device != dev:
                raise ValueError("DenseStepDecoder needs contiguous bfloat16 tensors on one device")

        def tagged(n, dt=torch.int32):
            return torch.zeros(n, dtype=dt, device=dev)

        self.XA, self.XB = tagged(d), tagged(d)
        self.QKV, self.A, self.HB = tagged((H + 2 * Hk) * Dh), tagged(H * Dh), tagged(D)
        self.PART, self.CAND = tagged(H * nsplit * (Dh + 2), torch.int64), tagged(self.nwg, torch.int64)
        self.logits = torch.zeros(V, dtype=torch.bfloat16, device=dev)
        self.token_log = torch.zeros(int(max_new_tokens), dtype=torch.int64, device=dev)
        self.state = torch.zeros(8, dtype=torch.int32, device=dev)
        cos, sin = cache.get_rope_tables(seqlen=S, head_dim=Dh, device=dev, dtype=torch.bfloat16)
        self.rope = (cos, sin)
        self._keep = [embed, norm, lm_head, layers]
        ph = []

        def gemv(W, N, K, inp, out, *, norm_w=None, epi=EP_STORE, aux=None, plain=None, shared=False):
            p = Phase()
            p.type, p.epilogue, p.N, p.K, p.nmat, p.mode = PH_GEMV, epi, N, K, len(W), int(mode)
            p.shared_in = int(shared)
            for i, w in enumerate(W):
                if tuple(w.shape) != (N, K):
                    raise ValueError(f"weight {tuple(w.shape)} is not [{N},{K}]")
                p.W[i] = w.data_ptr()
            if norm_w is not None:
                p.norm_w, p.fparam = norm_w.data_ptr(), float(eps)
            p.inp, p.out0 = inp, out
            if aux is not None:
                p.aux0 = aux
            if plain is not None:
                p.plain_out = plain.data_ptr()
            ph.append(p)

        e = Phase()
        e.type, e.N, e.K = PH_EMBED, d, int(embed.shape[0])
        e.W[0] = embed.data_ptr()
        e.out0 = _tb(self.XA, L + 1, 0)
        ph.append(e)
        for l, lw in enumerate(layers):
            cache._ensure_layer_spec(l, h=Hk, dh=Dh)
            kc, vc = cache.key_cache[l][0], cache.value_cache[l][0]
            xin, xmid, xout = _tb(self.XA, L + 1, l), _tb(self.XB, L, l), _tb(self.XA, L + 1, l + 1)
            gemv([lw["wqkv"]], (H + 2 * Hk) * Dh, d, xin, _tb(self.QKV, L, l), norm_w=lw["n1"])
            a = Phase()
            a.type, a.H, a.Hk, a.Dh, a.S, a.nsplit = PH_ATTN, H, Hk, Dh, S, nsplit
            a.fparam = 1.0 / math.sqrt(Dh)
            a.cos, a.sin, a.rope_len = cos.data_ptr(), sin.data_ptr(), int(cos.shape[0])
            a.k_cache, a.v_cache, a.sc_s, a.sc_h = kc.data_ptr(), vc.data_ptr(), kc.stride(0), kc.stride(1)
            a.inp, a.out0 = _tb(self.QKV, L, l), _tb(self.PART, L, l)
            ph.append(a)
            m = Phase()
            m.type, m.H, m.Dh, m.nsplit = PH_MERGE, H, Dh, nsplit
            m.inp, m.out0 = _tb(self.PART, L, l), _tb(self.A, L, l)
            ph.append(m)
            gemv([lw["wo"]], d, H * Dh, _tb(self.A, L, l), xmid, epi=EP_RESID, aux=xin)
            gemv([lw["wg"], lw["wu"]], D, d, xmid, _tb(self.HB, L, l), norm_w=lw["n2"], epi=EP_SWIGLU, shared=True)
            gemv([lw["wd"]], d, D, _tb(self.HB, L, l), xout, epi=EP_RESID, aux=xmid)
            cache._layer_initialized[l] = True
        gemv([lm_head], V, d, _tb(self.XA, L + 1, L), _tb(self.CAND, 1, 0), norm_w=norm, epi=EP_LOGITS, plain=self.logits)
        g = Phase()
        g.type = PH_ARGMAX
        g.inp = _tb(self.CAND, 1, 0)
        g.plain_out = self.token_log.data_ptr()
        ph.append(g)
        self.composed = False
        self.leading = False
        self._names = ["embed"] + [n for _ in range(L) for n in self.PHASE_NAMES[1:]] + ["lm_head", "argmax"]
        self._finish(ph, dev)


def decode_engine_choice() -> str:
    """FLASHSVD_AMD_DECODE_ENGINE = auto (default) | persistent | graph."""
    import os
    v = os.getenv("FLASHSVD_AMD_DECODE_ENGINE", "auto").strip().lower()
    if v not in ("auto", "persistent", "graph"):
        raise ValueError(f"FLASHSVD_AMD_DECODE_ENGINE={v!r}: expected auto, persistent or graph")
    return v


def make_persistent_decoder(model, cache, batch_size: int, *, max_new_tokens: int = 4096):
    """A PersistentDecoder when the engine choice and the model allow it, else None (the caller then uses
    graphs.GraphedDecoder).  With the choice "persistent" an unsupported model raises instead."""
    choice = decode_engine_choice()
    if choice == "graph":
        return None
    try:
        if int(batch_size) != 1:
            raise ValueError("the persistent step decodes one sequence")
        return PersistentDecoder(model, cache, max_new_tokens=max_new_tokens)
    except (ValueError, TypeError, _lib.FlashSVDHipError):
        if choice == "persistent":
            raise
        return None
