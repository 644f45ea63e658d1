"""The low-rank modules inside the model objects the reference actually uses: an UNMODIFIED transformers
LlamaForCausalLM / LlamaDecoderLayer with SVD_LlamaAttention and SVD_LlamaMLP swapped in
(utils/model_utils.py:586-671, benchmark/mlp/bench_svd_llama_decode_graph.py:104-111), decoded through the manual
per-token step (utils/evaluator.py:39-82), and the process-global layer-tail patch of that HF class
(utils/model_utils.py:768-786)."""
import pytest
import torch
from torch import nn

from oracle import flashsvd_oracle as O
from tests.util import assert_close_bf16, bounds, model_from_oracle, rand_bf16

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


class _UV(nn.Module):
    """A wrapped factor pair as SVD-LLM checkpoints hold it: y = u_proj(v_proj(x))."""

    def __init__(self, u, v):
        super().__init__()
        self.v_proj = nn.Linear(v.shape[1], v.shape[0], bias=False)
        self.u_proj = nn.Linear(u.shape[1], u.shape[0], bias=False)
        self.v_proj.weight.data, self.u_proj.weight.data = v.clone(), u.clone()

    def forward(self, x):
        return self.u_proj(self.v_proj(x))


def _mw(dtype=BF16):
    return O.make_model(d=256, n_heads=4, n_kv_heads=2, head_dim=128, ffn=512, attn_rank=64, mlp_rank=128, n_layers=2,
                        vocab=400, dtype=dtype, seed=11, std=0.05)


def _hf_from_oracle(mw):
    """transformers LlamaForCausalLM (its own classes throughout) holding the oracle's weights as wrapped factor pairs,
    then converted in place: only self_attn / mlp of every layer are replaced."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from flashsvd_amd import checkpoint as ck
    m = mw.meta
    cfg = LlamaConfig(vocab_size=m["vocab"], hidden_size=m["d"], intermediate_size=m["ffn"], num_hidden_layers=m["n_layers"],
                      num_attention_heads=mw.n_heads, num_key_value_heads=mw.n_kv_heads, head_dim=mw.head_dim, rms_norm_eps=mw.eps,
                      attention_bias=False, mlp_bias=False, tie_word_embeddings=False, max_position_embeddings=256)
    hf = LlamaForCausalLM(cfg).to(mw.embed.dtype).eval()
    with torch.no_grad():
        hf.model.embed_tokens.weight.copy_(mw.embed)
        hf.lm_head.weight.copy_(mw.lm_head)
        hf.model.norm.weight.copy_(mw.norm)
        for layer, b in zip(hf.model.layers, mw.blocks):
            for p in ("q", "k", "v", "o"):
                setattr(layer.self_attn, f"{p}_proj", _UV(getattr(b, f"{p}_u"), getattr(b, f"{p}_v")))
            for p in ("gate", "up", "down"):
                setattr(layer.mlp, f"{p}_proj", _UV(getattr(b, f"{p}_u"), getattr(b, f"{p}_v")))
            layer.input_layernorm.weight.copy_(b.ln1)
            layer.post_attention_layernorm.weight.copy_(b.ln2)
    hf = hf.cuda()
    for p in hf.parameters():
        p.requires_grad_(False)
    return ck.convert_uv_wrapped_llama(hf)


def _decode(model, prompt, n_new):
    """Prompt pass and greedy tokens through the manual step; returns tokens and the logits of every step."""
    from flashsvd_amd import api
    from flashsvd_amd.runtime.cache import FlashSVDV15DenseKVCache
    Lp = prompt.shape[1]
    cache = FlashSVDV15DenseKVCache(model.config, max_batch_size=1, max_cache_len=Lp + n_new + 2, device="cuda",
                                    dtype=model.lm_head.weight.dtype)
    assert api._can_use_manual_llama_decode_step(model)
    out = api._manual_llama_decode_step(model, prompt.cuda(), past_key_values=cache, cache_position=torch.arange(Lp))
    toks, logits = [], [out.logits[:, -1].clone()]
    tok = out.logits[:, -1].float().argmax(-1, keepdim=True)
    toks.append(int(tok))
    for s in range(n_new - 1):
        out = api._manual_llama_decode_step(model, tok, past_key_values=cache, cache_position=torch.tensor([Lp + s]))
        logits.append(out.logits[:, -1].clone())
        tok = out.logits[:, -1].float().argmax(-1, keepdim=True)
        toks.append(int(tok))
    return toks, torch.stack(logits, 1)


@pytest.fixture()
def unpatched():
    from flashsvd_amd import llama
    llama.unpatch_hf_llama_decoder_layer()
    keep = llama.LAYER_TAIL_GRAPH_ENABLED
    yield
    llama.unpatch_hf_llama_decoder_layer()
    llama.LAYER_TAIL_GRAPH_ENABLED = keep


@pytest.mark.parametrize("dtype", [BF16, torch.float16], ids=["bf16", "fp16"])
def test_modules_inside_unmodified_hf_model(unpatched, monkeypatch, dtype):
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer, LlamaRMSNorm
    from flashsvd_amd import api, llama
    mw = _mw(dtype)
    own = model_from_oracle(mw)
    hf = _hf_from_oracle(mw)
    lay = hf.model.layers[0]
    assert type(lay) is LlamaDecoderLayer and type(lay.input_layernorm) is LlamaRMSNorm
    assert isinstance(lay.self_attn, llama.SVD_LlamaAttention) and isinstance(lay.mlp, llama.SVD_LlamaMLP)
    prompt = torch.randint(0, 400, (1, 19), generator=torch.Generator().manual_seed(2))
    n_new = 8
    ref_tok, _, _, ref_logits = O.greedy_decode(mw, prompt, n_new, "dense", return_logits=True)
    t_own, l_own = _decode(own, prompt, n_new)
    # 1. the HF layer class untouched: its own forward, its own torch RMSNorm and residual adds around our modules
    t_hf, l_hf = _decode(hf, prompt, n_new)
    same = next((s for s in range(n_new) if t_hf[s] != ref_tok[0, s]), n_new)
    assert same >= n_new - 2, f"HF-hosted tokens {t_hf} vs oracle {ref_tok.tolist()}"
    for s in range(same):
        r = ref_logits[:, s].float()
        assert_close_bf16(l_hf[:, s], r, f"HF-hosted logits step {s}", abs_tol=3 * bounds(r)["abs_tol"], rel_tol=3e-2)
    # 2. the process-global patch: same class object, now bit for bit what this package's own decoder layer computes
    api.enable_flashsvd_llama_layer_tail_cuda_graph()
    api.enable_flashsvd_llama_layer_tail_cuda_graph()          # idempotent
    assert type(hf.model.layers[0]) is LlamaDecoderLayer
    t_p, l_p = _decode(hf, prompt, n_new)
    assert t_p == t_own and torch.equal(l_p, l_own), "patched HF layers differ from the package's own model"
    # 3. with the layer_tail scope on, the tail is replayed from a captured graph: still the same bits
    monkeypatch.setenv("FLASH_SVD_MLP_CUDA_GRAPH", "1")
    monkeypatch.setenv("FLASH_SVD_MLP_CUDA_GRAPH_SCOPE", "layer_tail")
    t_g, l_g = _decode(hf, prompt, n_new)
    assert t_g == t_own and torch.equal(l_g, l_own)
    assert any(len(l.mlp._flashsvd_layer_graph_cache) > 0 for l in hf.model.layers), "no layer-tail graph was captured"


def test_hf_layer_with_foreign_attention_graph_scopes(unpatched, monkeypatch):
    """The arrangement of benchmark/mlp/bench_svd_llama_decode_graph.py: an HF LlamaDecoderLayer whose attention is a
    stand-in and whose MLP is SVD_LlamaMLP, run eager / with the MLP graph / with the layer-tail graph (:177-200);
    the three outputs agree and match the oracle's x + mlp(rms(x))."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer
    from flashsvd_amd import api, llama

    class DummySelfAttention(nn.Module):
        def forward(self, hidden_states, **kwargs):
            return torch.zeros_like(hidden_states), None

    d, D, R = 512, 1024, 128
    cfg = LlamaConfig(hidden_size=d, intermediate_size=D, hidden_act="silu", num_attention_heads=4, num_key_value_heads=4,
                      num_hidden_layers=1, max_position_embeddings=256, rms_norm_eps=1e-6, attention_bias=False, mlp_bias=False)
    layer = LlamaDecoderLayer(cfg, layer_idx=0).to(device="cuda", dtype=BF16).eval()
    layer.self_attn = DummySelfAttention()
    mlp = llama.SVD_LlamaMLP(hidden_size=d, intermediate_size=D, hidden_act="silu", ratio=0.5, rank=R).to(device="cuda", dtype=BF16).eval()
    w = {n: rand_bf16(*s, std=0.05, seed=i) for i, (n, s) in enumerate(
        dict(gate_v=(R, d), gate_u=(D, R), up_v=(R, d), up_u=(D, R), down_v=(R, D), down_u=(d, R)).items())}
    for n, t in w.items():
        getattr(mlp, f"{n}_proj").weight.data.copy_(t)
    layer.mlp = mlp
    nw = rand_bf16(d, std=0.1, seed=9) + 1.0
    layer.post_attention_layernorm.weight.data.copy_(nw)
    api.enable_flashsvd_llama_layer_tail_cuda_graph()
    x = rand_bf16(3, 1, d, seed=10)
    z = torch.zeros(1)
    bw = O.BlockWeights(q_v=z, q_u=z, k_v=z, k_u=z, v_v=z, v_u=z, o_v=z, o_u=z, ln1=z, ln2=nw, **w)
    ref = x + O.mlp_forward(bw, O.rms_norm(x, nw, 1e-6))
    outs = {}
    for mode, env in (("eager", {"FLASH_SVD_MLP_CUDA_GRAPH": "0"}),
                      ("mlp_graph", {"FLASH_SVD_MLP_CUDA_GRAPH": "1", "FLASH_SVD_MLP_CUDA_GRAPH_SCOPE": "mlp"}),
                      ("layer_tail_graph", {"FLASH_SVD_MLP_CUDA_GRAPH": "1", "FLASH_SVD_MLP_CUDA_GRAPH_SCOPE": "layer_tail"})):
        monkeypatch.delenv("FLASH_SVD_MLP_CUDA_GRAPH_SCOPE", raising=False)
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        with torch.no_grad():
            out = layer(x.cuda(), use_cache=False)
            out = out[0] if isinstance(out, (tuple, list)) else out
            outs[mode] = out.clone()
            again = layer(x.cuda(), use_cache=False)        # a replay of whatever was captured
            again = again[0] if isinstance(again, (tuple, list)) else again
            assert torch.equal(again, outs[mode])
        assert_close_bf16(outs[mode], ref, mode, **bounds(ref))
    assert torch.equal(outs["eager"], outs["layer_tail_graph"])
    assert len(mlp._flashsvd_layer_graph_cache) == 1
