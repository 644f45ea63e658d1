"""HIP-graph capture of the decode step (hipStreamBeginCapture through torch.cuda.CUDAGraph).

A decode token at 7B shape is ~300 kernel launches of 2-10 us each; replaying them as one graph
removes the per-launch host cost.  Capture follows the warm-up-then-capture protocol of the
reference (benchmark/attn/decode_compare.py:381-411): three eager runs on a side stream, then
capture on that stream.  Nothing in the captured region allocates through hipMalloc or issues
memset nodes: scratch comes from torch's capture pool and counters are reset by the kernels.
"""
from __future__ import annotations

from typing import Callable

import torch


class GraphedCallable:
    """``fn(static_input) -> tensor`` captured once; calls copy the input in and replay."""

    def __init__(self, fn: Callable[[torch.Tensor], torch.Tensor], example: torch.Tensor, warmup: int = 3):
        self.static_in = example.clone()
        side = torch.cuda.Stream(device=example.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                fn(self.static_in)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.static_out = fn(self.static_in)

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        self.static_in.copy_(x)
        self.graph.replay()
        return self.static_out


class GraphedDecoder:
    """Whole-step greedy decode as one graph: embed -> layers -> norm+lm_head -> argmax, with the
    token id and the write position living on the device and advanced inside the graph, so a
    run of N tokens is N replays with no host synchronisation in between."""

    def __init__(self, model, cache, batch_size: int, *, nsplit=None, warmup: int = 3):
        from . import hip_ops
        self.model, self.cache, self.B = model, cache, int(batch_size)
        dev = model.lm_head.weight.device
        cfg = model.config
        H = int(cfg.num_attention_heads)
        Dh = int(getattr(cfg, "head_dim", None) or cfg.hidden_size // H)
        self.nsplit = nsplit or hip_ops.pick_nsplit(cache.max_cache_len, self.B, H, Dh)
        self.attn_ws = hip_ops.attn_workspace(self.B, H, Dh, self.nsplit, dev)
        self.rope = cache.get_rope_tables(seqlen=cache.max_cache_len, head_dim=Dh, device=dev, dtype=model.lm_head.weight.dtype)
        self.tokens = torch.zeros(self.B, 1, dtype=torch.long, device=dev)
        self.positions = torch.zeros(self.B, dtype=torch.int32, device=dev)
        self.logits = None
        self.hidden = None
        self.graph = None
        self.warmup = int(warmup)

    def _step(self):
        logits, hidden = self.model.decode_step(self.tokens, self.cache, self.positions, rope=self.rope,
                                                attn_ws=self.attn_ws, nsplit=self.nsplit, return_hidden=True)
        nxt = logits[:, -1, :].argmax(dim=-1, keepdim=True)
        self.tokens.copy_(nxt)
        self.positions.add_(1)
        return logits, hidden

    def eager_step(self):
        """One un-captured step on the current stream (same kernels, same buffers)."""
        self.logits, self.hidden = self._step()
        self.cache._seen_tokens += 1
        return self.tokens

    def capture(self) -> None:
        tok0, pos0 = self.tokens.clone(), self.positions.clone()
        side = torch.cuda.Stream(device=self.tokens.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, self.warmup)):
                self._step()
                self.positions.copy_(pos0)   # warm-ups rewrite the same slot
                self.tokens.copy_(tok0)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits, self.hidden = self._step()
        self.tokens.copy_(tok0)
        self.positions.copy_(pos0)
        torch.cuda.synchronize()

    def set_state(self, tokens: torch.Tensor, position: int) -> None:
        if position < 0 or position >= self.cache.max_cache_len:
            raise IndexError(f"decode position {position} outside the cache (max {self.cache.max_cache_len})")
        self.tokens.copy_(tokens.reshape(self.B, 1))
        self.positions.fill_(int(position))
        self._host_pos = int(position)

    def step(self) -> torch.Tensor:
        """Replay one token; returns the device tensor holding the next token ids [B,1]."""
        if self.graph is None:
            self.capture()
        if getattr(self, "_host_pos", 0) + 1 > self.cache.max_cache_len:
            raise IndexError(f"decode position {self._host_pos} outside the cache (max {self.cache.max_cache_len})")
        self.graph.replay()
        self._host_pos = getattr(self, "_host_pos", 0) + 1
        self.cache._seen_tokens += 1
        return self.tokens
