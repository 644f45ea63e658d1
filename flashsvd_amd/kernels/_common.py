"""Shared plumbing of the operator wrappers: dtype codes, zero-initialised scratch, stream."""
from __future__ import annotations

import torch

from .. import _lib

DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
_SCRATCH: dict = {}


def dtype_code(t: torch.Tensor) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}; expected bfloat16, float16 or float32") from None


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def scratch(device: torch.device, nbytes: int, tag: str) -> torch.Tensor:
    """A cached, zero-initialised int32 buffer of at least ``nbytes`` (the kernels leave their
    counters at zero, so one buffer per (device, tag) serves every call on that stream; calls that
    overlap on different streams must not share it)."""
    key = (device, tag)
    buf = _SCRATCH.get(key)
    need = max(1, (int(nbytes) + 3) // 4)
    if buf is None or buf.numel() < need:
        buf = torch.zeros(need, dtype=torch.int32, device=device)
        _SCRATCH[key] = buf
    return buf


def check(name: str, rc: int) -> None:
    _lib.check(name, rc)


def inner_contig(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


_TRANSPOSED: dict = {}
TWIN_BUILDS = [0]          # how many twins have been built (tests count copies with it)


def linear_layout_of(W: torch.Tensor) -> torch.Tensor:
    """The nn.Linear-layout twin ``W.T.contiguous()`` of a reference-layout operand ``W [K, N]`` (``x @ W``), built once
    per tensor and kept while the tensor lives and is not written to (keyed by storage address, shape, strides and
    version counter, checked against a weak reference).  The reference re-lays its operands out on every call
    (``.contiguous()``, kernels/mlp/decode/dual_split_triton.py:576-581; ``pack_qkv_shared_bases`` is the same idea for
    the head bases); here the copy is what lets the reference-layout operators stream weights the way the product path
    does — every output a contiguous row."""
    import weakref
    key = (W.data_ptr(), tuple(W.shape), tuple(W.stride()), W._version, W.dtype)
    hit = _TRANSPOSED.get(key)
    if hit is not None and hit[0]() is W:
        return hit[1]
    out = W.t().contiguous()
    TWIN_BUILDS[0] += 1
    if len(_TRANSPOSED) > 512:
        _TRANSPOSED.clear()

    def _drop(ref, key=key):                     # the operand died: its twin goes with it
        cur = _TRANSPOSED.get(key)
        if cur is not None and cur[0] is ref:
            del _TRANSPOSED[key]
    _TRANSPOSED[key] = (weakref.ref(W, _drop), out)
    return out
