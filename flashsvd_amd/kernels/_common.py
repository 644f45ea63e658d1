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
