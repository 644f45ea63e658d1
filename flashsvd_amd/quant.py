"""Group-wise int4 / int8 factor linears under the decode kernels.

``PackedQuantLinear`` keeps the buffers, state-dict keys and quantisation rule of the reference's module of the
same name (src/quant/packed_quant_linear.py:47-172: ``qweight`` uint8 with two int4 columns per byte, ``scales``
fp16 and ``zeros`` int16 per group of input columns, optional ``bias``), so a checkpoint written by the reference's
quantisation scripts loads as it is.  On the GPU a 4-bit module runs on the packed bytes:

* up to ``GEMV_ROWS`` activation rows (decode): ``fsvd_linear_q4`` streams the int4 rows, a quarter of the 16-bit bytes;
* more rows (prefill): the weight is expanded to the activation type by ``fsvd_dequant_q4`` into a scratch matrix that
  lives for the call, and the matrix-core projection runs on it.

Activations are bf16 or fp16; the module computes in the type of its input.

``FLASH_SVD_QUANT_BACKEND`` (the reference's switch, :174-213) picks ``auto`` (the rule above), ``quant`` / ``int4`` /
``packed`` (always the int4 stream) or ``dense`` / ``cached_dense`` / ``fp16`` / ``dequant_cache`` (expand once, keep the
16-bit matrix, run every call on it).  8-bit modules always take the dense route.  Quantising (``pack_weight``) is
offline preparation and runs in torch on whatever device the weight is on.

``replace_linears_with_packed_quant_inplace`` and ``extract_flashsvd_rank_map`` follow src/quant/common.py:80-149.
"""
from __future__ import annotations

import math
import os
from typing import Dict, Iterable, Optional

import torch
import torch.nn as nn

GEMV_ROWS = 16          # activation rows up to which the int4 stream is used (in slices of four)


def pack_int4(q: torch.Tensor) -> torch.Tensor:
    if q.dtype != torch.uint8:
        q = q.to(torch.uint8)
    if q.shape[1] % 2:
        q = torch.cat([q, torch.zeros((q.shape[0], 1), dtype=torch.uint8, device=q.device)], dim=1)
    return (q[:, 0::2] & 0x0F) | ((q[:, 1::2] & 0x0F) << 4)


def unpack_int4(packed: torch.Tensor, in_features: int) -> torch.Tensor:
    out = torch.empty((packed.shape[0], packed.shape[1] * 2), dtype=torch.uint8, device=packed.device)
    out[:, 0::2] = packed & 0x0F
    out[:, 1::2] = (packed >> 4) & 0x0F
    return out[:, :in_features]


class PackedQuantLinear(nn.Module):
    def __init__(self, *, in_features: int, out_features: int, bits: int, group_size: int, bias: bool,
                 compute_dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if bits not in (4, 8):
            raise ValueError(f"PackedQuantLinear only supports 4/8 bits, got {bits}")
        self.in_features, self.out_features = int(in_features), int(out_features)
        self.bits, self.group_size, self.compute_dtype = int(bits), int(group_size), compute_dtype
        groups = 1 if self.group_size <= 0 else int(math.ceil(self.in_features / self.group_size))
        cols = (self.in_features + 1) // 2 if self.bits == 4 else self.in_features
        self.register_buffer("qweight", torch.zeros(self.out_features, cols, dtype=torch.uint8), persistent=True)
        self.register_buffer("scales", torch.zeros(self.out_features, groups, dtype=torch.float16), persistent=True)
        self.register_buffer("zeros", torch.zeros(self.out_features, groups, dtype=torch.int16), persistent=True)
        if bias:
            self.register_buffer("bias", torch.zeros(self.out_features, dtype=compute_dtype), persistent=True)
        else:
            self.bias = None
        self._dense = None          # (key, bf16 weight) kept by the dense backend

    # ---- quantisation ----------------------------------------------------------------------------------
    @classmethod
    def from_linear(cls, linear: nn.Linear, *, bits: int, group_size: int, sym: bool,
                    compute_dtype: Optional[torch.dtype] = None) -> "PackedQuantLinear":
        weight = linear.weight.detach()
        bias = None if linear.bias is None else linear.bias.detach()
        module = cls(in_features=int(linear.in_features), out_features=int(linear.out_features), bits=int(bits),
                     group_size=int(group_size), bias=bias is not None, compute_dtype=compute_dtype or weight.dtype)
        module.pack_weight(weight, bias=bias, sym=bool(sym))
        return module

    def pack_weight(self, weight: torch.Tensor, *, bias: Optional[torch.Tensor], sym: bool) -> None:
        """Min/max quantisation per group of input columns: scale = (max - min) / (2^bits - 1), zero = round(-min / scale)
        (``sym``: range centred, zero = 2^(bits-1)); an all-zero group takes the range [-1, 1]."""
        weight = weight.detach().to(torch.float32)
        if tuple(weight.shape) != (self.out_features, self.in_features):
            raise ValueError(f"weight shape mismatch: got {tuple(weight.shape)}, expected {(self.out_features, self.in_features)}")
        group = self.in_features if self.group_size <= 0 else int(self.group_size)
        maxq = float((1 << self.bits) - 1)
        qs, ss, zs = [], [], []
        for start in range(0, self.in_features, group):
            chunk = weight[:, start:min(self.in_features, start + group)]
            xmin, xmax = chunk.min(dim=1).values, chunk.max(dim=1).values
            if sym:
                xmax = torch.maximum(xmax.abs(), xmin.abs())
                xmin = -xmax
            dead = (xmin == 0) & (xmax == 0)
            xmin = torch.where(dead, torch.full_like(xmin, -1.0), xmin)
            xmax = torch.where(dead, torch.full_like(xmax, 1.0), xmax)
            scale = (xmax - xmin) / maxq
            scale = torch.where(scale == 0, torch.ones_like(scale), scale)
            zero = torch.full_like(scale, int((maxq + 1) / 2)) if sym else torch.round(-xmin / scale)
            qs.append(torch.clamp(torch.round(chunk / scale.unsqueeze(1)) + zero.unsqueeze(1), 0, maxq).to(torch.uint8))
            ss.append(scale.to(torch.float16))
            zs.append(zero.to(torch.int16))
        q = torch.cat(qs, dim=1).contiguous()
        self.scales = torch.stack(ss, dim=1).contiguous()
        self.zeros = torch.stack(zs, dim=1).contiguous()
        self.qweight = pack_int4(q).contiguous() if self.bits == 4 else q
        if self.bias is not None:
            self.bias = bias.to(dtype=self.compute_dtype).contiguous() if bias is not None else None
        self._dense = None

    # ---- dense form --------------------------------------------------------------------------------------
    def dequantize(self, *, dtype: Optional[torch.dtype] = None, device=None) -> torch.Tensor:
        """scale * (q - zero), rounded once to ``dtype``.  4-bit buffers on the GPU with a bf16 or fp16 result go through
        the HIP expansion kernel; everything else is tensor arithmetic (tests, CPU tools)."""
        dtype = dtype or self.compute_dtype
        device = torch.device(device) if device is not None else self.qweight.device
        if self.bits == 4 and dtype in (torch.bfloat16, torch.float16) and device.type == "cuda" and self.qweight.is_cuda:
            from . import hip_ops
            return hip_ops.dequant_q4(self.qweight, self.scales, self.zeros, in_features=self.in_features,
                                      group_size=self.group_size, dtype=dtype)
        q = (unpack_int4(self.qweight, self.in_features) if self.bits == 4 else self.qweight).to(device=device, dtype=torch.float32)
        scales = self.scales.to(device=device, dtype=torch.float32)
        zeros = self.zeros.to(device=device, dtype=torch.float32)
        group = self.in_features if self.group_size <= 0 else int(self.group_size)
        cols = [scales[:, g].unsqueeze(1) * (q[:, g * group:min(self.in_features, (g + 1) * group)] - zeros[:, g].unsqueeze(1))
                for g in range(int(scales.shape[1]))]
        return torch.cat(cols, dim=1).to(dtype)

    @property
    def weight(self) -> torch.Tensor:
        return self.dequantize()

    def _backend(self) -> str:
        mode = str(os.environ.get("FLASH_SVD_QUANT_BACKEND", "auto")).strip().lower()
        if mode in ("dense", "cached_dense", "fp16", "dequant_cache"):
            return "dense"
        if mode in ("quant", "int4", "int8", "packed"):
            return "quant"
        if mode in ("auto", "", "1", "on"):
            return "auto"
        raise ValueError(f"FLASH_SVD_QUANT_BACKEND={mode!r}: expected auto, quant or dense (there is no path without the GPU kernels)")

    def _cached_dense(self, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        key = (self.qweight.data_ptr(), self.scales.data_ptr(), self.qweight.device, dtype)
        if self._dense is None or self._dense[0] != key:
            self._dense = (key, self.dequantize(dtype=dtype))
        return self._dense[1]

    def streams_int4(self, rows: int) -> bool:
        """True when a call with ``rows`` activation rows reads the packed bytes directly."""
        if self.bits != 4 or self.in_features % 256:
            return False
        g = self.group_size
        if 0 < g < self.in_features and (g < 32 or g & (g - 1)):
            return False
        backend = self._backend()
        return backend == "quant" or (backend == "auto" and rows <= GEMV_ROWS)

    def run(self, x: torch.Tensor, *, norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
            residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The projection with the fused prologue / epilogue of the 16-bit kernels, in the type of ``x`` (bf16 or fp16)."""
        from . import hip_ops
        if not x.is_cuda:
            raise RuntimeError("PackedQuantLinear runs on the GPU kernels only; use dequantize() for CPU-side inspection")
        rows = x.numel() // max(1, x.shape[-1])
        if self.streams_int4(rows):
            bias = self.bias if self.bias is None or self.bias.dtype == x.dtype else self.bias.to(x.dtype)
            return hip_ops.linear_q4(x, self.qweight, self.scales, self.zeros, group_size=self.group_size, bias=bias,
                                     norm_weight=norm_weight, eps=eps, residual=residual, out=out)
        if x.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"PackedQuantLinear computes in bfloat16 or float16, got {x.dtype}")
        w = self._cached_dense(x.dtype) if self._backend() == "dense" else self.dequantize(dtype=x.dtype)
        bias = self.bias if self.bias is None or self.bias.dtype == x.dtype else self.bias.to(x.dtype)
        return hip_ops.linear(x, w, bias, norm_weight=norm_weight, eps=eps, residual=residual, out=out)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.run(x)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, bits={self.bits}, group_size={self.group_size}"


def apply_linear(mod: nn.Module, x: torch.Tensor, *, norm_weight=None, eps: float = 1e-6, residual=None, out=None) -> torch.Tensor:
    """One factor projection through the kernel that fits the module: int4 stream or bf16."""
    if isinstance(mod, PackedQuantLinear):
        return mod.run(x, norm_weight=norm_weight, eps=eps, residual=residual, out=out)
    from . import hip_ops
    return hip_ops.linear(x, mod.weight, getattr(mod, "bias", None), norm_weight=norm_weight, eps=eps, residual=residual, out=out)


def pack_quant_rows(mods) -> Optional[tuple]:
    """(qweight, scales, zeros) with the rows of all ``mods`` one below the other, so that projections sharing their input
    are one weight stream; the modules' buffers become row slices of the packed tensors (no second copy).  None when the
    modules cannot share a launch (mixed types, widths, group sizes, or a bias)."""
    mods = list(mods)
    if not mods or not all(isinstance(m, PackedQuantLinear) for m in mods):
        return None
    m0 = mods[0]
    if m0.bits != 4 or any(m.bits != 4 or m.in_features != m0.in_features or m.group_size != m0.group_size or m.bias is not None
                           or m.qweight.device != m0.qweight.device for m in mods):
        return None
    packed = []
    for name in ("qweight", "scales", "zeros"):
        parts = [getattr(m, name) for m in mods]
        base, row, shared = parts[0], 0, True
        for t in parts:
            if t.untyped_storage().data_ptr() != base.untyped_storage().data_ptr() or not t.is_contiguous() or \
                    t.storage_offset() != base.storage_offset() + row * base.shape[1]:
                shared = False
                break
            row += t.shape[0]
        if shared:
            packed.append(torch.as_strided(base, (row, base.shape[1]), (base.shape[1], 1), base.storage_offset()))
            continue
        cat = torch.cat(parts, dim=0).contiguous()
        row = 0
        for m, t in zip(mods, parts):
            setattr(m, name, cat[row:row + t.shape[0]])
            row += t.shape[0]
        packed.append(cat)
    for m in mods:
        m._dense = None
    return tuple(packed)


def is_quantized(*mods) -> bool:
    return any(isinstance(m, PackedQuantLinear) for m in mods)


# ---- model-level helpers (src/quant/common.py) ---------------------------------------------------------
def proj_out_features(module) -> int:
    if module is None:
        return 0
    if hasattr(module, "out_features"):
        return int(module.out_features)
    weight = getattr(module, "weight", None)
    return int(weight.shape[0]) if weight is not None else 0


def extract_flashsvd_rank_map(model: nn.Module) -> Dict[str, Dict[str, Dict[str, int]]]:
    rank_map: Dict[str, Dict[str, Dict[str, int]]] = {}
    for idx, layer in enumerate(getattr(getattr(model, "model", None), "layers", None) or ()):
        attn, mlp = getattr(layer, "self_attn", None), getattr(layer, "mlp", None)
        if attn is None or mlp is None:
            continue
        rank_map[str(idx)] = {
            "self_attn": {f"{p}_rank": proj_out_features(getattr(attn, f"{p}_v_proj", None)) for p in ("q", "k", "v", "o")},
            "mlp": {f"{p}_rank": proj_out_features(getattr(mlp, f"{p}_v_proj", None)) for p in ("gate", "up", "down")},
        }
    return rank_map


def get_submodule(root: nn.Module, name: str) -> nn.Module:
    cur = root
    for part in name.split("."):
        cur = getattr(cur, part)
    return cur


def set_submodule(root: nn.Module, name: str, new_module: nn.Module) -> None:
    parts = name.split(".")
    parent = root
    for part in parts[:-1]:
        parent = getattr(parent, part)
    setattr(parent, parts[-1], new_module)


def factor_linear_names(model: nn.Module) -> list:
    """Names of every low-rank factor linear of the decoder layers (the modules the reference's scripts quantise)."""
    names = []
    for idx, _ in enumerate(model.model.layers):
        for blk, projs in (("self_attn", ("q", "k", "v", "o")), ("mlp", ("gate", "up", "down"))):
            for p in projs:
                names += [f"model.layers.{idx}.{blk}.{p}_v_proj", f"model.layers.{idx}.{blk}.{p}_u_proj"]
    return names


def replace_linears_with_packed_quant_inplace(model: nn.Module, *, module_names: Iterable[str], bits: int, group_size: int,
                                              sym: bool, compute_dtype: Optional[torch.dtype] = None) -> int:
    replaced, seen = 0, set()
    for name in module_names:
        if not name or name in seen:
            continue
        seen.add(name)
        module = get_submodule(model, name)
        if not isinstance(module, nn.Linear):
            continue
        set_submodule(model, name, PackedQuantLinear.from_linear(module, bits=int(bits), group_size=int(group_size), sym=bool(sym),
                                                                 compute_dtype=compute_dtype or module.weight.dtype))
        replaced += 1
    for layer in getattr(getattr(model, "model", None), "layers", None) or ():
        if hasattr(layer.self_attn, "_reset_runtime_state"):
            layer.self_attn._reset_runtime_state()
        if hasattr(layer.mlp, "_packed_gu_v"):
            layer.mlp._packed_gu_v = None
            layer.mlp._packed_key = None
        for name in ("_flashsvd_graph_cache", "_flashsvd_layer_graph_cache"):  # captured graphs point at the old weights
            if isinstance(getattr(layer.mlp, name, None), dict):
                getattr(layer.mlp, name).clear()
    return replaced
