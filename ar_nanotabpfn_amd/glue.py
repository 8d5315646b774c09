"""Row-wise glue ops of the transformer layer (residual + bias + LayerNorm, bias + GELU).

On a HIP device they are single fused kernels of ``libartab_attention.so``
(``artab_add_layernorm``, ``artab_bias_gelu``); on CPU tensors — the model itself is
plain PyTorch and can be built and inspected anywhere — the same arithmetic is spelled
with torch ops.  The attention path has no such CPU spelling.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import _lib

__all__ = ["add_layer_norm", "bias_gelu"]


def _rows2d(t: Tensor) -> Tensor:
    """View as [rows, D] with unit column stride (copy only if the layout forces one)."""
    t2 = t.reshape(-1, t.shape[-1])
    if t2.stride(1) != 1 or t2.stride(0) % 4 or t2.data_ptr() % 16:
        t2 = t2.contiguous()
    return t2


def _ptr(t: Optional[Tensor]):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def add_layer_norm(x: Tensor, y: Optional[Tensor], bias: Optional[Tensor], norm: nn.LayerNorm) -> Tensor:
    """``norm(x + y + bias)`` in one pass; ``y`` and ``bias`` are optional."""
    D = x.shape[-1]
    if not x.is_cuda or D % 4 or D > 1024 or x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        t = x if y is None else x + y
        if bias is not None:
            t = t + bias
        return norm(t)
    lib = _lib.load()
    x2 = _rows2d(x)
    y2 = _rows2d(y) if y is not None else None
    out = torch.empty((x2.shape[0], D), device=x.device, dtype=x.dtype)
    _lib.check(
        lib.artab_add_layernorm(
            _ptr(x2), x2.stride(0), _ptr(y2), y2.stride(0) if y2 is not None else 0, _ptr(bias),
            _ptr(norm.weight), _ptr(norm.bias), _ptr(out), x2.shape[0], D, float(norm.eps),
            _lib.dtype_code(x.dtype), _lib.current_stream(x.device),
        )
    )
    return out.view(x.shape)


def bias_gelu(x: Tensor, bias: Optional[Tensor]) -> Tensor:
    """``gelu(x + bias)``, erf form."""
    D = x.shape[-1]
    if not x.is_cuda or D % 4 or x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        return F.gelu(x if bias is None else x + bias)
    lib = _lib.load()
    x2 = _rows2d(x)
    out = torch.empty((x2.shape[0], D), device=x.device, dtype=x.dtype)
    _lib.check(
        lib.artab_bias_gelu(_ptr(x2), x2.stride(0), _ptr(bias), _ptr(out), x2.shape[0], D,
                            _lib.dtype_code(x.dtype), _lib.current_stream(x.device))
    )
    return out.view(x.shape)
