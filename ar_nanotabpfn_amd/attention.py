"""Attention module and mask descriptors (host-side mirror of the reference's
``ar_tabpfn/model/attention.py``).

The reference expresses masks as ``BlockMask`` objects for ``flex_attention``.
Here a mask is a small structural descriptor — the kernels carry each pattern as
a tile schedule — with the same constructor names and the same caching:

* ``create_dense_mask`` / ``create_context_self_attention_mask``: everything
  attends to everything (attention.py:72-83, :178-196);
* ``DecodeMask`` (inference.py:500-523) and ``TeacherForcingMask``
  (inference.py:525-577) are built by the predictor.

* ``create_row_mask`` (attention.py:86-175): the context / buffer / target mask of the
  training forward; the row attention under it has a device backward pass
  (``attention_kernels.row_mask_attention``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch
from torch import Tensor, nn

from . import attention_kernels as ak

__all__ = [
    "MultiheadAttention",
    "DenseMask",
    "DecodeMask",
    "TeacherForcingMask",
    "RowMask",
    "create_dense_mask",
    "create_context_self_attention_mask",
    "create_row_mask",
    "clear_mask_cache",
]


@dataclass(frozen=True)
class DenseMask:
    """All ``seq_len`` queries see all ``seq_len`` keys."""

    seq_len: int


@dataclass(frozen=True)
class DecodeMask:
    """``num_new`` new rows after ``num_cached`` cached keys; the last new row is the
    target (sees ``kv < num_cached + q``), the others are buffers (``kv <= num_cached + q``)."""

    num_cached: int
    num_new: int


@dataclass(frozen=True)
class TeacherForcingMask:
    """``[Buffer_0..Nt-1, Target_0..Nt-1]`` after ``num_cached`` context keys."""

    num_cached: int
    num_targets: int


@dataclass(frozen=True)
class RowMask:
    """Rows ``[context | buffer | target]`` of the training forward (attention.py:86-175):
    everyone sees the context; buffer row j also sees buffers ``<= j``; target row with offset
    ``o`` sees buffers ``<= o % buffer_len`` while ``o < attending_chunks * buffer_len``; target
    keys are seen by nobody."""

    num_rows: int
    context_len: int
    buffer_len: int
    attending_chunks: int

    def dense(self, device="cpu") -> Tensor:
        """The mask as a ``[R, R]`` boolean tensor (True = attend), for inspection and tests."""
        q = torch.arange(self.num_rows, device=device)[:, None]
        kv = torch.arange(self.num_rows, device=device)[None, :]
        Nc, Nb, A = self.context_len, self.buffer_len, self.attending_chunks
        tstart = Nc + Nb
        prefix = kv < Nc
        ctx_buf = (q < tstart) & (kv < tstart) & (q >= kv)
        off = q - tstart
        tgt_buf = (q >= tstart) & (kv >= Nc) & (kv < tstart) & (off < A * Nb) & ((kv - Nc) <= off % max(Nb, 1))
        return prefix | ctx_buf | tgt_buf


_mask_cache = {}


def create_dense_mask(seq_len: int, device="cuda") -> DenseMask:
    key = ("dense", seq_len, str(device))
    if key not in _mask_cache:
        _mask_cache[key] = DenseMask(seq_len)
    return _mask_cache[key]


def create_context_self_attention_mask(context_len: int, device="cuda") -> DenseMask:
    key = ("context_self", context_len, str(device))
    if key not in _mask_cache:
        _mask_cache[key] = DenseMask(context_len)
    return _mask_cache[key]


def create_row_mask(num_rows: int, context_len: int, buffer_len: int, attending_chunks=None,
                    device="cuda") -> RowMask:
    """Row mask with context / buffer / target sections (attention.py:86-175).  By default half
    of the target chunks attend to the buffer: ``target_len // (2 * buffer_len)`` (:111-112)."""
    target_len = num_rows - context_len - buffer_len
    if attending_chunks is None:
        attending_chunks = target_len // (2 * buffer_len)
    key = ("row", num_rows, context_len, buffer_len, attending_chunks, str(device))
    if key not in _mask_cache:
        _mask_cache[key] = RowMask(num_rows, context_len, buffer_len, attending_chunks)
    return _mask_cache[key]


def clear_mask_cache() -> None:
    _mask_cache.clear()


class _InferenceOnly(torch.autograd.Function):
    """Marks the result of an attention call that has no backward pass: the forward value passes
    through, a gradient arriving here raises instead of silently stopping."""

    @staticmethod
    def forward(ctx, out, *inputs):
        return out.view_as(out)

    @staticmethod
    def backward(ctx, grad):
        raise NotImplementedError("dense attention has no backward pass (it serves the context prefill); "
                                  "only the row attention under a RowMask is differentiable")


class MultiheadAttention(nn.Module):
    """Bias-free q/k/v/out projections around the device attention kernels; returns
    the per-head K and V for caching, like attention.py:31-61."""

    def __init__(self, d_model: int, n_heads: int):
        super().__init__()
        if d_model % n_heads:
            raise ValueError("d_model must be divisible by n_heads")
        self.n_heads = n_heads
        self.head_dim = d_model // n_heads
        self.scale = self.head_dim ** -0.5
        self.q_proj = nn.Linear(d_model, d_model, bias=False)
        self.k_proj = nn.Linear(d_model, d_model, bias=False)
        self.v_proj = nn.Linear(d_model, d_model, bias=False)
        self.out_proj = nn.Linear(d_model, d_model, bias=False)

    def split_heads(self, x: Tensor) -> Tensor:
        """``[B,S,D] -> [B,H,S,Dh]`` as a strided view (no copy)."""
        B, S, _ = x.shape
        return x.view(B, S, self.n_heads, self.head_dim).transpose(1, 2)

    def forward(self, q: Tensor, k: Tensor, v: Tensor, block_mask) -> Tuple[Tensor, Tuple[Tensor, Tensor]]:
        if not isinstance(block_mask, (DenseMask, RowMask)):
            raise NotImplementedError("MultiheadAttention.forward takes a DenseMask or a RowMask; decode and "
                                      "teacher-forcing masks go through the predictor")
        B, Sq, D = q.shape
        qh = self.split_heads(self.q_proj(q))
        kh = self.split_heads(self.k_proj(k))
        vh = self.split_heads(self.v_proj(v))
        if isinstance(block_mask, RowMask):
            if kh.shape[2] != Sq or block_mask.num_rows != Sq:
                raise ValueError("row mask expects num_rows queries and keys")
            out = ak.row_mask_attention(qh, kh, vh, block_mask.context_len, block_mask.buffer_len,
                                        block_mask.attending_chunks)
            return self.out_proj(out.transpose(1, 2).reshape(B, Sq, D)), (kh, vh)
        if kh.shape[2] != Sq or block_mask.seq_len != Sq:
            raise ValueError("dense mask expects equally many queries and keys")
        out = ak.prefill_attention(qh, kh, vh)
        if torch.is_grad_enabled() and (qh.requires_grad or kh.requires_grad or vh.requires_grad):
            out = _InferenceOnly.apply(out, qh, kh, vh)
        return self.out_proj(out.transpose(1, 2).reshape(B, Sq, D)), (kh, vh)
