"""Row-wise glue ops of the transformer layer (residual + bias + LayerNorm, bias + GELU)
and the two whole-layer fusions around the attention call.

On a HIP device they are single fused kernels of ``libartab_attention.so``
(``artab_add_layernorm``, ``artab_bias_gelu``, ``artab_layer_pre``, ``artab_layer_post``);
on CPU tensors — the model itself is
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

__all__ = ["add_layer_norm", "bias_gelu", "layer_fusable", "pack_weight", "layer_pre", "layer_post", "layer_post_pre", "SampleEmbedStep", "DecodeStepBoundary"]


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


_FUSED_WIDTHS = (128, 256, 512)


def layer_fusable(x: Tensor, d_model: int, d_ff: int) -> bool:
    """True when ``layer_pre`` / ``layer_post`` cover this layer (16-bit dtype on a HIP device,
    widths the kernels are built for)."""
    return (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16)
            and d_model in _FUSED_WIDTHS and d_ff in _FUSED_WIDTHS)


def _rows16(t: Tensor) -> Tensor:
    """[rows, D] view with unit column stride, 16-byte aligned rows."""
    t2 = t.reshape(-1, t.shape[-1])
    if t2.stride(1) != 1 or t2.stride(0) % 8 or t2.data_ptr() % 16:
        t2 = t2.contiguous()
    return t2


def pack_weight(w: Tensor) -> Tensor:
    """A ``torch.nn.Linear`` weight ``[N, K]`` in the operand order of the fused layer kernels
    (``[N/32, K/16, 64, 8]``, see ``artab_pack_linear_weight``); done once per weight."""
    w = w.detach().contiguous()
    N, K = w.shape
    packed = torch.empty((N // 32, K // 16, 64, 8), device=w.device, dtype=w.dtype)
    _lib.check(_lib.load().artab_pack_linear_weight(_ptr(w), _ptr(packed), N, K, _lib.dtype_code(w.dtype),
                                                    _lib.current_stream(w.device)))
    return packed


def layer_pre(x: Tensor, w_fo: Tensor, norm1: nn.LayerNorm, w_qkv: Tensor):
    """``y = norm1(x + x @ W_fo.T)``, ``qkv = y @ W_qkv.T`` in one launch; ``w_fo`` and
    ``w_qkv`` are the packed forms (``pack_weight``) of ``W_fo [D, D]`` and ``W_qkv [3D, D]``.

    Returns ``(y [rows, D], qkv [rows, 3D])``."""
    D = x.shape[-1]
    x2 = _rows16(x)
    rows = x2.shape[0]
    y = torch.empty((rows, D), device=x.device, dtype=x.dtype)
    qkv = torch.empty((rows, 3 * D), device=x.device, dtype=x.dtype)
    _lib.check(
        _lib.load().artab_layer_pre(
            _ptr(x2), x2.stride(0), _ptr(w_fo), _ptr(norm1.weight), _ptr(norm1.bias), float(norm1.eps),
            _ptr(w_qkv), _ptr(y), _ptr(qkv), rows, D, _lib.dtype_code(x.dtype), _lib.current_stream(x.device),
        )
    )
    return y, qkv


def layer_post(attn: Tensor, y: Tensor, w_o: Tensor, norm2: nn.LayerNorm, w_1: Tensor, b_1: Optional[Tensor],
               w_2: Tensor, b_2: Optional[Tensor], norm3: nn.LayerNorm) -> Tensor:
    """``x1 = norm2(y + attn @ W_o.T)``; ``norm3(x1 + gelu(x1 @ W_1.T + b_1) @ W_2.T + b_2)`` in
    one launch; ``w_o``, ``w_1``, ``w_2`` are packed (``pack_weight``).

    ``attn`` and ``y`` are ``[rows, D]``-shaped (any leading dims); returns ``[rows, D]``."""
    D = y.shape[-1]
    y2 = _rows16(y)
    rows = y2.shape[0]
    out = torch.empty((rows, D), device=y.device, dtype=y.dtype)
    if hasattr(attn, "desc"):  # unmerged partials: merged while the kernel loads its input
        _lib.check(
            _lib.load().artab_layer_post_from_partials(
                ctypes.byref(attn.desc), _ptr(y2), y2.stride(0), _ptr(w_o), _ptr(norm2.weight), _ptr(norm2.bias),
                float(norm2.eps), _ptr(w_1), _ptr(b_1), _ptr(w_2), _ptr(b_2),
                _ptr(norm3.weight), _ptr(norm3.bias), float(norm3.eps), _ptr(out), rows, D, w_1.shape[0] * 32,
                _lib.dtype_code(y.dtype), _lib.current_stream(y.device),
            )
        )
        return out
    a2 = _rows16(attn)
    _lib.check(
        _lib.load().artab_layer_post(
            _ptr(a2), a2.stride(0), _ptr(y2), y2.stride(0), _ptr(w_o), _ptr(norm2.weight), _ptr(norm2.bias),
            float(norm2.eps), _ptr(w_1), _ptr(b_1), _ptr(w_2), _ptr(b_2),
            _ptr(norm3.weight), _ptr(norm3.bias), float(norm3.eps), _ptr(out), rows, D, w_1.shape[0] * 32,
            _lib.dtype_code(y.dtype), _lib.current_stream(y.device),
        )
    )
    return out


def layer_post_pre(attn: Tensor, y: Tensor, w_o: Tensor, norm2: nn.LayerNorm, w_1: Tensor, b_1: Optional[Tensor],
                   w_2: Tensor, b_2: Optional[Tensor], norm3: nn.LayerNorm, next_w_fo: Tensor,
                   next_norm1: nn.LayerNorm, next_w_qkv: Tensor):
    """``layer_post`` of one layer and ``layer_pre`` of the next in one launch; the layer output
    between them is not materialised.  Returns the next layer's ``(y [rows, D], qkv [rows, 3D])``."""
    D = y.shape[-1]
    y2 = _rows16(y)
    rows = y2.shape[0]
    y_next = torch.empty((rows, D), device=y.device, dtype=y.dtype)
    qkv_next = torch.empty((rows, 3 * D), device=y.device, dtype=y.dtype)
    if hasattr(attn, "desc"):  # unmerged partials
        _lib.check(
            _lib.load().artab_layer_post_pre_from_partials(
                ctypes.byref(attn.desc), _ptr(y2), y2.stride(0), _ptr(w_o), _ptr(norm2.weight), _ptr(norm2.bias),
                float(norm2.eps), _ptr(w_1), _ptr(b_1), _ptr(w_2), _ptr(b_2),
                _ptr(norm3.weight), _ptr(norm3.bias), float(norm3.eps),
                _ptr(next_w_fo), _ptr(next_norm1.weight), _ptr(next_norm1.bias), float(next_norm1.eps),
                _ptr(next_w_qkv), _ptr(y_next), _ptr(qkv_next), rows, D, w_1.shape[0] * 32,
                _lib.dtype_code(y.dtype), _lib.current_stream(y.device),
            )
        )
        return y_next, qkv_next
    a2 = _rows16(attn)
    _lib.check(
        _lib.load().artab_layer_post_pre(
            _ptr(a2), a2.stride(0), _ptr(y2), y2.stride(0), _ptr(w_o), _ptr(norm2.weight), _ptr(norm2.bias),
            float(norm2.eps), _ptr(w_1), _ptr(b_1), _ptr(w_2), _ptr(b_2),
            _ptr(norm3.weight), _ptr(norm3.bias), float(norm3.eps),
            _ptr(next_w_fo), _ptr(next_norm1.weight), _ptr(next_norm1.bias), float(next_norm1.eps), _ptr(next_w_qkv),
            _ptr(y_next), _ptr(qkv_next), rows, D, w_1.shape[0] * 32,
            _lib.dtype_code(y.dtype), _lib.current_stream(y.device),
        )
    )
    return y_next, qkv_next


class SampleEmbedStep:
    """The tail of a decode step as one launch (``artab_decode_sample_embed``): final norm,
    mixture head, one draw per trajectory, prediction write, embedding of the next
    ``[buffer, target]`` pair.  Built once per (model, batch, targets); ``__call__`` only
    launches, so it can be recorded into a graph.

    ``x_mean [B,Nt]``: feature mean of every target row; ``rand_u``/``rand_n [Nt,B]`` float32
    variates (refilled by the caller before each sampling run); ``step``: int32 device scalar;
    ``preds [B,Nt]``; ``emb [B,2,D]``.
    """

    MAX_COMPONENTS = 10

    @staticmethod
    def supported(embedder, backbone, head, x: Tensor) -> bool:
        D = backbone.norm.normalized_shape[0]
        lin1, lin2 = head.head[0], head.head[2]
        return (layer_fusable(x, D, lin1.out_features) and head.dim_y == 1
                and head.num_components <= SampleEmbedStep.MAX_COMPONENTS
                and lin2.out_features == 3 * head.num_components)

    def __init__(self, embedder, backbone, head, ar_tokens: Tensor, x_mean: Tensor, rand_u: Tensor, rand_n: Tensor,
                 step: Tensor, preds: Tensor, emb: Tensor, advance: Optional[Tensor] = None):
        lin1, lin2 = head.head[0], head.head[2]
        dev, dt = emb.device, emb.dtype
        B, Nt = preds.shape
        D, F_ = lin1.in_features, lin1.out_features
        assert x_mean.shape == (B, Nt) and rand_u.shape == (Nt, B) and rand_n.shape == (Nt, B)
        assert rand_u.dtype == torch.float32 and rand_n.dtype == torch.float32 and step.dtype == torch.int32
        assert emb.shape == (B, 2, D) and emb.is_contiguous() and preds.is_contiguous() and x_mean.is_contiguous()
        w2 = torch.zeros((32, F_), device=dev, dtype=dt)
        w2[: lin2.out_features] = lin2.weight.detach()
        b2 = torch.zeros(32, device=dev, dtype=dt)
        if lin2.bias is not None:
            b2[: lin2.out_features] = lin2.bias.detach()
        # everything the launch points at is kept alive here
        self._keep = dict(
            w_h1=pack_weight(lin1.weight), w_h2=pack_weight(w2), b_h2=b2,
            w_x=embedder.x_embed.weight.detach().reshape(-1).contiguous(),
            w_y=embedder.y_embed.weight.detach().reshape(-1).contiguous(),
            ar_tokens=ar_tokens.detach().contiguous(), x_mean=x_mean, rand_u=rand_u, rand_n=rand_n, step=step,
            preds=preds, emb=emb,
        )
        k = self._keep
        self.dtype_code = _lib.dtype_code(dt)
        self.device = dev
        a = _lib.ArtabSampleEmbedArgs()
        a.norm_gamma, a.norm_beta, a.eps = backbone.norm.weight.data_ptr(), backbone.norm.bias.data_ptr(), backbone.norm.eps
        a.w_h1, a.b_h1 = k["w_h1"].data_ptr(), (lin1.bias.data_ptr() if lin1.bias is not None else None)
        a.w_h2, a.b_h2 = k["w_h2"].data_ptr(), b2.data_ptr()
        a.mean_bias, a.std_bias, a.weight_bias = (head.mean_bias.data_ptr(), head.std_bias.data_ptr(),
                                                  head.weight_bias.data_ptr())
        a.K, a.std_min, a.std_max = head.num_components, float(head.std_min), 2.0
        a.rand_u, a.rand_n, a.x_mean = rand_u.data_ptr(), rand_n.data_ptr(), x_mean.data_ptr()
        a.w_x, a.b_x = k["w_x"].data_ptr(), embedder.x_embed.bias.data_ptr()
        a.w_y, a.b_y = k["w_y"].data_ptr(), embedder.y_embed.bias.data_ptr()
        a.markers = embedder.marker_embed.weight.data_ptr()
        a.ar_tokens, a.bs = k["ar_tokens"].data_ptr(), ar_tokens.shape[0]
        a.step, a.Nt = step.data_ptr(), Nt
        a.preds, a.emb_next = preds.data_ptr(), emb.data_ptr()
        a.B, a.D, a.F = B, D, F_
        # ``advance``: contiguous int32 loop counters that the launch increments itself (the last
        # workgroup to finish does it), instead of a separate add launched by the caller
        self.advances = advance is not None
        if advance is not None:
            assert advance.dtype == torch.int32 and advance.is_contiguous() and 1 <= advance.numel() <= 8
            k["advance"] = advance
            k["ticket"] = torch.zeros(1, device=dev, dtype=torch.int32)
            a.advance, a.n_advance, a.ticket = advance.data_ptr(), advance.numel(), k["ticket"].data_ptr()
        self.args = a

    def __call__(self, x_last: Tensor) -> None:
        """``x_last [B,2,D]`` (or ``[B,1,D]``): output of the last layer; its last row per
        trajectory is the target row."""
        B, N, D = x_last.shape
        if x_last.stride(2) != 1 or x_last.stride(0) % 8:
            x_last = x_last.contiguous()
        tgt = x_last[:, N - 1]
        self.args.x_last, self.args.ld_row = tgt.data_ptr(), tgt.stride(0)
        _lib.check(_lib.load().artab_decode_sample_embed(ctypes.byref(self.args), self.dtype_code,
                                                         _lib.current_stream(self.device)))


class DecodeStepBoundary:
    """Everything between the last attention call of one decode step and the first of the next
    as one launch (``artab_decode_step_boundary``): the last layer's ``finish`` on the target
    rows, the step tail (``SampleEmbedStep``) and the first layer's ``pre_attention`` on the rows
    the tail has embedded.  Row for row the results are those of the three launches.

    ``y_next [B,2,D]`` / ``qkv_next [B,2,3D]`` receive the first layer's normed feature stage and
    projections of the next step; ``state`` is the ``(y, q, k, v)`` tuple over them in the form
    ``TwoStageTransformerLayer.pre_attention`` returns.
    """

    MAX_TRAJECTORIES = 4096  # twice as many rows still take the 16-row tiles of the layer kernels
    # At d_model 512 a workgroup streams 3 MB of weights and is bound by that; eight trajectories
    # per workgroup instead of sixteen rows then double the traffic of the first two parts for
    # nothing (measured at B=2048, d_model 512: 457 against 462 target-steps/s with three launches).
    MAX_WIDTH = 256

    @staticmethod
    def supported(tail: "SampleEmbedStep", first_layer, last_layer, x: Tensor) -> bool:
        F_ = last_layer.ff[0].out_features
        return (tail is not None and tail.advances and tail.args.F == F_ and first_layer.ff[0].out_features == F_
                and first_layer.attn_rows.n_heads == last_layer.attn_rows.n_heads
                and last_layer.fused_for(x) and first_layer.fused_for(x)
                and tail.args.B <= DecodeStepBoundary.MAX_TRAJECTORIES
                and tail.args.D <= DecodeStepBoundary.MAX_WIDTH
                and _lib.tuning.get("ARTAB_TILE_ROWS") in (None, 16))

    def __init__(self, tail: "SampleEmbedStep", first_layer, last_layer, y_next: Tensor, qkv_next: Tensor):
        B, D = tail.args.B, tail.args.D
        assert y_next.shape == (B, 2, D) and qkv_next.shape == (B, 2, 3 * D)
        assert y_next.is_contiguous() and qkv_next.is_contiguous()
        self.tail, self.first, self.last = tail, first_layer, last_layer
        self.y_next, self.qkv_next = y_next, qkv_next
        a = first_layer.attn_rows
        qkv = qkv_next.view(B, 2, 3, a.n_heads, a.head_dim)
        self.state = (y_next, qkv[:, :, 0].transpose(1, 2), qkv[:, :, 1].transpose(1, 2), qkv[:, :, 2].transpose(1, 2))

    def load_state(self, emb: Tensor) -> None:
        """The state a launch would have left for the embedded rows ``emb [B,2,D]``."""
        p_fo, p_qkv = self.first.packed_weights()[:2]
        y, qkv = layer_pre(emb, p_fo, self.first.norm1, p_qkv)
        self.y_next.view(y.shape).copy_(y)
        self.qkv_next.view(qkv.shape).copy_(qkv)

    def __call__(self, y: Tensor, attn) -> None:
        """``y [B,1,D]``: the last layer's normed feature stage of the target rows (any row
        stride); ``attn``: their attention output ``[B,H,1,Dh]`` or its unmerged partials."""
        last, first = self.last, self.first
        B, D = self.tail.args.B, self.tail.args.D
        y2 = y.reshape(B, D) if y.stride(-1) == 1 and y.stride(0) % 8 == 0 else y.reshape(B, D).contiguous()
        if y2.data_ptr() % 16:
            y2 = y2.contiguous()
        p_o, p_1, p_2 = last.packed_weights()[2:]
        n_fo, n_qkv = first.packed_weights()[:2]
        if hasattr(attn, "desc"):
            parts, a_ptr, lda = ctypes.byref(attn.desc), None, 0
        else:
            a2 = _rows16(attn.transpose(1, 2).reshape(B, D))
            parts, a_ptr, lda = None, _ptr(a2), a2.stride(0)
        _lib.check(
            _lib.load().artab_decode_step_boundary(
                parts, a_ptr, lda, _ptr(y2), y2.stride(0), _ptr(p_o), _ptr(last.norm2.weight), _ptr(last.norm2.bias),
                float(last.norm2.eps), _ptr(p_1), _ptr(last.ff[0].bias), _ptr(p_2), _ptr(last.ff[2].bias),
                _ptr(last.norm3.weight), _ptr(last.norm3.bias), float(last.norm3.eps), ctypes.byref(self.tail.args),
                _ptr(n_fo), _ptr(first.norm1.weight), _ptr(first.norm1.bias), float(first.norm1.eps), _ptr(n_qkv),
                _ptr(self.y_next), _ptr(self.qkv_next), last.ff[0].out_features, self.tail.dtype_code,
                _lib.current_stream(self.tail.device),
            )
        )
