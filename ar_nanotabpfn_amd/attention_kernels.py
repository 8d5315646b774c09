"""Attention entry points of the AR-TabPFN inference path, served by HIP kernels.

Host-side mirror of the reference's ``ar_tabpfn/model/triton_kernels.py``: the
same callables with the same argument meaning and error behaviour, each a thin
wrapper that describes its tensors to the C ABI (``include/artab_attention.h``)
and launches on the current stream.  All arithmetic happens on the device;
tensors that are not on a HIP device raise ``RuntimeError``.

The ``use_triton`` flag of the reference selects between its Triton kernel and
its eager PyTorch path.  Here it selects between the MFMA kernels (True, the
default; used whenever dtype/head_dim allow) and the portable float32-arithmetic
kernel (False).
"""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib

__all__ = [
    "AttentionPartials",
    "QueueOrder",
    "concurrent_stream",
    "hip_available",
    "triton_available",
    "context_attention",
    "triton_context_attention",
    "pytorch_context_attention",
    "buffer_attention",
    "pytorch_buffer_attention",
    "teacher_forcing_buffer_attention",
    "pytorch_teacher_forcing_buffer_attention",
    "merge_attention_outputs",
    "hybrid_attention",
    "hybrid_teacher_forcing_attention",
    "cross_attention",
    "decode_attention",
    "teacher_forcing_attention",
    "prefill_attention",
    "row_mask_attention",
    "row_mask_attention_backward",
]


def hip_available() -> bool:
    """True when the HIP extension is built and a HIP device is visible."""
    return _lib.library_built() and torch.cuda.is_available()


def triton_available() -> bool:
    """Availability probe under the reference's name (triton_kernels.py:527-529)."""
    return hip_available()


def _impl(use_triton: bool) -> int:
    return _lib.IMPL_AUTO if use_triton else _lib.IMPL_PORTABLE


def _alloc_out(q: Tensor) -> Tensor:
    """Output ``[B,H,Lq,Dh]`` backed by ``[B,Lq,H,Dh]`` storage, so the caller's
    ``out.transpose(1, 2).reshape(B, Lq, H*Dh)`` (inference.py:825) is a free view."""
    B, H, Lq, Dh = q.shape
    return torch.empty((B, Lq, H, Dh), device=q.device, dtype=q.dtype).transpose(1, 2)


def _ctx_views(k_ctx: Tensor, v_ctx: Tensor):
    if k_ctx.dim() == 3:
        return _lib.view4(k_ctx, shared_batch=True), _lib.view4(v_ctx, shared_batch=True), k_ctx.shape[0], k_ctx.shape[1]
    return _lib.view4(k_ctx), _lib.view4(v_ctx), k_ctx.shape[1], k_ctx.shape[2]


def _workspace_for(q: Tensor, Nc: int):
    B, H, Lq, Dh = q.shape
    lib = _lib.load()
    nbytes = lib.artab_workspace_bytes(B, H, Lq, Nc, Dh, _lib.dtype_code(q.dtype))
    ws = _lib.workspace(q.device, nbytes)
    if ws is None:
        return None, 0
    return ctypes.c_void_p(ws.data_ptr()), ws.numel() * 4


def context_attention(
    q: Tensor, k_ctx: Tensor, v_ctx: Tensor, scale: Optional[float] = None, use_triton: bool = True
) -> Tuple[Tensor, Tensor]:
    """Attention of ``q [B,H,Lq,D]`` over the context with log-sum-exp.

    ``k_ctx``/``v_ctx``: ``[H,Nc,D]`` shared by the batch (triton_kernels.py:347-475,
    :532-567) or ``[B,H,Nc,D]`` per dataset.  Returns ``out [B,H,Lq,D]`` (q's dtype)
    and ``lse [B,H,Lq]`` float32.
    """
    dev = _lib.require_device(q, k_ctx, v_ctx)
    lib = _lib.load()
    B, H, Lq, Dh = q.shape
    kv, vv, Hk, Nc = _ctx_views(k_ctx, v_ctx)
    if Hk != H or k_ctx.shape[-1] != Dh or v_ctx.shape != k_ctx.shape:
        raise ValueError(f"context K/V {tuple(k_ctx.shape)} do not match q {tuple(q.shape)}")
    if k_ctx.dtype != q.dtype or v_ctx.dtype != q.dtype:
        raise ValueError("q, k_ctx and v_ctx must share one dtype")
    out = _alloc_out(q)
    lse = torch.empty((B, H, Lq), device=dev, dtype=torch.float32)
    ws_ptr, ws_bytes = _workspace_for(q, Nc)
    qv, ov = _lib.view4(q), _lib.view4(out)
    _lib.check(
        lib.artab_context_attention(
            _lib.ref(qv), _lib.ref(kv), _lib.ref(vv), _lib.ref(ov), ctypes.c_void_p(lse.data_ptr()),
            B, H, Lq, Nc, Dh, float(scale) if scale is not None else 0.0, _lib.dtype_code(q.dtype),
            ws_ptr, ws_bytes, _impl(use_triton), _lib.current_stream(dev),
        )
    )
    return out, lse


def triton_context_attention(q: Tensor, k_ctx: Tensor, v_ctx: Tensor, scale: Optional[float] = None):
    """Name kept from triton_kernels.py:347-411; runs the MFMA kernel."""
    return context_attention(q, k_ctx, v_ctx, scale=scale, use_triton=True)


def pytorch_context_attention(q: Tensor, k_ctx: Tensor, v_ctx: Tensor, scale: Optional[float] = None):
    """Name kept from triton_kernels.py:532-567; runs the portable float32 kernel."""
    return context_attention(q, k_ctx, v_ctx, scale=scale, use_triton=False)


def buffer_attention(
    q: Tensor, k_buf: Tensor, v_buf: Tensor, mask: Optional[Tensor] = None, scale: Optional[float] = None
) -> Tuple[Tensor, Tensor]:
    """Per-trajectory attention over buffer K/V with an optional boolean mask
    (True = attend, broadcastable to ``[B,H,Lq,Nb]``) and log-sum-exp
    (triton_kernels.py:570-614).  Rows with no visible key: out 0, lse -inf."""
    dev = _lib.require_device(q, k_buf, v_buf, mask)
    lib = _lib.load()
    B, H, Lq, Dh = q.shape
    Nb = k_buf.shape[2]
    if k_buf.shape != v_buf.shape or k_buf.shape[0] != B or k_buf.shape[1] != H or k_buf.shape[3] != Dh:
        raise ValueError(f"buffer K/V {tuple(k_buf.shape)} do not match q {tuple(q.shape)}")
    out = _alloc_out(q)
    lse = torch.empty((B, H, Lq), device=dev, dtype=torch.float32)
    mask_ptr, msb, msh, msq, keep = None, 0, 0, 0, None
    if mask is not None and Nb > 0:
        m = mask
        if m.dtype != torch.uint8:
            m = m.to(torch.uint8)  # before expanding: broadcast axes stay stride-0 views
        while m.dim() < 4:
            m = m.unsqueeze(0)
        m = m.expand(B, H, Lq, Nb)
        if m.stride(3) != 1:
            m = m.contiguous()
        keep = m
        mask_ptr, msb, msh, msq = ctypes.c_void_p(m.data_ptr()), m.stride(0), m.stride(1), m.stride(2)
    qv, ov = _lib.view4(q), _lib.view4(out)
    kv = _lib.view4(k_buf) if Nb > 0 else None
    vv = _lib.view4(v_buf) if Nb > 0 else None
    _lib.check(
        lib.artab_buffer_attention(
            _lib.ref(qv), _lib.ref(kv), _lib.ref(vv), mask_ptr, msb, msh, msq, _lib.ref(ov),
            ctypes.c_void_p(lse.data_ptr()), B, H, Lq, Nb, Dh,
            float(scale) if scale is not None else 0.0, _lib.dtype_code(q.dtype), _lib.current_stream(dev),
        )
    )
    del keep
    return out, lse


pytorch_buffer_attention = buffer_attention


def _tf_mask(num_targets: int, device) -> Tensor:
    """``[1,1,2Nt,Nt]`` teacher-forcing buffer mask (triton_kernels.py:620-637)."""
    q_idx = torch.arange(2 * num_targets, device=device)
    kv_idx = torch.arange(num_targets, device=device)
    buffer_mask = kv_idx[None, :] <= q_idx[:, None]
    target_mask = kv_idx[None, :] < (q_idx - num_targets)[:, None]
    return torch.where((q_idx < num_targets)[:, None], buffer_mask, target_mask)[None, None]


def teacher_forcing_buffer_attention(
    q: Tensor, k_buf: Tensor, v_buf: Tensor, num_targets: int, scale: Optional[float] = None
) -> Tuple[Tensor, Tensor]:
    """Buffer part of teacher forcing with its LSE (triton_kernels.py:640-659)."""
    if q.shape[2] != 2 * num_targets:
        raise ValueError("Expected 2*num_targets queries for teacher forcing.")
    if k_buf.shape[2] != num_targets:
        raise ValueError("Expected buffer length to match num_targets.")
    return buffer_attention(q, k_buf, v_buf, mask=_tf_mask(num_targets, q.device), scale=scale)


pytorch_teacher_forcing_buffer_attention = teacher_forcing_buffer_attention


def merge_attention_outputs(out_ctx: Tensor, lse_ctx: Tensor, out_buf: Tensor, lse_buf: Tensor) -> Tensor:
    """Merge two partial attention outputs by their log-sum-exps (triton_kernels.py:478-524)."""
    dev = _lib.require_device(out_ctx, lse_ctx, out_buf, lse_buf)
    lib = _lib.load()
    B, H, Lq, Dh = out_ctx.shape
    if out_buf.shape != out_ctx.shape or lse_ctx.shape != (B, H, Lq) or lse_buf.shape != (B, H, Lq):
        raise ValueError("merge_attention_outputs: shape mismatch")
    if out_buf.dtype != out_ctx.dtype:
        out_buf = out_buf.to(out_ctx.dtype)
    la = lse_ctx.to(torch.float32).contiguous()
    lb = lse_buf.to(torch.float32).contiguous()
    out = _alloc_out(out_ctx)
    av, bv, ov = _lib.view4(out_ctx), _lib.view4(out_buf), _lib.view4(out)
    _lib.check(
        lib.artab_merge_attention_outputs(
            _lib.ref(av), ctypes.c_void_p(la.data_ptr()), _lib.ref(bv), ctypes.c_void_p(lb.data_ptr()),
            _lib.ref(ov), B, H, Lq, Dh, _lib.dtype_code(out_ctx.dtype), _lib.current_stream(dev),
        )
    )
    return out


def decode_attention(
    q: Tensor,
    k_ctx: Tensor,
    v_ctx: Tensor,
    k_buf_cache: Optional[Tensor],
    v_buf_cache: Optional[Tensor],
    n_buf: int,
    k_new: Optional[Tensor] = None,
    v_new: Optional[Tensor] = None,
    use_triton: bool = True,
    n_buf_device: Optional[Tensor] = None,
    side_stream: Optional["torch.cuda.Stream"] = None,
    leave_partials: bool = False,
    order: Optional["QueueOrder"] = None,
):
    """One decode step of row attention (inference.py:785-823) in one call.

    ``q [B,H,Lq,D]`` with Lq in {1,2}; ``k_buf_cache``/``v_buf_cache`` are the
    preallocated ``[B,H,cap,D]`` caches whose rows ``[0,n_buf)`` are valid.  With
    ``k_new``/``v_new [B,H,1,D]`` the row is appended in place at slot ``n_buf`` and
    all queries see it; the caller advances its cursor.  Raises ``ValueError`` for
    Lq outside {1,2} (:765-768) and for a full cache (:247-250).

    ``n_buf_device`` (one int32 on the device) makes the kernels read the committed
    length at run time, for launches recorded in a HIP graph; ``n_buf`` is then the
    upper bound that is validated against the cache capacity.

    ``side_stream`` (a default-priority stream of the same device) lets the buffer pass
    run next to the context pass (``artab_decode_attention_overlapped``); the call is
    still ordered on the current stream.

    ``order`` (with ``side_stream`` and ``leave_partials``) orders the two streams through the
    counters of a ``QueueOrder`` instead of two events per call
    (``artab_decode_attention_partials_ordered``): the caller makes ``side_stream`` wait for the
    current stream before the first such call and the current stream for ``side_stream`` after
    the last, and checks ``order.failed()`` before using the results.

    ``leave_partials=True`` skips the final merge where the schedule produces partial results
    and returns an ``AttentionPartials`` for ``glue.layer_post`` / ``layer_post_pre`` to merge
    while they load their input; where it does not, the merged tensor is returned as usual.
    """
    dev = _lib.require_device(q, k_ctx, v_ctx, k_buf_cache, v_buf_cache, k_new, v_new)
    lib = _lib.load()
    B, H, Lq, Dh = q.shape
    if Lq not in (1, 2):
        raise ValueError("Shared-context decode only supports N=1 (target) or N=2 (buffer, target).")
    kv, vv, Hk, Nc = _ctx_views(k_ctx, v_ctx)
    if Hk != H or k_ctx.shape[-1] != Dh:
        raise ValueError(f"context K/V {tuple(k_ctx.shape)} do not match q {tuple(q.shape)}")
    cap = k_buf_cache.shape[2] if k_buf_cache is not None else 0
    if n_buf_device is not None and (n_buf_device.dtype != torch.int32 or not n_buf_device.is_cuda):
        raise ValueError("n_buf_device must be an int32 tensor on the device")
    out = _alloc_out(q)
    ws_ptr, ws_bytes = _workspace_for(q, Nc)
    qv, ov = _lib.view4(q), _lib.view4(out)
    kbv, vbv = _lib.view4(k_buf_cache), _lib.view4(v_buf_cache)
    knv, vnv = _lib.view4(k_new), _lib.view4(v_new)
    args = (
        _lib.ref(qv), _lib.ref(kv), _lib.ref(vv), _lib.ref(kbv), _lib.ref(vbv), _lib.ref(knv), _lib.ref(vnv),
        _lib.ref(ov), B, H, Lq, Nc, int(n_buf),
        ctypes.c_void_p(n_buf_device.data_ptr()) if n_buf_device is not None else None,
        cap, Dh, 0.0, _lib.dtype_code(q.dtype),
        ws_ptr, ws_bytes, _impl(use_triton), _lib.current_stream(dev),
    )
    side = ctypes.c_void_p(side_stream.cuda_stream) if side_stream is not None else None
    if order is not None:
        if not leave_partials or side_stream is None:
            raise ValueError("counter-ordered decode needs side_stream and leave_partials=True")
        desc = _lib.ArtabAttentionPartials()
        flags = _lib.ORDER_CONSUMER_WAITS if order.consumer_waits else 0
        _lib.check(lib.artab_decode_attention_partials_ordered(
            *args, side, ctypes.byref(desc), ctypes.c_void_p(order.state.data_ptr()), int(order.timeout_us), flags))
        parts = AttentionPartials(desc, q.dtype, q.device)
        parts.order = order
        return parts
    if leave_partials:
        desc = _lib.ArtabAttentionPartials()
        _lib.check(lib.artab_decode_attention_partials(*args, side, ctypes.byref(desc)))
        if desc.n_slots > 0:
            return AttentionPartials(desc, q.dtype, q.device)
    elif side_stream is not None:
        _lib.check(lib.artab_decode_attention_overlapped(*args, side))
    else:
        _lib.check(lib.artab_decode_attention(*args))
    return out


class QueueOrder:
    """Counters in device memory that order two streams without events (``artab_order_*``):
    ``state`` holds counter "main" at int32 index 0, counter "side" at 32 and ``failed`` at 64."""

    MAIN, SIDE = 0, 1

    def __init__(self, device, timeout_us: int = 2_000_000):
        self.state = torch.zeros(128, device=device, dtype=torch.int32)
        if self.state.data_ptr() % 128:
            raise RuntimeError("queue-order state is not 128-byte aligned")
        self.timeout_us = int(timeout_us)
        # Let the consumer of an ordered attention call's partials (``glue.layer_post_pre`` /
        # ``layer_post``, ``AttentionPartials.merged``) wait for the side stream itself instead of
        # a wait launch inside the call.
        self.consumer_waits = True

    def signal(self, queue: int, stream: "torch.cuda.Stream") -> None:
        _lib.check(_lib.load().artab_order_signal(
            ctypes.c_void_p(self.state.data_ptr()), int(queue), ctypes.c_void_p(stream.cuda_stream)))

    def wait(self, queue: int, stream: "torch.cuda.Stream", timeout_us: Optional[int] = None) -> None:
        _lib.check(_lib.load().artab_order_wait(
            ctypes.c_void_p(self.state.data_ptr()), int(queue),
            int(self.timeout_us if timeout_us is None else timeout_us), ctypes.c_void_p(stream.cuda_stream)))

    def failed(self) -> int:
        """Number of waits that gave up (synchronises with the device)."""
        return int(self.state[64].item())

    def reset(self) -> None:
        self.state.zero_()

    def streams_run_concurrently(self, main: "torch.cuda.Stream", side: "torch.cuda.Stream",
                                 timeout_us: int = 50_000) -> bool:
        """One round of the protocol on the two streams: ``side`` waits for a signal that is launched
        on ``main`` after it.  False when the wait timed out, i.e. the two streams are served by one
        hardware queue (or a tool serialises launches) and counters cannot order them."""
        side.wait_stream(main)
        self.wait(self.SIDE, side, timeout_us)
        self.signal(self.MAIN, main)
        self.signal(self.SIDE, side)
        self.wait(self.MAIN, main, timeout_us)
        main.wait_stream(side)
        main.synchronize()
        ok = self.failed() == 0
        self.reset()
        main.synchronize()
        return ok


def concurrent_stream(device, main: Optional["torch.cuda.Stream"] = None, tries: int = 8):
    """A default-priority stream that runs side by side with ``main`` (default: the current
    stream), and whether that was confirmed.  The runtime serves its streams from a few hardware
    queues; two streams that land on the same one execute one after the other, which silently
    serialises the two passes of a decode step (and makes counter ordering impossible).  Candidates
    are probed with one round of the ``QueueOrder`` protocol (50 ms when it fails); call this
    outside graph capture."""
    main = torch.cuda.current_stream(device) if main is None else main
    probe = QueueOrder(device)
    side = None
    for _ in range(max(1, tries)):
        side = torch.cuda.Stream(device=device)
        if side.cuda_stream != main.cuda_stream and probe.streams_run_concurrently(main, side):
            return side, True
    return side, False


class AttentionPartials:
    """Unmerged attention result of a decode step (``artab_attention_partials``): it points into
    the device's split workspace and is valid until the next attention call on that device."""

    def __init__(self, desc, dtype, device):
        self.desc, self.dtype, self.device = desc, dtype, device
        self.order = None  # the QueueOrder of an ordered call

    @property
    def shape(self):  # of the merged [B,H,Lq,Dh] result
        return (self.desc.B, self.desc.H, self.desc.Lq, self.desc.Dh)

    def merged(self) -> Tensor:
        """The merged ``[B,H,Lq,Dh]`` tensor (``artab_merge_attention_partials``), for callers whose
        next step is not one of the layer kernels that merge on load."""
        B, H, Lq, Dh = self.shape
        out = torch.empty((B, Lq, H, Dh), device=self.device, dtype=self.dtype).transpose(1, 2)
        ov = _lib.view4(out)
        _lib.check(_lib.load().artab_merge_attention_partials(
            ctypes.byref(self.desc), _lib.ref(ov), _lib.dtype_code(self.dtype), _lib.current_stream(self.device)))
        return out


def teacher_forcing_attention(
    q: Tensor, k_ctx: Tensor, v_ctx: Tensor, k_buf: Tensor, v_buf: Tensor, num_targets: int,
    use_triton: bool = True, return_lse: bool = False,
):
    """Teacher-forced attention with the mask as a tile schedule; context shared
    ``[H,Nc,D]`` or per dataset ``[B,H,Nc,D]``."""
    dev = _lib.require_device(q, k_ctx, v_ctx, k_buf, v_buf)
    lib = _lib.load()
    B, H, Lq, Dh = q.shape
    if Lq != 2 * num_targets:
        raise ValueError("Expected 2*num_targets queries for teacher forcing.")
    if k_buf.shape[2] != num_targets:
        raise ValueError("Expected buffer length to match num_targets.")
    kv, vv, Hk, Nc = _ctx_views(k_ctx, v_ctx)
    if Hk != H or k_ctx.shape[-1] != Dh:
        raise ValueError(f"context K/V {tuple(k_ctx.shape)} do not match q {tuple(q.shape)}")
    out = _alloc_out(q)
    lse = torch.empty((B, H, Lq), device=dev, dtype=torch.float32) if return_lse else None
    qv, ov, kbv, vbv = _lib.view4(q), _lib.view4(out), _lib.view4(k_buf), _lib.view4(v_buf)
    _lib.check(
        lib.artab_teacher_forcing_attention(
            _lib.ref(qv), _lib.ref(kv), _lib.ref(vv), _lib.ref(kbv), _lib.ref(vbv), _lib.ref(ov),
            ctypes.c_void_p(lse.data_ptr()) if lse is not None else None,
            B, H, num_targets, Nc, Dh, 0.0, _lib.dtype_code(q.dtype), _impl(use_triton), _lib.current_stream(dev),
        )
    )
    return (out, lse) if return_lse else out


def prefill_attention(
    q: Tensor, k: Tensor, v: Tensor, k_cache: Optional[Tensor] = None, v_cache: Optional[Tensor] = None,
    use_triton: bool = True,
) -> Tensor:
    """Dense self-attention over the context rows plus the cache write
    (inference.py:618-622, :672-676).  ``k_cache``/``v_cache``: ``[H,Nc',D]`` (shared:
    batch entry 0 is stored) or ``[B,H,Nc',D]`` with Nc' >= Nc."""
    dev = _lib.require_device(q, k, v, k_cache, v_cache)
    lib = _lib.load()
    B, H, Nc, Dh = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("prefill expects q, k, v of one shape [B,H,Nc,D]")
    out = _alloc_out(q)
    kcv = vcv = None
    cache_batches = 0
    if k_cache is not None:
        shared = k_cache.dim() == 3
        rows = k_cache.shape[1] if shared else k_cache.shape[2]
        if rows < Nc:
            raise ValueError(f"cache holds {rows} rows, context has {Nc}")
        kcv, vcv = _lib.view4(k_cache, shared_batch=shared), _lib.view4(v_cache, shared_batch=shared)
        cache_batches = 1 if shared else k_cache.shape[0]
    qv, kv, vv, ov = _lib.view4(q), _lib.view4(k), _lib.view4(v), _lib.view4(out)
    _lib.check(
        lib.artab_prefill_attention(
            _lib.ref(qv), _lib.ref(kv), _lib.ref(vv), _lib.ref(ov), _lib.ref(kcv), _lib.ref(vcv), cache_batches,
            B, H, Nc, Dh, 0.0, _lib.dtype_code(q.dtype), _impl(use_triton), _lib.current_stream(dev),
        )
    )
    return out


def _row_mask_forward(q: Tensor, k: Tensor, v: Tensor, context_len: int, buffer_len: int, attending_chunks: int,
                      use_triton: bool, want_lse: bool):
    dev = _lib.require_device(q, k, v)
    lib = _lib.load()
    B, H, R, Dh = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("row-mask attention expects q, k, v of one shape [B,H,R,D]")
    out = _alloc_out(q)
    lse = torch.empty((B, H, R), device=q.device, dtype=torch.float32) if want_lse else None
    qv, kv, vv, ov = _lib.view4(q), _lib.view4(k), _lib.view4(v), _lib.view4(out)
    _lib.check(
        lib.artab_row_mask_attention(
            _lib.ref(qv), _lib.ref(kv), _lib.ref(vv), _lib.ref(ov), lse.data_ptr() if want_lse else None,
            B, H, R, int(context_len), int(buffer_len), int(attending_chunks), Dh, 0.0, _lib.dtype_code(q.dtype),
            _impl(use_triton), _lib.current_stream(dev),
        )
    )
    return out, lse


def row_mask_attention_backward(q: Tensor, k: Tensor, v: Tensor, out: Tensor, dout: Tensor, lse: Tensor,
                                context_len: int, buffer_len: int, attending_chunks: int,
                                use_triton: bool = True) -> Tuple[Tensor, Tensor, Tensor]:
    """Gradients of ``row_mask_attention`` for the output gradient ``dout``: ``(dq, dk, dv)``, each
    ``[B,H,R,D]`` (views of one ``[B,R,3,H,D]`` tensor, the layout of a fused q/k/v projection).
    ``out`` and ``lse`` are what the forward returned.  The gradients autograd derives for the
    reference's flex_attention call under ``create_row_mask`` (attention.py:57-59, :86-175)."""
    dev = _lib.require_device(q, k, v, out, dout)
    lib = _lib.load()
    B, H, R, Dh = q.shape
    for name, t in (("k", k), ("v", v), ("out", out), ("dout", dout)):
        if t.shape != q.shape or t.dtype != q.dtype:
            raise ValueError(f"{name} must have q's shape {tuple(q.shape)} and dtype")
    if lse.shape != (B, H, R) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("lse must be a contiguous float32 [B,H,R] tensor")
    if dout.stride(-1) != 1 or any(st % (16 // dout.element_size()) for st in dout.stride()[:-1]):
        dout = dout.contiguous()
    grads = torch.empty((B, R, 3, H, Dh), device=q.device, dtype=q.dtype)
    dq, dk, dv = (grads[:, :, i].transpose(1, 2) for i in range(3))
    delta = torch.empty((B, H, R), device=q.device, dtype=torch.float32)
    views = [_lib.view4(t) for t in (q, k, v, out, dout)]
    gviews = [_lib.view4(t) for t in (dq, dk, dv)]
    _lib.check(
        lib.artab_row_mask_attention_backward(
            *[_lib.ref(x) for x in views], lse.data_ptr(), delta.data_ptr(), *[_lib.ref(x) for x in gviews],
            B, H, R, int(context_len), int(buffer_len), int(attending_chunks), Dh, 0.0, _lib.dtype_code(q.dtype),
            _impl(use_triton), _lib.current_stream(dev),
        )
    )
    return dq, dk, dv


class _RowMaskAttention(torch.autograd.Function):
    """``row_mask_attention`` with its device backward pass (two launches: dQ, then dK and dV)."""

    @staticmethod
    def forward(ctx, q, k, v, context_len, buffer_len, attending_chunks, use_triton):
        out, lse = _row_mask_forward(q, k, v, context_len, buffer_len, attending_chunks, use_triton, want_lse=True)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.mask = (context_len, buffer_len, attending_chunks, use_triton)
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dout):
        # The device backward pass is not itself differentiable: asking for a second derivative
        # raises instead of treating dq, dk, dv as constants.
        q, k, v, out, lse = ctx.saved_tensors
        context_len, buffer_len, attending_chunks, use_triton = ctx.mask
        dq, dk, dv = row_mask_attention_backward(q, k, v, out, dout, lse, context_len, buffer_len, attending_chunks,
                                                 use_triton)
        return dq, dk, dv, None, None, None, None


def row_mask_attention(q: Tensor, k: Tensor, v: Tensor, context_len: int, buffer_len: int, attending_chunks: int,
                       use_triton: bool = True) -> Tensor:
    """Row attention of the training forward: ``q, k, v [B,H,R,D]`` with rows
    ``[context | buffer | target]`` under the mask of ``create_row_mask``
    (attention.py:86-175), carried as a tile schedule.  Differentiable: when gradients are
    being recorded for q, k or v the call goes through ``_RowMaskAttention``."""
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return _RowMaskAttention.apply(q, k, v, int(context_len), int(buffer_len), int(attending_chunks), use_triton)
    return _row_mask_forward(q, k, v, context_len, buffer_len, attending_chunks, use_triton, want_lse=False)[0]


def hybrid_attention(
    q: Tensor, k_ctx: Tensor, v_ctx: Tensor, k_buf: Tensor, v_buf: Tensor,
    buf_mask: Optional[Tensor] = None, use_triton: bool = True,
) -> Tensor:
    """Context attention + buffer attention + LSE merge (triton_kernels.py:705-755).

    An empty buffer returns the context part alone (:735-741).  Without a mask and
    with at most two queries this is one fused decode call; otherwise the three
    device steps run one after another exactly as the reference composes them.
    """
    Lq = q.shape[2]
    if k_buf.shape[2] == 0:
        out, _ = context_attention(q, k_ctx, v_ctx, use_triton=use_triton)
        return out
    if buf_mask is None and Lq in (1, 2):
        return decode_attention(q, k_ctx, v_ctx, k_buf, v_buf, k_buf.shape[2], use_triton=use_triton)
    out_ctx, lse_ctx = context_attention(q, k_ctx, v_ctx, use_triton=use_triton)
    out_buf, lse_buf = buffer_attention(q, k_buf, v_buf, mask=buf_mask)
    return merge_attention_outputs(out_ctx, lse_ctx, out_buf, lse_buf)


def hybrid_teacher_forcing_attention(
    q: Tensor, k_ctx: Tensor, v_ctx: Tensor, k_buf: Tensor, v_buf: Tensor, num_targets: int,
    use_triton: bool = True,
) -> Tensor:
    """Teacher-forcing attention (triton_kernels.py:662-702) as one kernel."""
    if k_buf.shape[2] == 0:
        out, _ = context_attention(q, k_ctx, v_ctx, use_triton=use_triton)
        return out
    return teacher_forcing_attention(q, k_ctx, v_ctx, k_buf, v_buf, num_targets, use_triton=use_triton)


def cross_attention(q: Tensor, k_ctx: Tensor, v_ctx: Tensor, use_triton: bool = True) -> Tensor:
    """Context attention without the LSE (triton_kernels.py:758-767)."""
    out, _ = context_attention(q, k_ctx, v_ctx, use_triton=use_triton)
    return out
