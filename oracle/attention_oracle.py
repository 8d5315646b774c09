"""CPU oracle for the AR-TabPFN attention hot path (TEST INFRASTRUCTURE ONLY).

This file is a numpy restatement of the reference's attention arithmetic.  It is
the checker the HIP kernels are compared against; nothing in the shipped package
imports it.  Only tests, the smoke entry and the CPU-baseline leg of the benchmark
may call it.

Every function cites the reference lines it follows (paths relative to the
reference checkout, ``ar_tabpfn/model/...``).  All arithmetic runs in the dtype
given by ``compute`` (float64 by default) on inputs that are up-cast first, so
the oracle is the exact-arithmetic answer for the given input bits; the
reference's own-dtype evaluation (bf16 scores/probabilities) is a noisier
evaluation of the same formulas.

Pinning status (what independently fixes each function; the tests that do it
live in ``tests/test_oracle.py``):

* ``context_attention``, ``buffer_attention``, ``dense_self_attention``: pinned
  by a pure-Python triple loop in ``loops_attention`` on tiny shapes, by
  ``scipy.special.logsumexp``/``softmax`` and by the ragged shapes the reference
  tests use (B=37, N_CTX=100; tests/test_triton_kernel.py:68-102).
* ``merge_attention_outputs``: pinned by the two closed forms the reference
  tests hold (lse 10 vs -10 -> out_ctx, equal lse -> arithmetic mean;
  tests/test_triton_kernel.py:345-382) and by merge == one softmax over the
  concatenated keys (:204-282), plus split invariance and commutativity.
* ``teacher_forcing_buffer_mask`` / ``teacher_forcing_mask`` / ``decode_mask``:
  pinned against each other (two independent statements in the reference) and
  by the closed-form pair count Nt**2; target 0 sees no buffer
  (tests/test_triton_kernel.py:135-151).
* ``hybrid_attention`` / ``hybrid_teacher_forcing_attention``: pinned by
  equality with masked full attention (tests/test_triton_kernel.py:157-198,
  :288-339).
* ``row_mask`` (training forward): pinned against the second, region-wise statement of
  the same mask that the reference holds (tests/visualize_masks.py:57-85), by the
  closed-form pair count, by a hand-written tiny case, and through the training loss
  the reference itself computed for the fixture (tests/golden/tiny_model.npz).
* ``row_mask_attention_backward``: pinned by central finite differences of
  ``row_mask_attention`` (an independent function: the directional derivative of
  sum(out * dout) along random directions in q, k and v), and by what the softmax fixes:
  the key gradients sum to the zero vector (one vector added to every key shifts every
  score of a row alike and leaves the output unchanged), the value gradients sum to the
  sum of the output gradients (every row of P sums to one), and target keys, which no row
  sees, get exact zeros.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np

__all__ = [
    "context_attention",
    "round_bf16",
    "context_attention_same_dtype",
    "buffer_attention",
    "merge_attention_outputs",
    "teacher_forcing_buffer_mask",
    "teacher_forcing_buffer_attention",
    "hybrid_attention",
    "hybrid_teacher_forcing_attention",
    "decode_mask",
    "teacher_forcing_mask",
    "row_mask",
    "row_mask_attention",
    "row_mask_attention_backward",
    "masked_full_attention",
    "dense_self_attention",
    "decode_step_attention",
    "loops_attention",
]


def _up(x, compute):
    return np.asarray(x, dtype=compute)


def _logsumexp(scores: np.ndarray) -> np.ndarray:
    """logsumexp over the last axis; rows that are all -inf give -inf (as torch)."""
    m = np.max(scores, axis=-1, keepdims=True) if scores.shape[-1] else np.full(
        scores.shape[:-1] + (1,), -np.inf, dtype=scores.dtype
    )
    m_safe = np.where(np.isfinite(m), m, 0.0)
    with np.errstate(divide="ignore"):
        out = np.log(np.sum(np.exp(scores - m_safe), axis=-1)) + m_safe[..., 0]
    return out


def _softmax(scores: np.ndarray) -> np.ndarray:
    """softmax over the last axis; all -inf rows give NaN exactly like torch.softmax."""
    if scores.shape[-1] == 0:
        return scores.copy()
    m = np.max(scores, axis=-1, keepdims=True)
    with np.errstate(invalid="ignore"):
        e = np.exp(scores - m)
        return e / np.sum(e, axis=-1, keepdims=True)


def context_attention(
    q, k_ctx, v_ctx, scale: Optional[float] = None, compute=np.float64
) -> Tuple[np.ndarray, np.ndarray]:
    """Attention of ``q [B,H,Lq,D]`` over a context K/V plus its log-sum-exp.

    ``k_ctx``/``v_ctx`` are ``[H,Nc,D]`` (one context for every batch element,
    triton_kernels.py:532-567 expands it as a stride-0 view, :554-555) or
    ``[B,H,Nc,D]`` (one context per dataset: the layout of the per-dataset cache
    ``layer.k_cache[:, :, :Nc]``, inference.py:124-130,618-619).

    Returns ``out [B,H,Lq,D]`` and ``lse [B,H,Lq]`` = logsumexp(q k^T * scale)
    (triton_kernels.py:558-565).
    """
    q = _up(q, compute)
    k = _up(k_ctx, compute)
    v = _up(v_ctx, compute)
    if k.ndim == 3:
        k = k[None]
        v = v[None]
    D = q.shape[-1]
    if scale is None:
        scale = D ** -0.5
    B, H, Lq, _ = q.shape
    if k.shape[0] == 1 and B > 1:
        # one context for the whole batch: fold (b, lq) into the row axis so the products are
        # plain per-head matrix multiplications (same arithmetic, BLAS speed)
        q2 = q.transpose(1, 0, 2, 3).reshape(H, B * Lq, D)
        scores = np.matmul(q2, k[0].transpose(0, 2, 1)) * scale  # [H, B*Lq, Nc]
        lse = _logsumexp(scores)
        out = np.matmul(_softmax(scores), v[0])
        out = out.reshape(H, B, Lq, D).transpose(1, 0, 2, 3)
        return out, lse.reshape(H, B, Lq).transpose(1, 0, 2)
    scores = np.matmul(q, k.transpose(0, 1, 3, 2)) * scale
    lse = _logsumexp(scores)
    out = np.matmul(_softmax(scores), v)
    return out, lse


def round_bf16(x) -> np.ndarray:
    """Round float32 values to the nearest bfloat16 (ties to even), returned as float32: what
    ``tensor.to(torch.bfloat16)`` does to finite values."""
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    u = a.view(np.uint32)
    bias = np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    r = ((u + bias) & np.uint32(0xFFFF0000)).astype(np.uint32)
    return r.view(np.float32).reshape(a.shape)


def context_attention_same_dtype(q, k_ctx, v_ctx, scale: Optional[float] = None) -> Tuple[np.ndarray, np.ndarray]:
    """``pytorch_context_attention`` (triton_kernels.py:532-567) as it evaluates on bfloat16
    tensors: every tensor-valued intermediate is rounded to bfloat16 where torch materialises one —
    the score matrix (:558, product accumulated in float32, rounded, scaled, rounded), the softmax
    (:564, computed in float32 from the rounded scores, rounded) and the output (:565) — while the
    LSE is the float32 logsumexp of the rounded scores (:561).  Secondary reference: looser than
    the float64 one by construction.  Shared ``[H,Nc,D]`` context only."""
    q32, k32, v32 = (round_bf16(a) for a in (q, k_ctx, v_ctx))
    D = q32.shape[-1]
    if scale is None:
        scale = D ** -0.5
    scores = round_bf16(np.einsum("bhqd,hnd->bhqn", q32, k32, dtype=np.float32))
    scores = round_bf16(scores * np.float32(scale))
    lse = _logsumexp(scores.astype(np.float32))
    attn = round_bf16(_softmax(scores.astype(np.float32)))
    out = round_bf16(np.einsum("bhqn,hnd->bhqd", attn, v32, dtype=np.float32))
    return out, lse


def buffer_attention(
    q, k_buf, v_buf, mask=None, scale: Optional[float] = None, compute=np.float64
) -> Tuple[np.ndarray, np.ndarray]:
    """Per-trajectory attention over buffer K/V ``[B,H,Nb,D]`` with optional mask.

    Follows triton_kernels.py:570-614: masked scores are -inf (:602), rows with
    no visible key give ``out = 0`` and ``lse = -inf`` (:603,:610-611).  ``mask``
    is boolean, True = attend, broadcastable to ``[B,H,Lq,Nb]``.
    """
    q = _up(q, compute)
    k = _up(k_buf, compute)
    v = _up(v_buf, compute)
    D = q.shape[-1]
    if scale is None:
        scale = D ** -0.5
    scores = np.matmul(q, k.transpose(0, 1, 3, 2)) * scale
    no_kv = None
    if mask is not None:
        mask = np.broadcast_to(np.asarray(mask, dtype=bool), scores.shape)
        scores = np.where(mask, scores, -np.inf)
        no_kv = ~mask.any(axis=-1)
    lse = _logsumexp(scores)
    attn = _softmax(scores)
    if no_kv is not None:
        attn = np.where(no_kv[..., None], 0.0, attn)
    out = np.matmul(attn, v)
    return out, lse


def merge_attention_outputs(out_ctx, lse_ctx, out_buf, lse_buf, compute=np.float64) -> np.ndarray:
    """Combine two partial softmax results through their log-sum-exps.

    triton_kernels.py:478-524:  m = max(lse_c, lse_b); w = exp(lse - m);
    out = (w_c out_c + w_b out_b) / (w_c + w_b).  Both lse = -inf gives NaN,
    exactly as the reference's formula does (:508-517).
    """
    out_ctx = _up(out_ctx, compute)
    out_buf = _up(out_buf, compute)
    lse_ctx = _up(lse_ctx, compute)
    lse_buf = _up(lse_buf, compute)
    with np.errstate(invalid="ignore"):
        lse_max = np.maximum(lse_ctx, lse_buf)
        w_ctx = np.exp(lse_ctx - lse_max)
        w_buf = np.exp(lse_buf - lse_max)
        w_total = w_ctx + w_buf
        w_ctx = w_ctx / w_total
        w_buf = w_buf / w_total
        return w_ctx[..., None] * out_ctx + w_buf[..., None] * out_buf


def teacher_forcing_buffer_mask(num_targets: int) -> np.ndarray:
    """Mask ``[1,1,2Nt,Nt]`` of the 2Nt teacher-forcing queries over Nt buffers.

    triton_kernels.py:620-637: query rows [0,Nt) are buffers and see ``kv <= q``;
    rows [Nt,2Nt) are targets and see ``kv < q - Nt``.
    """
    q_idx = np.arange(2 * num_targets)
    kv_idx = np.arange(num_targets)
    is_buffer = q_idx < num_targets
    buffer_mask = kv_idx[None, :] <= q_idx[:, None]
    target_mask = kv_idx[None, :] < (q_idx - num_targets)[:, None]
    mask = np.where(is_buffer[:, None], buffer_mask, target_mask)
    return mask[None, None]


def teacher_forcing_buffer_attention(q, k_buf, v_buf, num_targets: int, scale=None, compute=np.float64):
    """triton_kernels.py:640-659 (shape checks included)."""
    if q.shape[2] != 2 * num_targets:
        raise ValueError("Expected 2*num_targets queries for teacher forcing.")
    if k_buf.shape[2] != num_targets:
        raise ValueError("Expected buffer length to match num_targets.")
    mask = teacher_forcing_buffer_mask(num_targets)
    return buffer_attention(q, k_buf, v_buf, mask=mask, scale=scale, compute=compute)


def hybrid_attention(q, k_ctx, v_ctx, k_buf, v_buf, buf_mask=None, compute=np.float64) -> np.ndarray:
    """Decode attention: context part + buffer part + merge (triton_kernels.py:705-755).

    An empty buffer returns the context part alone (:735-741).
    """
    if k_buf.shape[2] == 0:
        out_ctx, _ = context_attention(q, k_ctx, v_ctx, compute=compute)
        return out_ctx
    out_ctx, lse_ctx = context_attention(q, k_ctx, v_ctx, compute=compute)
    out_buf, lse_buf = buffer_attention(q, k_buf, v_buf, mask=buf_mask, compute=compute)
    return merge_attention_outputs(out_ctx, lse_ctx, out_buf, lse_buf, compute=compute)


def hybrid_teacher_forcing_attention(q, k_ctx, v_ctx, k_buf, v_buf, num_targets: int, compute=np.float64):
    """Teacher-forcing attention: context + masked buffer + merge (triton_kernels.py:662-702)."""
    if k_buf.shape[2] == 0:
        out_ctx, _ = context_attention(q, k_ctx, v_ctx, compute=compute)
        return out_ctx
    out_ctx, lse_ctx = context_attention(q, k_ctx, v_ctx, compute=compute)
    out_buf, lse_buf = teacher_forcing_buffer_attention(q, k_buf, v_buf, num_targets, compute=compute)
    return merge_attention_outputs(out_ctx, lse_ctx, out_buf, lse_buf, compute=compute)


def decode_mask(num_cached: int, num_new: int) -> np.ndarray:
    """Dense ``[num_new, num_cached+num_new]`` form of the per-trajectory decode mask.

    inference.py:500-523: the last new row is the target and sees
    ``kv < num_cached + q``; earlier new rows are buffers and see
    ``kv < num_cached + q + 1``.
    """
    q_idx = np.arange(num_new)[:, None]
    kv_idx = np.arange(num_cached + num_new)[None, :]
    is_target = q_idx == num_new - 1
    is_buffer = q_idx < num_new - 1
    target_pattern = is_target & (kv_idx < num_cached + q_idx)
    buffer_pattern = is_buffer & (kv_idx < num_cached + q_idx + 1)
    return target_pattern | buffer_pattern


def teacher_forcing_mask(num_cached: int, num_targets: int) -> np.ndarray:
    """Dense ``[2Nt, num_cached+2Nt]`` form of the full-cache teacher-forcing mask.

    inference.py:525-577: everyone sees the cached context; buffer query i sees
    buffer keys j <= i; target query i sees buffer keys j < i; target keys
    (the last Nt columns) are never visible.
    """
    Nt = num_targets
    q_idx = np.arange(2 * Nt)[:, None]
    kv_idx = np.arange(num_cached + 2 * Nt)[None, :]
    attends_context = kv_idx < num_cached
    is_buffer_query = q_idx < Nt
    kv_is_buffer = (kv_idx >= num_cached) & (kv_idx < num_cached + Nt)
    buffer_kv_idx = kv_idx - num_cached
    buffer_causal = kv_is_buffer & (buffer_kv_idx <= q_idx)
    is_target_query = q_idx >= Nt
    target_idx = q_idx - Nt
    target_to_buffer = kv_is_buffer & (buffer_kv_idx < target_idx)
    return attends_context | (is_buffer_query & buffer_causal) | (is_target_query & target_to_buffer)


def row_mask(num_rows: int, context_len: int, buffer_len: int, attending_chunks: Optional[int] = None) -> np.ndarray:
    """Dense ``[R, R]`` form of the training row mask over ``[context | buffer | target]`` rows.

    attention.py:86-175, the three mask_mods that are or-ed (:165-169): ``prefix_mask``
    (kv < context_len, :127-129), ``localized_causal_ctx_buf`` (q and kv below
    context_len + buffer_len and q >= kv, :131-136) and ``chunked_target_buffer`` (q a target,
    kv a buffer, target offset below attending_chunks * buffer_len, buffer offset <=
    target offset mod buffer_len, :138-160).  attending_chunks defaults to
    target_len // (2 * buffer_len) (:111-112).
    """
    target_len = num_rows - context_len - buffer_len
    if attending_chunks is None:
        attending_chunks = target_len // (2 * buffer_len)
    target_start = context_len + buffer_len
    q_idx = np.arange(num_rows)[:, None]
    kv_idx = np.arange(num_rows)[None, :]
    prefix = kv_idx < context_len
    ctx_buf_end = context_len + buffer_len
    localized = (q_idx < ctx_buf_end) & (kv_idx < ctx_buf_end) & (q_idx >= kv_idx)
    q_in_target = q_idx >= target_start
    kv_in_buffer = (kv_idx >= context_len) & (kv_idx < target_start)
    target_offset = q_idx - target_start
    buffer_offset = kv_idx - context_len
    in_attending_region = target_offset < attending_chunks * buffer_len
    chunk_position = target_offset % max(buffer_len, 1)
    chunked = q_in_target & kv_in_buffer & in_attending_region & (buffer_offset <= chunk_position)
    return prefix | localized | chunked


def row_mask_attention(q, k, v, context_len: int, buffer_len: int, attending_chunks: Optional[int] = None,
                       compute=np.float64):
    """Row attention of the training forward: one masked softmax over all rows under
    ``row_mask`` (flex_attention with the BlockMask of attention.py:86-175, as called at
    attention.py:57-59).  ``q, k, v [B,H,R,D]``; returns ``out``."""
    R = q.shape[2]
    mask = row_mask(R, context_len, buffer_len, attending_chunks)[None, None]
    out, _ = buffer_attention(q, k, v, mask=mask, compute=compute)
    return out


def row_mask_attention_backward(q, k, v, dout, context_len: int, buffer_len: int,
                                attending_chunks: Optional[int] = None, scale: Optional[float] = None,
                                compute=np.float64):
    """Gradients of ``row_mask_attention`` with respect to q, k and v for an output gradient
    ``dout [B,H,R,D]``: what autograd derives for the reference's flex_attention call
    (attention.py:57-59) inside its training step (train.py:289-300).  Written out from the
    softmax Jacobian: with ``P`` the masked softmax of ``scale q k^T`` and ``O = P v``,

        dv = P^T dout,  dP = dout v^T,  dS = P * (dP - rowsum(dout * O)),
        dq = scale dS k,  dk = scale dS^T q.

    Returns ``(dq, dk, dv)``."""
    q, k, v, dout = _up(q, compute), _up(k, compute), _up(v, compute), _up(dout, compute)
    R, D = q.shape[2], q.shape[3]
    if scale is None:
        scale = D ** -0.5
    mask = row_mask(R, context_len, buffer_len, attending_chunks)[None, None]
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * compute(scale)
    s = np.where(mask, s, -np.inf)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    p = p / p.sum(axis=-1, keepdims=True)
    out = np.einsum("bhqk,bhkd->bhqd", p, v)
    dv = np.einsum("bhqk,bhqd->bhkd", p, dout)
    dp = np.einsum("bhqd,bhkd->bhqk", dout, v)
    ds = p * (dp - (dout * out).sum(axis=-1, keepdims=True))
    dq = np.einsum("bhqk,bhkd->bhqd", ds, k) * compute(scale)
    dk = np.einsum("bhqk,bhqd->bhkd", ds, q) * compute(scale)
    return dq, dk, dv


def masked_full_attention(q, k_full, v_full, mask=None, scale=None, compute=np.float64):
    """One masked softmax over an explicit key set: the ground truth every split
    scheme must equal (the construction of tests/test_triton_kernel.py:176-196).

    ``k_full``/``v_full`` ``[B,H,N,D]``; ``mask`` broadcastable to ``[B,H,Lq,N]``.
    Returns ``(out, lse)``.
    """
    return buffer_attention(q, k_full, v_full, mask=mask, scale=scale, compute=compute)


def dense_self_attention(q, k, v, scale=None, compute=np.float64):
    """Bidirectional self-attention of the context prefill (dense mask,
    attention.py:72-83 used at inference.py:168-169,622,676).  Returns (out, lse)."""
    return buffer_attention(q, k, v, mask=None, scale=scale, compute=compute)


def decode_step_attention(q, k_ctx, v_ctx, k_buf, v_buf, k_new=None, v_new=None, compute=np.float64):
    """One shared-context decode step for ``Lq`` in {1,2} (inference.py:785-823).

    With ``k_new``/``v_new`` ``[B,H,1,D]`` given (the N==2 step) both queries see
    context + committed buffers + the new row (:802-814) and the appended caches
    are returned; otherwise the single target query sees context + committed
    buffers (:790-795).  Returns ``(out, k_buf_after, v_buf_after)``.
    """
    if k_new is not None:
        k_all = np.concatenate([np.asarray(k_buf), np.asarray(k_new)], axis=2)
        v_all = np.concatenate([np.asarray(v_buf), np.asarray(v_new)], axis=2)
    else:
        k_all, v_all = np.asarray(k_buf), np.asarray(v_buf)
    out = hybrid_attention(q, k_ctx, v_ctx, k_all, v_all, compute=compute)
    return out, k_all, v_all


def loops_attention(q, k, v, mask=None, scale=None):
    """Pure-Python float64 loops over ``q [Lq,D]``, ``k,v [N,D]`` (tiny inputs only).

    Independent of numpy's einsum/softmax: used to pin the vectorised functions.
    Rows with no visible key give out = 0, lse = -inf.
    """
    Lq, D = len(q), len(q[0])
    N = len(k)
    if scale is None:
        scale = D ** -0.5
    out = [[0.0] * D for _ in range(Lq)]
    lse = [-math.inf] * Lq
    for i in range(Lq):
        s = []
        for j in range(N):
            if mask is not None and not mask[i][j]:
                continue
            acc = 0.0
            for d in range(D):
                acc += float(q[i][d]) * float(k[j][d])
            s.append((j, acc * scale))
        if not s:
            continue
        m = max(x for _, x in s)
        z = sum(math.exp(x - m) for _, x in s)
        lse[i] = m + math.log(z)
        for j, x in s:
            w = math.exp(x - m) / z
            for d in range(D):
                out[i][d] += w * float(v[j][d])
    return out, lse
