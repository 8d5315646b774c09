"""Autoregressive predictor with KV caching (host-side mirror of the reference's
``ar_tabpfn/model/inference.py``), driving the HIP attention kernels.

Same constructor, method names, cache attributes and state as the reference's
``ARTabPFNPredictor``.  Two cache layouts, selected by ``backend`` under the
reference's names:

* ``"triton_shared_context"`` — one context K/V ``[H,Nc,Dh]`` for every trajectory
  (``layer.k_ctx_cache`` / ``v_ctx_cache``) plus a preallocated per-trajectory buffer
  cache ``[B,H,max_buf,Dh]`` (``layer.k_buf_cache`` / ``v_buf_cache``) that decode
  steps append to in place (inference.py:107-122, :746-833).
* ``"flex_attention"`` — one full cache ``[B,H,max_seq,Dh]`` per batch entry
  (``layer.k_cache`` / ``v_cache``) for per-dataset contexts (inference.py:124-135,
  :687-744).

Both run on the same kernels; the names only choose the layout.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from . import attention_kernels as ak
from .attention import DecodeMask, TeacherForcingMask
from . import _lib
from .glue import SampleEmbedStep, DecodeStepBoundary, add_layer_norm

__all__ = ["ARTabPFNPredictor"]


class _GraphState:
    """Static tensors and the recorded graph of the sampling loop."""


_SHARED = "triton_shared_context"
_PER_DATASET = "flex_attention"
_ALIASES = {"shared_context": _SHARED, "per_dataset": _PER_DATASET}


class ARTabPFNPredictor:
    """Joint sampling and log-density evaluation (inference.py:32-453)."""

    def __init__(self, embedder, backbone, head, ar_tokens, backend: str = "flex_attention"):
        self.embedder = embedder
        self.backbone = backbone
        self.head = head
        self.ar_tokens = ar_tokens
        backend = _ALIASES.get(backend, backend)
        if backend not in (_PER_DATASET, _SHARED):
            raise ValueError(f"Unsupported backend: {backend}")
        self.backend = backend
        self.seq_len = 0          # committed keys in the full cache (per-dataset layout)
        self.context_len = 0      # context rows (shared layout)
        self.buffer_len = 0       # committed buffer rows (shared layout)
        self.max_buffer_len = 0   # capacity of the buffer cache (shared layout)
        self._device = None
        self._dtype = None
        # Replay the decode step of sample_sequence from a recorded HIP graph (shared
        # layout on a HIP device only).  Set to False to launch every kernel from Python.
        self.use_hip_graph = True
        # Instead of replaying the recorded graphs, issue the launches they hold one by one from the
        # host: same kernels, streams, ordering and scratch memory (for instrumented runs).
        self.launch_live = False
        self.fuse_step_tail = True   # head + draw + next embedding as one launch inside the graph
        # Run the HBM-bound buffer pass of a decode step on a second stream, next to the
        # compute-bound context pass (shared layout, HIP device).
        self.overlap_buffer_pass = True
        # Leave the attention partials of a decode step unmerged; the layer kernel that follows
        # merges them while loading its input.
        self.merge_in_layer = True
        # Sample the trajectories as this many independent groups, each replaying its own recorded
        # step on its own stream with its own scratch memory.  Measured at B=1024, N_ctx=16384:
        # 2 groups 846 steps/s against 948 for one — a context pass that shares the CUs with another
        # group's buffer pass slows down by as much as the overlap saves — so the default is one.
        self.decode_chains = 1
        # Decode steps recorded into one graph (a replay boundary costs about 5 us on the device); a
        # one-step graph covers the remainder.  Measured at B=1024, N_ctx=16384: 1 step per graph
        # -1.7 %, 8 against 4 +0.2 %, 16 loses what the longer remainder of one-step replays costs.
        self.steps_per_graph = 8
        self.single_steps_first = True  # order of the replays of a run: remainder steps, then the long graphs
        self.fuse_step_boundary = True  # last layer's tail, step tail and first layer's head as one launch
        self.min_chain_batch = 256   # groups smaller than this are not worth their fixed costs
        # Order the two streams of the recorded step through counters in device memory instead of
        # two events per layer (``attention_kernels.QueueOrder``); used when the two streams are found
        # to run concurrently, otherwise (and when set to False) the events are used.
        self.counter_ordering = True
        # In the sampling loop the last layer finishes the target row only: the buffer row's output
        # of that layer is read by nobody (its K/V were cached before the attention call).
        self.target_only_last_layer = True
        self._side_streams = {}
        self._graph_state = None
        self._graph_params = None    # the tensors a recorded step points at (collected at first use)
        self.graph_recordings = 0    # HIP graphs recorded so far (a run that only replays leaves it unchanged)

    @classmethod
    def from_trained_model(cls, model, backend: str = "flex_attention") -> "ARTabPFNPredictor":
        return cls(model.embedder, model.backbone, model.head, model.ar_tokens, backend=backend)

    # ------------------------------------------------------------------ cache state

    def init_kv_cache(self, batch_size: int, max_seq_len: int, device=None, dtype=None) -> None:
        """Allocate the caches.  ``max_seq_len`` is the buffer capacity for the shared
        layout and context + buffers (+ targets for teacher forcing) for the full cache,
        as in the reference (inference.py:94-95)."""
        if device is None or dtype is None:
            param = next(self.backbone.parameters())
            device = device or param.device
            dtype = dtype or param.dtype
        self._device, self._dtype = device, dtype
        self.seq_len = self.context_len = self.buffer_len = 0
        def zeros(layer, name, shape):
            # same contents as a fresh torch.zeros; memory (and its address, which recorded
            # HIP graphs refer to) is kept when the shape, dtype and device are unchanged
            old = getattr(layer, name, None)
            if (isinstance(old, torch.Tensor) and tuple(old.shape) == tuple(shape) and old.dtype == dtype
                    and old.device == torch.device(device) and old.is_contiguous()):
                old.zero_()
            else:
                setattr(layer, name, torch.zeros(shape, device=device, dtype=dtype))

        if self.backend == _SHARED:
            self.max_buffer_len = max_seq_len
            for layer in self.backbone.layers:
                H, Dh = layer.attn_rows.n_heads, layer.attn_rows.head_dim
                old = getattr(layer, "k_ctx_cache", None)
                if not (isinstance(old, torch.Tensor) and old.dim() == 3 and old.shape[0] == H and old.shape[2] == Dh
                        and old.dtype == dtype and old.device == torch.device(device)):
                    layer.k_ctx_cache = torch.empty((H, 0, Dh), device=device, dtype=dtype)
                    layer.v_ctx_cache = torch.empty_like(layer.k_ctx_cache)
                zeros(layer, "k_buf_cache", (batch_size, H, max_seq_len, Dh))
                zeros(layer, "v_buf_cache", (batch_size, H, max_seq_len, Dh))
            return
        self.max_buffer_len = 0
        for layer in self.backbone.layers:
            H, Dh = layer.attn_rows.n_heads, layer.attn_rows.head_dim
            zeros(layer, "k_cache", (batch_size, H, max_seq_len, Dh))
            zeros(layer, "v_cache", (batch_size, H, max_seq_len, Dh))

    def _side_stream(self, device, tag=0):
        if device.type != "cuda":
            return None
        key = (device.index if device.index is not None else torch.cuda.current_device(), tag)
        current = torch.cuda.current_stream(device)
        side = self._side_streams.get(key)
        if side is None or side.cuda_stream == current.cuda_stream:
            # torch hands out streams from a small pool, round-robin, and the runtime serves them from a
            # few hardware queues: a "new" stream can be the one that is current, or share its queue,
            # and the two passes would silently run one after the other.  Probe for one that does not.
            if torch.cuda.is_current_stream_capturing():
                for _ in range(8):
                    side = torch.cuda.Stream(device=device)  # default priority
                    if side.cuda_stream != current.cuda_stream:
                        break
            else:
                side, _ = ak.concurrent_stream(device, current)
            self._side_streams[key] = side
        return side

    def clear_cache(self) -> None:
        """Reset the cursors, keep the memory (inference.py:137-141)."""
        self.seq_len = self.context_len = self.buffer_len = 0

    # ------------------------------------------------------------------ the layer stack

    def _run_layers(self, x_row: Optional[Tensor], attend, last_layer_rows: Optional[slice] = None, state=None,
                    finish=None) -> Tensor:
        """``x_row [B,N,D]`` through every layer; ``attend(layer, q, k, v) -> [B,H,N,Dh]`` is the
        row attention of the pass at hand (it also owns the cache writes).  Between two
        attention calls the tail of one layer and the head of the next run as one launch where
        the fused kernels cover them (``TwoStageTransformerLayer.finish_then_pre``).

        ``last_layer_rows`` names the rows whose output the caller will read.  A row's output of
        the last layer feeds nothing but that read (its K/V for the caches come from the
        projection in front of the attention call, which still sees every row), so the last layer
        runs its queries and everything behind them for those rows only; the result is then
        ``[B, len(rows), D]``.  A decode step reads the target row alone (inference.py:318-320):
        half the queries of the last context pass.

        ``state``: the first layer's ``pre_attention`` result when somebody has computed it
        already (``x_row`` is then not read); ``finish(y, attn)``: what to do with the last
        layer's feature stage and attention output instead of ``layer.finish`` (the step
        boundary launch of a recorded decode step, whose result this function then returns)."""
        layers = list(self.backbone.layers)
        if state is None:
            state = layers[0].pre_attention(x_row)
        for idx, layer in enumerate(layers):
            y, q, k, v = state
            if idx + 1 == len(layers):
                if last_layer_rows is not None:
                    y, q = y[:, last_layer_rows], q[:, :, last_layer_rows]
                attn = attend(layer, q, k, v)
                return finish(y, attn) if finish is not None else layer.finish(y, attn)
            state = layer.finish_then_pre(y, attend(layer, q, k, v), layers[idx + 1])

    # ------------------------------------------------------------------ prefill

    @torch.no_grad()
    def prefill_context(self, x_context: Tensor, y_context: Tensor) -> None:
        """Encode the context and fill the caches; rows ``[0,Nc)`` hold context K/V
        afterwards (inference.py:143-178)."""
        if self.backend == _SHARED:
            self.prefill_context_shared(x_context, y_context)
            return
        x_row = self.embedder.embed_context(x_context, y_context)
        Nc = x_row.shape[1]
        for layer in self.backbone.layers:
            if layer.k_cache.shape[2] < Nc:
                raise ValueError("KV cache too small for the context; call init_kv_cache with a larger max_seq_len.")
        self._run_layers(x_row, lambda layer, q, k, v: ak.prefill_attention(q, k, v, layer.k_cache, layer.v_cache))
        self.seq_len = Nc

    @torch.no_grad()
    def prefill_context_shared(self, x_context: Tensor, y_context: Tensor) -> None:
        """Shared layout: only batch entry 0 is encoded — the context is taken to be the
        same for every trajectory (inference.py:180-223)."""
        Nc = x_context.shape[1]
        x_row = self.embedder.embed_context(x_context[0:1], y_context[0:1])
        for layer in self.backbone.layers:
            H, Dh = layer.attn_rows.n_heads, layer.attn_rows.head_dim
            if layer.k_ctx_cache.shape[1] != Nc or layer.k_ctx_cache.shape[0] != H:
                layer.k_ctx_cache = torch.zeros(H, Nc, Dh, device=x_row.device, dtype=x_row.dtype)
                layer.v_ctx_cache = torch.zeros_like(layer.k_ctx_cache)
        self._run_layers(
            x_row, lambda layer, q, k, v: ak.prefill_attention(q, k, v, layer.k_ctx_cache, layer.v_ctx_cache))
        self.context_len = Nc
        self.buffer_len = 0
        self.seq_len = Nc
        self._prefill_batch_size = x_context.shape[0]

    # ------------------------------------------------------------------ decode

    @torch.no_grad()
    def transformer_decode(self, embedding: Tensor, commit: int) -> Tensor:
        """Run ``[B,N,D]`` new rows through the stack against the caches and commit the
        first ``commit`` of them (N-1 for ``[buffer, target]``, 0 for ``[target]``);
        returns the normed ``[B,N,D]`` (inference.py:225-276)."""
        B, N, D = embedding.shape
        x_row = embedding
        if self.backend == _SHARED:
            if self.buffer_len + commit > self.max_buffer_len:
                raise ValueError("Shared-context buffer cache exceeded; increase max buffer length.")
            if N not in (1, 2):
                raise ValueError("Shared-context decode only supports N=1 (target) or N=2 (buffer, target).")
            x_row = self._run_layers(x_row, lambda layer, q, k, v: self._attend_decode_shared(layer, q, k, v))
            self.buffer_len += commit
            self.seq_len = self.context_len + self.buffer_len
            return add_layer_norm(x_row, None, None, self.backbone.norm)

        mask = DecodeMask(num_cached=self.seq_len, num_new=N)
        start = self.seq_len
        x_row = self._run_layers(x_row, lambda layer, q, k, v: self._attend_with_cache(layer, q, k, v, mask, start))
        self.seq_len += commit
        return add_layer_norm(x_row, None, None, self.backbone.norm)

    def _layer_decode_with_cache_shared(self, layer, x_row: Tensor, commit: int = 1,
                                        n_buf_device: Optional[Tensor] = None) -> Tensor:
        """One layer of a decode step on the shared layout (inference.py:746-833): both
        queries of a ``[buffer, target]`` pair see context + committed buffers + the new
        buffer row, which is appended in place by the same kernel call."""
        B, N, D = x_row.shape
        if N not in (1, 2):
            raise ValueError("Shared-context decode only supports N=1 (target) or N=2 (buffer, target).")
        x_row, q, k_new, v_new = layer.pre_attention(x_row)
        return layer.finish(x_row, self._attend_decode_shared(layer, q, k_new, v_new, n_buf_device))

    def _attend_decode_shared(self, layer, q: Tensor, k_new: Tensor, v_new: Tensor,
                              n_buf_device: Optional[Tensor] = None, rows: Optional[slice] = None,
                              chain: int = 0, order=None) -> Tensor:
        """The attention call of a shared-layout decode step (inference.py:785-823).  ``rows``
        restricts it to a group of trajectories (a slice of the batch axis of the buffer cache)."""
        # k_new / v_new hold every new row of the step — [target] or [buffer, target] — even when q
        # has been cut down to the rows whose output is read
        has_buffer_row = k_new.shape[2] == 2
        k_ctx = layer.k_ctx_cache[:, : self.context_len]
        v_ctx = layer.v_ctx_cache[:, : self.context_len]
        k_buf = layer.k_buf_cache if rows is None else layer.k_buf_cache[rows]
        v_buf = layer.v_buf_cache if rows is None else layer.v_buf_cache[rows]
        # with a device-side length the host value is only the bound that is validated
        n_buf = self.buffer_len if n_buf_device is None else self.max_buffer_len - (1 if has_buffer_row else 0)
        side = self._side_stream(q.device, chain) if self.overlap_buffer_pass else None
        # where the layer's fused kernel can merge the partial results itself, leave them unmerged
        partials = self.merge_in_layer and layer.fused_for(q)
        if not has_buffer_row:
            attn = ak.decode_attention(q, k_ctx, v_ctx, k_buf, v_buf, n_buf,
                                       n_buf_device=n_buf_device, side_stream=side, leave_partials=partials)
        else:
            attn = ak.decode_attention(
                q, k_ctx, v_ctx, k_buf, v_buf, n_buf,
                k_new[:, :, 0:1], v_new[:, :, 0:1], n_buf_device=n_buf_device, side_stream=side,
                leave_partials=partials, order=order,
            )
        return attn

    def _layer_decode_with_cache(self, layer, x_row: Tensor, mask, cache_start: int) -> Tensor:
        """One layer on the full per-dataset cache (inference.py:687-744): the new K/V are
        written at ``[cache_start, cache_start+N)`` and the queries attend under ``mask``."""
        x_row, q, k_new, v_new = layer.pre_attention(x_row)
        return layer.finish(x_row, self._attend_with_cache(layer, q, k_new, v_new, mask, cache_start))

    def _attend_with_cache(self, layer, q: Tensor, k_new: Tensor, v_new: Tensor, mask, cache_start: int) -> Tensor:
        """Cache write + attention of one layer on the per-dataset layout (inference.py:704-741)."""
        N = q.shape[2]
        if layer.k_cache.shape[2] < cache_start + N:
            raise ValueError("KV cache exceeded; increase max_seq_len.")
        if isinstance(mask, TeacherForcingMask):
            Nt = mask.num_targets
            layer.k_cache[:, :, cache_start : cache_start + N] = k_new
            layer.v_cache[:, :, cache_start : cache_start + N] = v_new
            attn = ak.teacher_forcing_attention(
                q, layer.k_cache[:, :, :cache_start], layer.v_cache[:, :, :cache_start],
                k_new[:, :, :Nt], v_new[:, :, :Nt], Nt,
            )
        elif N in (1, 2):
            # context = cached keys of this batch entry; the new buffer row lands in slot
            # cache_start of the same cache (the "buffer" view starts there)
            k_tail, v_tail = layer.k_cache[:, :, cache_start:], layer.v_cache[:, :, cache_start:]
            attn = ak.decode_attention(
                q, layer.k_cache[:, :, :cache_start], layer.v_cache[:, :, :cache_start], k_tail, v_tail, 0,
                k_new[:, :, 0:1] if N == 2 else None, v_new[:, :, 0:1] if N == 2 else None,
            )
            if N == 2:  # the reference also parks the target's K/V behind it until the next step
                layer.k_cache[:, :, cache_start + 1 : cache_start + 2] = k_new[:, :, 1:2]
                layer.v_cache[:, :, cache_start + 1 : cache_start + 2] = v_new[:, :, 1:2]
            else:
                layer.k_cache[:, :, cache_start : cache_start + 1] = k_new
                layer.v_cache[:, :, cache_start : cache_start + 1] = v_new
        else:
            # general N: cached keys + causal part among the new rows (inference.py:512-519)
            layer.k_cache[:, :, cache_start : cache_start + N] = k_new
            layer.v_cache[:, :, cache_start : cache_start + N] = v_new
            out_c, lse_c = ak.context_attention(q, layer.k_cache[:, :, :cache_start], layer.v_cache[:, :, :cache_start])
            qi = torch.arange(N, device=q.device)[:, None]
            kj = torch.arange(N, device=q.device)[None, :]
            new_mask = torch.where(qi == N - 1, kj < qi, kj <= qi)[None, None]
            out_n, lse_n = ak.buffer_attention(q, k_new, v_new, mask=new_mask)
            attn = ak.merge_attention_outputs(out_c, lse_c, out_n, lse_n)
        return attn

    @torch.no_grad()
    def autoregressive_decode(self, x_target: Tensor, prev_x: Optional[Tensor] = None,
                              prev_y: Optional[Tensor] = None, ar_idx: int = 0) -> Tensor:
        """Decode one target, feeding the previous prediction back as a buffer row;
        returns the sampled ``[B,1]`` (inference.py:278-320)."""
        target_emb = self.embedder.embed_target(x_target)
        if prev_x is not None and prev_y is not None:
            buffer_emb = self.embedder.embed_buffer(prev_x, prev_y) + self.ar_tokens[ar_idx]
            embedding, commit = torch.cat([buffer_emb, target_emb], dim=1), 1
        else:
            embedding, commit = target_emb, 0
        z = self.transformer_decode(embedding, commit=commit)
        return self.head.sample(z[:, -1:, :])[:, :, 0, 0]

    @torch.no_grad()
    def sample_sequence(self, x_context: Tensor, y_context: Tensor, x_target: Tensor) -> Tensor:
        """Sample all targets autoregressively -> ``[B,Nt]`` (inference.py:322-366).

        On a HIP device with the shared layout the steps after the first are replayed
        from one recorded HIP graph (same kernels, same order; the step index and the
        buffer length live in device memory), which removes the per-kernel launch cost
        of the Python loop."""
        B, Nc, _ = x_context.shape
        Nt = x_target.shape[1]
        device, dtype = x_context.device, x_context.dtype
        self.init_kv_cache(B, Nt if self.backend == _SHARED else Nc + Nt, device, dtype)
        self.prefill_context(x_context, y_context)
        return self.decode_targets(x_target)

    @torch.no_grad()
    def decode_targets(self, x_target: Tensor) -> Tensor:
        """The decode loop of ``sample_sequence`` (inference.py:353-366) on caches that
        are already initialised and prefilled: samples ``x_target [B,Nt,F]`` in order."""
        Nt = x_target.shape[1]
        if (self.use_hip_graph and self.backend == _SHARED and x_target.is_cuda and Nt >= 3
                and self.buffer_len == 0 and Nt <= self.max_buffer_len):
            return self._sample_sequence_graph(x_target)
        preds = []
        prev_x = prev_y = None
        for t in range(Nt):
            x_t = x_target[:, t : t + 1, :]
            y_t = self.autoregressive_decode(x_t, prev_x, prev_y, t % self.ar_tokens.shape[0])
            preds.append(y_t)
            prev_x, prev_y = x_t, y_t
        return torch.cat(preds, dim=1)

    def _graph_step(self, st) -> None:
        """One ``[buffer, target]`` decode step driven entirely by device-side state
        (the body that is recorded): step index ``st.t``, buffer length ``st.nbuf``."""
        if st.boundary is not None:
            # the previous step's boundary launch has left the first layer's feature stage and
            # projections of this step's rows; this step's ends with the same launch
            self._run_layers(
                None, lambda layer, q, k, v: self._attend_decode_shared(layer, q, k, v, n_buf_device=st.nbuf,
                                                                        rows=st.rows, chain=st.chain,
                                                                        order=st.order_active),
                last_layer_rows=self._last_layer_rows(), state=st.boundary.state, finish=st.boundary)
            return
        if st.tail is not None:
            # embedding of this step was left in st.emb by the previous step's tail launch
            x_row = self._run_layers(
                st.emb, lambda layer, q, k, v: self._attend_decode_shared(layer, q, k, v, n_buf_device=st.nbuf,
                                                                          rows=st.rows, chain=st.chain,
                                                                          order=st.order_active),
                last_layer_rows=self._last_layer_rows())
            st.tail(x_row)          # norm, head, draw, preds[:, t], embedding of step t + 1, (t, nbuf) += 1
            return
        bs = self.ar_tokens.shape[0]
        t = st.t.long()
        x_t = st.x_target.index_select(1, t)
        x_p = st.x_target.index_select(1, t - 1)
        tok = self.ar_tokens.index_select(0, torch.remainder(t, bs))  # ar_tokens[t % bs], inference.py:359
        buffer_emb = self.embedder.embed_buffer(x_p, st.y_prev) + tok
        x_row = torch.cat([buffer_emb, self.embedder.embed_target(x_t)], dim=1)
        x_row = self._run_layers(
            x_row, lambda layer, q, k, v: self._attend_decode_shared(layer, q, k, v, n_buf_device=st.nbuf,
                                                                      rows=st.rows, chain=st.chain,
                                                                      order=st.order_active),
            last_layer_rows=self._last_layer_rows())
        z = add_layer_norm(x_row, None, None, self.backbone.norm)
        y = self.head.sample(z[:, -1:, :])[:, :, 0, 0]
        st.preds.index_copy_(1, t, y)
        st.y_prev.copy_(y)
        st.counters.add_(1)

    def _first_step(self, st) -> None:
        """The step of the first target (``[target]`` alone, empty buffer) in the form that can be
        recorded: embedding from the device-side copy of the targets, the layer stack against the
        context, then the one-launch tail with the step counter at 0."""
        emb0 = self.embedder.embed_target(st.x_target[:, 0:1])
        x_row = self._run_layers(emb0, lambda layer, q, k, v: self._attend_decode_shared(layer, q, k, v,
                                                                                        rows=st.rows, chain=st.chain),
                                 finish=st.boundary)
        if st.boundary is None:
            st.tail(x_row)  # norm, head, draw, preds[:, 0], embedding of step 1, (t, nbuf) += 1
        st.nbuf.zero_()     # the first target commits no buffer row

    def _last_layer_rows(self) -> Optional[slice]:
        """Rows of a ``[buffer, target]`` step that the last layer has to finish: the target."""
        return slice(1, 2) if self.target_only_last_layer else None

    def _chain_rows(self, B: int):
        """Batch slices of the trajectory groups that are sampled side by side."""
        n = max(1, int(self.decode_chains))
        while n > 1 and B // n < self.min_chain_batch:
            n -= 1
        bounds = [B * i // n for i in range(n + 1)]
        return [slice(bounds[i], bounds[i + 1]) for i in range(n)]

    def _sample_sequence_graph(self, x_target: Tensor) -> Tensor:
        B, Nt, F_ = x_target.shape
        device, dtype = x_target.device, x_target.dtype
        layer0 = self.backbone.layers[0]
        # (walking the module tree costs a millisecond of host time with the GPU idle: done once; a
        # weight that is updated or moved changes its version or address and is seen through the key)
        if self._graph_params is None:
            self._graph_params = (list(self.backbone.parameters()) + list(self.embedder.parameters()) +
                                  list(self.head.parameters()) + [self.ar_tokens])
        params = self._graph_params
        chain_rows = self._chain_rows(B)
        # The recorded step depends on the capacity of the buffer cache, not on how many steps are
        # replayed: loop state is sized for the capacity, so runs of any length share one recording.
        cap = self.max_buffer_len
        key = (B, cap, F_, self.context_len, dtype, str(device), layer0.k_ctx_cache.data_ptr(),
               layer0.k_buf_cache.data_ptr(), self.fuse_step_tail, self.overlap_buffer_pass, self.merge_in_layer,
               len(chain_rows), int(self.steps_per_graph), bool(self.counter_ordering),
               bool(self.target_only_last_layer), bool(self.fuse_step_boundary), tuple((p.data_ptr(), p._version) for p in params))
        gs = self._graph_state
        if gs is None or gs.key != key:
            gs = _GraphState()
            gs.key = key
            gs.x_target = torch.zeros((B, cap, F_), device=device, dtype=dtype)
            gs.chains = []
            fused_tail = self.fuse_step_tail and SampleEmbedStep.supported(self.embedder, self.backbone, self.head,
                                                                           x_target)
            for idx, rows in enumerate(chain_rows):
                st = _GraphState()
                Bc = rows.stop - rows.start
                st.rows = rows if len(chain_rows) > 1 else None
                st.chain = idx
                st.stream = torch.cuda.Stream(device=device) if len(chain_rows) > 1 else None  # default priority
                st.x_target = gs.x_target[rows]
                st.y_prev = torch.zeros((Bc, 1), device=device, dtype=dtype)
                st.preds = torch.zeros((Bc, cap), device=device, dtype=dtype)
                st.counters = torch.zeros(2, device=device, dtype=torch.int32)  # (step index t, buffer length)
                st.t, st.nbuf = st.counters[0:1], st.counters[1:2]
                st.graph = None
                st.graph_many = None   # steps_per_graph steps in one graph
                st.graph_first = None  # the first target's step (no buffer row yet)
                st.tail = None
                st.boundary = None  # last post + tail + first pre of the next step as one launch
                st.order = st.order_active = None
                if self._counter_ordering_applies(x_target):
                    order = ak.QueueOrder(device)
                    if order.streams_run_concurrently(torch.cuda.current_stream(device),
                                                      self._side_stream(device, idx)):
                        st.order = order
                if fused_tail:
                    D = self.backbone.d_model
                    st.emb = torch.zeros((Bc, 2, D), device=device, dtype=dtype)
                    st.x_mean = torch.zeros((Bc, cap), device=device, dtype=dtype)
                    st.rand_u = torch.zeros((cap, Bc), device=device, dtype=torch.float32)
                    st.rand_n = torch.zeros((cap, Bc), device=device, dtype=torch.float32)
                    st.tail = SampleEmbedStep(self.embedder, self.backbone, self.head, self.ar_tokens, st.x_mean,
                                              st.rand_u, st.rand_n, st.t, st.preds, st.emb, advance=st.counters)
                    layers = self.backbone.layers
                    if (self.fuse_step_boundary and self.target_only_last_layer
                            and DecodeStepBoundary.supported(st.tail, layers[0], layers[-1], x_target)):
                        st.boundary = DecodeStepBoundary(
                            st.tail, layers[0], layers[-1], torch.zeros((Bc, 2, D), device=device, dtype=dtype),
                            torch.zeros((Bc, 2, 3 * D), device=device, dtype=dtype))
                gs.chains.append(st)
            gs.tail = gs.chains[0].tail
            self._graph_state = gs
        gs.x_target[:, :Nt].copy_(x_target)

        current = torch.cuda.current_stream(device)
        # First target: no buffer row yet (N = 1).  With the one-launch tail and one trajectory
        # group it is a recorded graph of its own (the tail draws y_0, writes it, leaves the
        # embedding of step 1 and moves the step counter on); otherwise it is launched directly.
        recorded_first = gs.tail is not None and len(gs.chains) == 1 and cap >= 2
        if gs.tail is not None:
            x_mean = gs.x_target[:, :Nt].mean(dim=-1)
            for st in gs.chains:
                rows = st.rows if st.rows is not None else slice(0, B)
                st.x_mean[:, :Nt].copy_(x_mean[rows])
                self._draw_step_variates(st.rand_u, st.rand_n)
        if recorded_first:
            st = gs.chains[0]
            if st.graph_first is None:
                with _lib.workspace_tag(1 + st.chain):
                    warm = torch.cuda.Stream(device=device)
                    warm.wait_stream(current)
                    with torch.cuda.stream(warm):
                        st.counters.zero_()
                        self._first_step(st)
                    current.wait_stream(warm)
                    st.graph_first = torch.cuda.CUDAGraph()
                    self.graph_recordings += 1
                    with torch.cuda.graph(st.graph_first):
                        self._first_step(st)
                    st.workspace_first = _lib.held_workspace(device)
            st.counters.zero_()
            self._run_recorded(st, "graph_first")
            y0 = emb1 = None
            if st.graph is None:  # the step graphs are still to be recorded: their warm-up starts from here
                y0, emb1 = st.preds[:, 0:1].clone(), st.emb.clone()
        else:
            y0 = self.autoregressive_decode(gs.x_target[:, 0:1, :], None, None, 0)
            emb1 = None
            if gs.tail is not None:
                bs = self.ar_tokens.shape[0]
                emb1 = torch.cat([self.embedder.embed_buffer(gs.x_target[:, 0:1], y0) + self.ar_tokens[1 % bs],
                                  self.embedder.embed_target(gs.x_target[:, 1:2])], dim=1)

        def reset(st):
            rows = st.rows if st.rows is not None else slice(0, B)
            st.y_prev.copy_(y0[rows])
            st.preds[:, 0:1] = y0[rows]
            st.t.fill_(1)
            st.nbuf.zero_()
            if st.tail is not None:
                st.emb.copy_(emb1[rows])
            if st.boundary is not None:
                st.boundary.load_state(st.emb)

        for st in gs.chains:
            if st.graph is not None:
                continue
            # warm-up on a side stream (workspace allocation, GEMM heuristics), then record;
            # the rows the warm-up steps append are overwritten by the real steps
            with _lib.workspace_tag(1 + st.chain):  # scratch of its own: eager calls use tag 0
                warm = torch.cuda.Stream(device=device)
                warm.wait_stream(current)
                with torch.cuda.stream(warm):
                    reset(st)
                    for _ in range(2):
                        self._graph_step(st)
                current.wait_stream(warm)
                reset(st)
                st.graph = self._record_steps(st, 1)
                if self.steps_per_graph > 1 and cap - 1 >= self.steps_per_graph:
                    reset(st)
                    st.graph_many = self._record_steps(st, self.steps_per_graph)
                # the recorded launches point into this scratch tensor: it lives as long as they do
                st.workspace = _lib.held_workspace(device)
                # a graph's first launch costs about half a millisecond more than the later ones
                # (it is set up on the device then): paid here, once, and not by the first run
                # that is long enough to use the graph
                for graph in (st.graph, st.graph_many):
                    if graph is not None:
                        reset(st)
                        graph.replay()
        gs.graph = gs.chains[0].graph
        if y0 is not None:  # (a recorded first step has left exactly this state behind)
            for st in gs.chains:
                reset(st)
        k = self.steps_per_graph if gs.chains[0].graph_many is not None else 1
        n_many, n_single = (Nt - 1) // k if k > 1 else 0, (Nt - 1) % k if k > 1 else Nt - 1
        # The one-step replays come first, so that the host queues the first long graph while
        # they run (measured: nothing at 20 steps, +0.4 % at 256).
        first_many = 0 if self.single_steps_first else n_many
        order = [i < first_many or i >= first_many + n_single for i in range(n_many + n_single)]
        if len(gs.chains) == 1:
            for many in order:
                self._run_recorded(gs.chains[0], "graph_many" if many else "graph")
        else:
            # every group replays its own step on its own stream; they meet again at the end
            for st in gs.chains:
                st.stream.wait_stream(current)
            for many in order:
                for st in gs.chains:
                    with torch.cuda.stream(st.stream):
                        self._run_recorded(st, "graph_many" if many else "graph")
            for st in gs.chains:
                current.wait_stream(st.stream)
        # the result is copied before the host waits for the failure flag of the counters, so that
        # the device does not sit idle between the last step and the copy
        result = (gs.chains[0].preds[:, :Nt].clone() if len(gs.chains) == 1
                  else torch.cat([st.preds[:, :Nt] for st in gs.chains], dim=0))
        if any(st.order is not None and st.order.failed() for st in gs.chains):
            # a wait on the counters timed out: the recorded streams did not run side by side.
            # The step's results are void; record it again with events and sample afresh.
            for st in gs.chains:
                if st.order is not None:
                    st.order.reset()
            self.counter_ordering = False
            self._graph_state = None
            return self._sample_sequence_graph(x_target)
        self.buffer_len = Nt - 1
        self.seq_len = self.context_len + self.buffer_len
        return result

    def _counter_ordering_applies(self, x: Tensor) -> bool:
        """Whether every layer's decode call takes the schedule that the counters can order: the
        streaming buffer pass beside the context pass, partials merged by the fused layer kernel."""
        if not (self.counter_ordering and self.overlap_buffer_pass and self.merge_in_layer and self.fuse_step_tail):
            return False
        return all(layer.attn_rows.head_dim == 32 and layer.fused_for(x) for layer in self.backbone.layers)

    def _issue_steps(self, st, n_steps: int) -> None:
        """The launches of ``n_steps`` decode steps of one trajectory group, on the current stream
        (and its side stream).  With counter ordering the side stream is forked once and rejoins
        at the end; the per-layer dependencies between the two streams are the counters' waits."""
        if st.order is None:
            for _ in range(n_steps):
                self._graph_step(st)
            return
        main = torch.cuda.current_stream()
        side = self._side_stream(main.device, st.chain)
        side.wait_stream(main)
        st.order_active = st.order
        try:
            for _ in range(n_steps):
                self._graph_step(st)
        finally:
            st.order_active = None
            main.wait_stream(side)

    def _record_steps(self, st, n_steps: int) -> "torch.cuda.CUDAGraph":
        """Record ``n_steps`` decode steps of one trajectory group into a HIP graph."""
        graph = torch.cuda.CUDAGraph()
        self.graph_recordings += 1
        with torch.cuda.graph(graph):
            self._issue_steps(st, n_steps)
        return graph

    def _run_recorded(self, st, which: str) -> None:
        """Replay one of the group's recorded graphs — or, with ``launch_live``, issue the very
        launches it holds one by one from the host (same kernels, streams, ordering and scratch
        memory; for instrumented runs, whose per-launch events cannot sit inside a graph)."""
        if not self.launch_live:
            getattr(st, which).replay()
            return
        with _lib.workspace_tag(1 + st.chain):
            if which == "graph_first":
                self._first_step(st)
            else:
                self._issue_steps(st, self.steps_per_graph if which == "graph_many" else 1)

    @staticmethod
    def _draw_step_variates(rand_u: Tensor, rand_n: Tensor) -> None:
        """Fresh variates for every (step, trajectory) of one sampling run, from torch's
        generator: uniform for the component pick, normal for the draw."""
        rand_u.uniform_()
        rand_n.normal_()

    # ------------------------------------------------------------------ teacher forcing

    @torch.no_grad()
    def evaluate_joint_density(self, x_context: Tensor, y_context: Tensor, x_target: Tensor,
                               y_target: Tensor) -> Tensor:
        """Log-density ``[B,Nt]`` of the targets in one teacher-forced pass
        (inference.py:368-453)."""
        if self.backend == _SHARED:
            return self._evaluate_joint_density_shared(x_context, y_context, x_target, y_target)
        return self._evaluate_joint_density_flex(x_context, y_context, x_target, y_target)

    def _teacher_forcing_embedding(self, x_target: Tensor, y_target: Tensor) -> Tensor:
        Nt = x_target.shape[1]
        pos = torch.arange(Nt, device=x_target.device) % self.ar_tokens.shape[0]
        buffer_emb = self.embedder.embed_buffer(x_target, y_target) + self.ar_tokens[pos]
        return torch.cat([buffer_emb, self.embedder.embed_target(x_target)], dim=1)

    def _evaluate_joint_density_shared(self, x_context, y_context, x_target, y_target) -> Tensor:
        B, Nt = x_context.shape[0], x_target.shape[1]
        self.init_kv_cache(B, Nt, x_context.device, x_context.dtype)
        self.prefill_context(x_context, y_context)
        z = self._teacher_forcing_decode_shared(self._teacher_forcing_embedding(x_target, y_target), Nt)
        return self.head.log_likelihood(z[:, Nt:, :], y_target.unsqueeze(-1))

    def _evaluate_joint_density_flex(self, x_context, y_context, x_target, y_target) -> Tensor:
        B, Nc = x_context.shape[0], x_context.shape[1]
        Nt = x_target.shape[1]
        self.init_kv_cache(B, Nc + 2 * Nt, x_context.device, x_context.dtype)
        self.prefill_context(x_context, y_context)
        z = self._teacher_forcing_decode(self._teacher_forcing_embedding(x_target, y_target), Nt)
        return self.head.log_likelihood(z[:, Nt:, :], y_target.unsqueeze(-1))

    @torch.no_grad()
    def _teacher_forcing_decode(self, embedding: Tensor, num_targets: int) -> Tensor:
        """``[buffers, targets]`` under the teacher-forcing mask on the full cache
        (inference.py:455-471)."""
        if embedding.shape[1] != 2 * num_targets:
            raise ValueError("Expected N == 2*num_targets for teacher forcing.")
        mask = TeacherForcingMask(num_cached=self.seq_len, num_targets=num_targets)
        start = self.seq_len
        x_row = self._run_layers(embedding, lambda layer, q, k, v: self._attend_with_cache(layer, q, k, v, mask, start))
        return add_layer_norm(x_row, None, None, self.backbone.norm)

    @torch.no_grad()
    def _teacher_forcing_decode_shared(self, embedding: Tensor, num_targets: int) -> Tensor:
        if embedding.shape[1] != 2 * num_targets:
            raise ValueError("Expected N == 2*num_targets for teacher forcing.")
        x_row = self._run_layers(
            embedding, lambda layer, q, k, v: self._attend_teacher_forcing_shared(layer, q, k, v, num_targets))
        return add_layer_norm(x_row, None, None, self.backbone.norm)

    def _layer_teacher_forcing_shared(self, layer, x_row: Tensor, num_targets: int) -> Tensor:
        """inference.py:835-890: buffer K/V are the fresh projections of the first Nt
        rows; the buffer cache is neither read nor written."""
        B, N, D = x_row.shape
        if N != 2 * num_targets:
            raise ValueError("Expected N == 2*num_targets for teacher forcing.")
        x_row, q, k, v = layer.pre_attention(x_row)
        return layer.finish(x_row, self._attend_teacher_forcing_shared(layer, q, k, v, num_targets))

    def _attend_teacher_forcing_shared(self, layer, q: Tensor, k: Tensor, v: Tensor, num_targets: int) -> Tensor:
        return ak.hybrid_teacher_forcing_attention(
            q, layer.k_ctx_cache[:, : self.context_len], layer.v_ctx_cache[:, : self.context_len],
            k[:, :, :num_targets], v[:, :, :num_targets], num_targets,
        )
