"""PyTorch-CPU restatement of the reference's inference path, op for op
(TEST INFRASTRUCTURE ONLY — never imported by the shipped package).

The numpy oracle beside this file fixes *values* (float64).  This module fixes *cost*: it runs the
same sequence of torch operations the reference runs when it has no device kernel — the branch
``use_triton and HAS_TRITON and q.is_cuda`` is false (triton_kernels.py:744-747) — so that timing
it on a host gives the "reference CPU path" figure a GPU result is reported next to:

* ``pytorch_context_attention`` (triton_kernels.py:532-567): K/V expanded as a stride-0 view
  ``[B,H,Nc,Dh]`` (:554-555), scores ``[B,H,Lq,Nc]`` materialised in the input dtype (:558),
  log-sum-exp of ``scores.float()`` (:561), softmax in the input dtype (:564);
* ``pytorch_buffer_attention`` (:570-614) with the optional boolean mask and the
  fully-masked-row rule (:598-611);
* ``merge_attention_outputs`` (:478-524);
* the teacher-forcing buffer mask and its attention (:620-659), ``hybrid_attention`` (:705-755)
  and ``hybrid_teacher_forcing_attention`` (:662-702);
* one decode layer ``_layer_decode_with_cache_shared`` (inference.py:746-833): feature attention
  over the single column *with* its q/k projections and softmax (dead work the reference does),
  two ``hybrid_attention`` calls, ``torch.cat`` of the buffer (:806-807), slice-assign append
  (:816-821), out_proj / norm2 / feed-forward / norm3 (:825-831);
* ``transformer_decode`` + ``autoregressive_decode`` (inference.py:225-320) with ``head.sample``
  (model.py:251-266);
* the per-dataset log-density path (inference.py:422-471, :525-577, :579-631, :687-744), whose
  ``flex_attention`` calls are restated as what flex's eager CPU fallback computes: scores in
  float32, boolean mask, softmax, output cast back to the input dtype.

Weights come as a ``state_dict`` (the reference's key names).  Every function is pinned against
the numpy oracle in ``tests/test_oracle.py`` (float32: 1e-4; the bf16 run only by its cost, which
is what it is for).
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch
import torch.nn.functional as F

Tensor = torch.Tensor
MARKER = {"target": 0, "context": 1, "buffer": 2}  # model.py:36-38


# ---------------------------------------------------------------------------------------------
# attention (triton_kernels.py:478-755)
# ---------------------------------------------------------------------------------------------

def merge_attention_outputs(out_ctx: Tensor, lse_ctx: Tensor, out_buf: Tensor, lse_buf: Tensor) -> Tensor:
    """triton_kernels.py:508-524."""
    lse_max = torch.maximum(lse_ctx, lse_buf)
    w_ctx = torch.exp(lse_ctx - lse_max)
    w_buf = torch.exp(lse_buf - lse_max)
    w_total = w_ctx + w_buf
    w_ctx = w_ctx / w_total
    w_buf = w_buf / w_total
    merged = w_ctx.unsqueeze(-1) * out_ctx + w_buf.unsqueeze(-1) * out_buf
    return merged.to(out_ctx.dtype)


def pytorch_context_attention(q: Tensor, k_ctx: Tensor, v_ctx: Tensor, scale: Optional[float] = None):
    """triton_kernels.py:549-567."""
    B, H, Lq, D = q.shape
    if scale is None:
        scale = D ** -0.5
    k_exp = k_ctx.unsqueeze(0).expand(B, -1, -1, -1)
    v_exp = v_ctx.unsqueeze(0).expand(B, -1, -1, -1)
    scores = torch.matmul(q, k_exp.transpose(-2, -1)) * scale
    lse = torch.logsumexp(scores.float(), dim=-1)
    attn = torch.softmax(scores, dim=-1)
    return torch.matmul(attn, v_exp), lse


def pytorch_buffer_attention(q: Tensor, k_buf: Tensor, v_buf: Tensor, mask: Optional[Tensor] = None,
                             scale: Optional[float] = None):
    """triton_kernels.py:589-614."""
    D = q.shape[-1]
    if scale is None:
        scale = D ** -0.5
    scores = torch.matmul(q, k_buf.transpose(-2, -1)) * scale
    no_kv = None
    if mask is not None:
        scores = scores.masked_fill(~mask, float("-inf"))
        no_kv = ~mask.any(dim=-1)
    lse = torch.logsumexp(scores.float(), dim=-1)
    attn = torch.softmax(scores, dim=-1)
    if no_kv is not None:
        attn = torch.where(no_kv.unsqueeze(-1), torch.zeros_like(attn), attn)
    return torch.matmul(attn, v_buf), lse


def teacher_forcing_buffer_mask(num_targets: int) -> Tensor:
    """triton_kernels.py:627-636: ``[1,1,2Nt,Nt]``, True = attend."""
    q_idx = torch.arange(2 * num_targets)
    kv_idx = torch.arange(num_targets)
    is_buffer = q_idx < num_targets
    buffer_mask = kv_idx[None, :] <= q_idx[:, None]
    target_mask = kv_idx[None, :] < (q_idx - num_targets)[:, None]
    return torch.where(is_buffer[:, None], buffer_mask, target_mask).unsqueeze(0).unsqueeze(0)


def hybrid_attention(q, k_ctx, v_ctx, k_buf, v_buf, buf_mask=None) -> Tensor:
    """triton_kernels.py:734-755 on the branch without a device kernel."""
    if k_buf.shape[2] == 0:
        return pytorch_context_attention(q, k_ctx, v_ctx)[0]
    out_ctx, lse_ctx = pytorch_context_attention(q, k_ctx, v_ctx)
    out_buf, lse_buf = pytorch_buffer_attention(q, k_buf, v_buf, mask=buf_mask)
    return merge_attention_outputs(out_ctx, lse_ctx, out_buf, lse_buf)


def hybrid_teacher_forcing_attention(q, k_ctx, v_ctx, k_buf, v_buf, num_targets: int) -> Tensor:
    """triton_kernels.py:684-702 (+ the shape checks of :653-656)."""
    if k_buf.shape[2] == 0:
        return pytorch_context_attention(q, k_ctx, v_ctx)[0]
    if q.shape[2] != 2 * num_targets:
        raise ValueError("Expected 2*num_targets queries for teacher forcing.")
    if k_buf.shape[2] != num_targets:
        raise ValueError("Expected buffer length to match num_targets.")
    out_ctx, lse_ctx = pytorch_context_attention(q, k_ctx, v_ctx)
    out_buf, lse_buf = pytorch_buffer_attention(q, k_buf, v_buf, mask=teacher_forcing_buffer_mask(num_targets))
    return merge_attention_outputs(out_ctx, lse_ctx, out_buf, lse_buf)


def masked_dense_attention(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor] = None) -> Tensor:
    """What ``flex_attention(q, k, v, block_mask=...)`` computes on a host (attention.py:57,
    inference.py:622, :735): scores in float32 at scale Dh^-0.5, boolean mask (True = attend),
    softmax, product with V, result in the input dtype."""
    scale = q.shape[-1] ** -0.5
    scores = torch.matmul(q.float(), k.float().transpose(-2, -1)) * scale
    if mask is not None:
        scores = scores.masked_fill(~mask, float("-inf"))
    return torch.matmul(torch.softmax(scores, dim=-1), v.float()).to(q.dtype)


def teacher_forcing_mask(num_cached: int, num_targets: int) -> Tensor:
    """inference.py:543-568 as a dense ``[2Nt, num_cached + 2Nt]`` boolean matrix."""
    Nt = num_targets
    q_idx = torch.arange(2 * Nt)[:, None]
    kv_idx = torch.arange(num_cached + 2 * Nt)[None, :]
    attends_context = kv_idx < num_cached
    kv_is_buffer = (kv_idx >= num_cached) & (kv_idx < num_cached + Nt)
    buffer_kv_idx = kv_idx - num_cached
    buffer_causal = kv_is_buffer & (buffer_kv_idx <= q_idx)
    target_to_buffer = kv_is_buffer & (buffer_kv_idx < q_idx - Nt)
    return attends_context | ((q_idx < Nt) & buffer_causal) | ((q_idx >= Nt) & target_to_buffer)


# ---------------------------------------------------------------------------------------------
# model pieces (model.py:23-272, attention.py:31-61)
# ---------------------------------------------------------------------------------------------

class TorchCpuModel:
    """The reference's modules applied functionally to a ``state_dict`` on the CPU."""

    def __init__(self, state_dict: Dict[str, Tensor], n_heads: int, dtype: torch.dtype = torch.float32):
        self.sd = {k: v.detach().to("cpu", dtype) for k, v in state_dict.items()}
        self.dtype = dtype
        self.n_heads = n_heads
        self.d_model = self.sd["embedder.marker_embed.weight"].shape[1]
        self.head_dim = self.d_model // n_heads
        self.n_layers = 1 + max(int(k.split(".")[2]) for k in self.sd if k.startswith("backbone.layers."))
        self.ar_tokens = self.sd["ar_tokens"]
        self.num_components = self.sd["head.mean_bias"].shape[0]

    def _p(self, i: int, name: str) -> Tensor:
        return self.sd[f"backbone.layers.{i}.{name}"]

    # embedder (model.py:51-76)
    def _embed(self, x: Tensor, y: Optional[Tensor], marker: str) -> Tensor:
        x_emb = F.linear(x.unsqueeze(-1), self.sd["embedder.x_embed.weight"], self.sd["embedder.x_embed.bias"])
        emb = x_emb.mean(dim=2)
        if y is not None:
            if y.dim() == 2:
                y = y.unsqueeze(-1)
            emb = emb + F.linear(y.unsqueeze(-1), self.sd["embedder.y_embed.weight"], self.sd["embedder.y_embed.bias"]).squeeze(2)
        return emb + self.sd["embedder.marker_embed.weight"][MARKER[marker]]

    def embed_context(self, x, y):
        return self._embed(x, y, "context")

    def embed_buffer(self, x, y):
        return self._embed(x, y, "buffer")

    def embed_target(self, x):
        return self._embed(x, None, "target")

    def _norm(self, x: Tensor, prefix: str) -> Tensor:
        return F.layer_norm(x, (self.d_model,), self.sd[prefix + ".weight"], self.sd[prefix + ".bias"])

    def _heads(self, t: Tensor) -> Tensor:
        B, N, _ = t.shape
        return t.view(B, N, self.n_heads, self.head_dim).transpose(1, 2)

    def feature_stage(self, i: int, x: Tensor) -> Tensor:
        """Feature attention over the single column + norm1 (inference.py:770-773 through
        attention.py:45-61): all four projections and a softmax over one key, as the reference
        computes them."""
        B, N, D = x.shape
        x_feat = x.reshape(B * N, 1, D)
        qh = self._heads(F.linear(x_feat, self._p(i, "attn_features.q_proj.weight")))
        kh = self._heads(F.linear(x_feat, self._p(i, "attn_features.k_proj.weight")))
        vh = self._heads(F.linear(x_feat, self._p(i, "attn_features.v_proj.weight")))
        out = masked_dense_attention(qh, kh, vh).transpose(1, 2).reshape(B * N, 1, D)
        attn_out = F.linear(out, self._p(i, "attn_features.out_proj.weight"))
        return self._norm((attn_out + x_feat).reshape(B, N, D), f"backbone.layers.{i}.norm1")

    def qkv(self, i: int, x_row: Tensor):
        return tuple(self._heads(F.linear(x_row, self._p(i, f"attn_rows.{n}.weight"))) for n in ("q_proj", "k_proj", "v_proj"))

    def post_attention(self, i: int, x_row: Tensor, attn_out: Tensor) -> Tensor:
        """inference.py:825-831."""
        B, H, N, Dh = attn_out.shape
        a = F.linear(attn_out.transpose(1, 2).reshape(B, N, H * Dh), self._p(i, "attn_rows.out_proj.weight"))
        x_row = self._norm(x_row + a, f"backbone.layers.{i}.norm2")
        h = F.gelu(F.linear(x_row, self._p(i, "ff.0.weight"), self._p(i, "ff.0.bias")))
        h = F.linear(h, self._p(i, "ff.2.weight"), self._p(i, "ff.2.bias"))
        return self._norm(x_row + h, f"backbone.layers.{i}.norm3")

    def final_norm(self, x: Tensor) -> Tensor:
        return self._norm(x, "backbone.norm")

    # mixture head (model.py:190-272)
    def head_parameterize(self, z: Tensor):
        B, T, _ = z.shape
        K = self.num_components
        h = F.gelu(F.linear(z, self.sd["head.head.0.weight"], self.sd["head.head.0.bias"]))
        raw = F.linear(h, self.sd["head.head.2.weight"], self.sd["head.head.2.bias"]).view(B, T, K, 1, 3)
        raw_mean, raw_std, raw_weight = raw.unbind(dim=-1)
        mean = raw_mean + self.sd["head.mean_bias"][None, None, :, None]
        std = F.softplus(raw_std + self.sd["head.std_bias"][None, None, :, None]).clamp(max=2.0) + 1e-3
        log_weight = F.log_softmax(raw_weight + self.sd["head.weight_bias"][None, None, :, None], dim=2)
        return mean, std, log_weight.exp(), log_weight

    def head_log_likelihood(self, z: Tensor, y: Tensor) -> Tensor:
        import math

        mean, std, _, log_weight = self.head_parameterize(z)
        y = y.unsqueeze(-1).unsqueeze(2)
        log_prob = -0.5 * (math.log(2 * math.pi) + 2 * std.log() + ((y - mean) / std) ** 2) + log_weight
        return torch.logsumexp(log_prob, dim=2).sum(dim=-1)

    def head_sample(self, z: Tensor) -> Tensor:
        """model.py:251-266 with one sample."""
        mean, std, weight, _ = self.head_parameterize(z)
        B, T, K, D = mean.shape
        weight_flat = weight.permute(0, 1, 3, 2).reshape(B * T * D, K)
        indices = torch.multinomial(weight_flat.float(), 1, replacement=True)
        sel_mean = torch.gather(mean.permute(0, 1, 3, 2).reshape(B * T * D, K), 1, indices).view(B, T, D, 1)
        sel_std = torch.gather(std.permute(0, 1, 3, 2).reshape(B * T * D, K), 1, indices).view(B, T, D, 1)
        return (sel_mean + sel_std * torch.randn_like(sel_mean)).permute(0, 1, 3, 2)


# ---------------------------------------------------------------------------------------------
# predictor (inference.py:82-488, :746-890)
# ---------------------------------------------------------------------------------------------

class TorchCpuPredictor:
    """``ARTabPFNPredictor`` on the shared-context backend (``backend="shared"``) or on the
    per-dataset full cache (``backend="per_dataset"``), restated over ``TorchCpuModel``."""

    def __init__(self, model: TorchCpuModel, backend: str = "shared"):
        if backend not in ("shared", "per_dataset"):
            raise ValueError(f"Unsupported backend: {backend}")
        self.m = model
        self.backend = backend
        self.context_len = self.buffer_len = self.max_buffer_len = self.seq_len = 0
        self.k_ctx: List[Tensor] = []
        self.v_ctx: List[Tensor] = []
        self.k_buf: List[Tensor] = []
        self.v_buf: List[Tensor] = []
        self.k_cache: List[Tensor] = []
        self.v_cache: List[Tensor] = []

    def init_kv_cache(self, batch_size: int, max_seq_len: int, context_len: int = 0):
        """inference.py:82-135: zero-filled caches (shared: context ``[H,Nc,Dh]`` + buffer
        ``[B,H,max_buf,Dh]``; per-dataset: ``[B,H,max_seq,Dh]``)."""
        m = self.m
        L, H, Dh = m.n_layers, m.n_heads, m.head_dim
        if self.backend == "shared":
            self.k_ctx = [torch.zeros(H, context_len, Dh, dtype=m.dtype) for _ in range(L)]
            self.v_ctx = [torch.zeros(H, context_len, Dh, dtype=m.dtype) for _ in range(L)]
            self.k_buf = [torch.zeros(batch_size, H, max_seq_len, Dh, dtype=m.dtype) for _ in range(L)]
            self.v_buf = [torch.zeros(batch_size, H, max_seq_len, Dh, dtype=m.dtype) for _ in range(L)]
            self.max_buffer_len = max_seq_len
        else:
            self.k_cache = [torch.zeros(batch_size, H, max_seq_len, Dh, dtype=m.dtype) for _ in range(L)]
            self.v_cache = [torch.zeros(batch_size, H, max_seq_len, Dh, dtype=m.dtype) for _ in range(L)]
        self.context_len = self.buffer_len = self.seq_len = 0

    def prefill_context(self, x_context: Tensor, y_context: Tensor) -> None:
        """inference.py:143-223, :579-685."""
        m = self.m
        if self.backend == "shared":
            x_context, y_context = x_context[0:1], y_context[0:1]  # :191-193
        x = m.embed_context(x_context, y_context)
        Nc = x.shape[1]
        for i in range(m.n_layers):
            x_row = m.feature_stage(i, x)
            q, k, v = m.qkv(i, x_row)
            if self.backend == "shared":
                if self.k_ctx[i].shape[1] != Nc:
                    self.k_ctx[i] = torch.zeros(m.n_heads, Nc, m.head_dim, dtype=m.dtype)
                    self.v_ctx[i] = torch.zeros(m.n_heads, Nc, m.head_dim, dtype=m.dtype)
                self.k_ctx[i][:, 0:Nc, :] = k[0]
                self.v_ctx[i][:, 0:Nc, :] = v[0]
            else:
                self.k_cache[i][:, :, 0:Nc, :] = k
                self.v_cache[i][:, :, 0:Nc, :] = v
            x = m.post_attention(i, x_row, masked_dense_attention(q, k, v))
        self.context_len = self.seq_len = Nc
        self.buffer_len = 0

    def _layer_decode_shared(self, i: int, x: Tensor) -> Tensor:
        """inference.py:746-833."""
        m = self.m
        B, N, D = x.shape
        if N not in (1, 2):
            raise ValueError("Shared-context decode only supports N=1 (target) or N=2 (buffer, target).")
        x_row = m.feature_stage(i, x)
        q, k_new, v_new = m.qkv(i, x_row)
        k_ctx, v_ctx = self.k_ctx[i][:, : self.context_len], self.v_ctx[i][:, : self.context_len]
        k_buf, v_buf = self.k_buf[i][:, :, : self.buffer_len], self.v_buf[i][:, :, : self.buffer_len]
        if N == 1:
            attn_out = hybrid_attention(q[:, :, 0:1], k_ctx, v_ctx, k_buf, v_buf)
        else:
            k_new_buf, v_new_buf = k_new[:, :, 0:1], v_new[:, :, 0:1]
            if self.buffer_len == 0:
                k_all, v_all = k_new_buf, v_new_buf
            else:
                k_all = torch.cat([k_buf, k_new_buf], dim=2)
                v_all = torch.cat([v_buf, v_new_buf], dim=2)
            out_buf = hybrid_attention(q[:, :, 0:1], k_ctx, v_ctx, k_all, v_all)
            out_tgt = hybrid_attention(q[:, :, 1:2], k_ctx, v_ctx, k_all, v_all)
            self.k_buf[i][:, :, self.buffer_len : self.buffer_len + 1] = k_new_buf
            self.v_buf[i][:, :, self.buffer_len : self.buffer_len + 1] = v_new_buf
            attn_out = torch.cat([out_buf, out_tgt], dim=2)
        return m.post_attention(i, x_row, attn_out)

    def transformer_decode(self, embedding: Tensor, commit: int) -> Tensor:
        """inference.py:225-260 (shared backend)."""
        if self.backend != "shared":
            raise ValueError("step-wise decode is restated for the shared-context backend only")
        if self.buffer_len + commit > self.max_buffer_len:
            raise ValueError("Shared-context buffer cache exceeded; increase max buffer length.")
        x = embedding
        for i in range(self.m.n_layers):
            x = self._layer_decode_shared(i, x)
        self.buffer_len += commit
        self.seq_len = self.context_len + self.buffer_len
        return self.m.final_norm(x)

    def autoregressive_decode(self, x_target, prev_x=None, prev_y=None, ar_idx: int = 0) -> Tensor:
        """inference.py:278-320."""
        target_emb = self.m.embed_target(x_target)
        if prev_x is not None and prev_y is not None:
            buffer_emb = self.m.embed_buffer(prev_x, prev_y) + self.m.ar_tokens[ar_idx]
            embedding, commit = torch.cat([buffer_emb, target_emb], dim=1), 1
        else:
            embedding, commit = target_emb, 0
        z = self.transformer_decode(embedding, commit)
        return self.m.head_sample(z[:, -1:, :])[:, :, 0, 0]

    def teacher_forcing_decode(self, embedding: Tensor, num_targets: int) -> Tensor:
        """Shared: inference.py:473-488 + :835-890.  Per-dataset: :455-471 + :687-744 (the new
        rows' K/V written behind the context, attention over the whole cache under the mask)."""
        m = self.m
        B, N, D = embedding.shape
        if N != 2 * num_targets:
            raise ValueError("Expected N == 2*num_targets for teacher forcing.")
        x = embedding
        mask = None if self.backend == "shared" else teacher_forcing_mask(self.seq_len, num_targets)
        for i in range(m.n_layers):
            x_row = m.feature_stage(i, x)
            q, k, v = m.qkv(i, x_row)
            if self.backend == "shared":
                attn = hybrid_teacher_forcing_attention(
                    q, self.k_ctx[i][:, : self.context_len], self.v_ctx[i][:, : self.context_len],
                    k[:, :, :num_targets], v[:, :, :num_targets], num_targets)
            else:
                s = self.seq_len
                self.k_cache[i][:, :, s : s + N] = k
                self.v_cache[i][:, :, s : s + N] = v
                attn = masked_dense_attention(q, self.k_cache[i][:, :, : s + N], self.v_cache[i][:, :, : s + N], mask)
            x = m.post_attention(i, x_row, attn)
        return m.final_norm(x)

    def evaluate_joint_density(self, x_context, y_context, x_target, y_target) -> Tensor:
        """inference.py:391-453."""
        m = self.m
        B, Nc, _ = x_context.shape
        Nt = x_target.shape[1]
        if self.backend == "shared":
            self.init_kv_cache(B, Nt, context_len=Nc)
        else:
            self.init_kv_cache(B, Nc + 2 * Nt)
        self.prefill_context(x_context, y_context)
        buffer_emb = m.embed_buffer(x_target, y_target) + m.ar_tokens[torch.arange(Nt) % m.ar_tokens.shape[0]]
        embedding = torch.cat([buffer_emb, m.embed_target(x_target)], dim=1)
        z = self.teacher_forcing_decode(embedding, Nt)
        return m.head_log_likelihood(z[:, Nt:, :], y_target)
