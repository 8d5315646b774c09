"""AR-TabPFN modules (host-side mirror of the reference's ``ar_tabpfn/model/model.py``).

Plain PyTorch-ROCm around the HIP attention kernels.  Module names, parameter
shapes, construction order (hence seeded initialisation) and ``state_dict`` keys
follow the reference so checkpoints interchange: ``embedder.{x_embed,y_embed}``,
``embedder.marker_embed``, ``backbone.layers.{i}.{attn_features,attn_rows}.*_proj``,
``backbone.layers.{i}.ff.{0,2}``, ``backbone.layers.{i}.norm{1,2,3}``,
``backbone.norm``, ``head.head.{0,2}``, ``head.{mean_bias,std_bias,weight_bias}``,
``ar_tokens`` (model.py:33-37, :89-98, :138, :172-184, :315).

``ARTabPFN.forward`` is the training objective (model.py:317-369): with gradients being
recorded the layers run as plain differentiable PyTorch around the device row attention and its
device backward pass; without, through the fused inference kernels.  Inference goes through
``ARTabPFNPredictor``.
"""

from __future__ import annotations

import math
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from .attention import DenseMask, MultiheadAttention, RowMask
from .glue import add_layer_norm, bias_gelu, layer_fusable, layer_post, layer_post_pre, layer_pre, pack_weight

__all__ = ["Embedder", "TwoStageTransformerLayer", "TwoStageTransformer", "MixtureGaussianHead", "ARTabPFN"]

_MARKERS = {"target": 0, "context": 1, "buffer": 2}  # model.py:36-38


class Embedder(nn.Module):
    """Scalar-wise feature embedding averaged over features, plus the y embedding and a
    learned marker per row kind (model.py:23-76)."""

    def __init__(self, d_model: int):
        super().__init__()
        self.x_embed = nn.Linear(1, d_model)
        self.y_embed = nn.Linear(1, d_model)
        self.marker_embed = nn.Embedding(3, d_model)

    def _x(self, x: Tensor) -> Tensor:
        # mean_c(x_c * w + b) == mean_c(x_c) * w + b: one [B,N,D] result instead of [B,N,C,D]
        return self.x_embed(x.mean(dim=-1, keepdim=True))

    def _y(self, y: Tensor) -> Tensor:
        return self.y_embed(y.unsqueeze(-1) if y.dim() == 2 else y)

    def _marker(self, kind: str) -> Tensor:
        return self.marker_embed.weight[_MARKERS[kind]]

    def embed_context(self, x: Tensor, y: Tensor) -> Tensor:
        """x ``[B,N,C]``, y ``[B,N]`` or ``[B,N,1]`` -> ``[B,N,D]``."""
        return self._x(x) + self._y(y) + self._marker("context")

    def embed_buffer(self, x: Tensor, y: Tensor) -> Tensor:
        """Buffer rows; the AR position token is added by the caller."""
        return self._x(x) + self._y(y) + self._marker("buffer")

    def embed_target(self, x: Tensor) -> Tensor:
        return self._x(x) + self._marker("target")


class TwoStageTransformerLayer(nn.Module):
    """Feature attention over columns, row attention, feed-forward; post-norm
    (model.py:79-126)."""

    def __init__(self, d_model: int, n_heads: int, d_ff: int):
        super().__init__()
        self.attn_features = MultiheadAttention(d_model, n_heads)
        self.attn_rows = MultiheadAttention(d_model, n_heads)
        self.ff = nn.Sequential(nn.Linear(d_model, d_ff), nn.GELU(), nn.Linear(d_ff, d_model))
        self.norm1 = nn.LayerNorm(d_model)
        self.norm2 = nn.LayerNorm(d_model)
        self.norm3 = nn.LayerNorm(d_model)

    def fused_weights(self):
        """Weights of the fused inference GEMMs, rebuilt when a source weight changes.

        * ``w_fo = out_proj.weight @ v_proj.weight`` of the feature attention: with a
          single column the block is ``out_proj(v_proj(x))`` — one matrix (product taken
          in float32, stored in the model dtype);
        * ``w_qkv``: the three row-attention projections stacked, so q, k, v come out of
          one GEMM as strided views of one ``[..., 3D]`` tensor.
        """
        af, ar = self.attn_features, self.attn_rows
        srcs = (af.v_proj.weight, af.out_proj.weight, ar.q_proj.weight, ar.k_proj.weight, ar.v_proj.weight)
        key = tuple((p.data_ptr(), p._version, p.dtype, p.device) for p in srcs)
        cached = getattr(self, "_fused_cache", None)
        if cached is None or cached[0] != key:
            with torch.no_grad():
                w_fo = (af.out_proj.weight.float() @ af.v_proj.weight.float()).to(af.v_proj.weight.dtype)
                w_qkv = torch.cat([ar.q_proj.weight, ar.k_proj.weight, ar.v_proj.weight], dim=0).contiguous()
            cached = (key, w_fo, w_qkv)
            self._fused_cache = cached
        return cached[1], cached[2]

    def feature_stage(self, x_row: Tensor) -> Tensor:
        """Feature attention for the single-column case (C = 1) followed by norm1.

        One key per query: the softmax weight is exactly 1, so the attention output is
        ``out_proj(v_proj(x))`` and the q/k projections do not enter
        (attention.py:52-61 with S = 1; inference.py:771-773).  One GEMM, then residual and
        norm1 in one fused pass."""
        w_fo, _ = self.fused_weights()
        x2d = x_row.reshape(-1, x_row.shape[-1])
        return add_layer_norm(x_row, torch.mm(x2d, w_fo.t()).view_as(x_row), None, self.norm1)

    def qkv_heads(self, x_row: Tensor):
        """q, k, v of the row attention as ``[B,H,N,Dh]`` strided views of one GEMM output."""
        _, w_qkv = self.fused_weights()
        B, N, D = x_row.shape
        a = self.attn_rows
        qkv = F.linear(x_row, w_qkv).view(B, N, 3, a.n_heads, a.head_dim)
        return qkv[:, :, 0].transpose(1, 2), qkv[:, :, 1].transpose(1, 2), qkv[:, :, 2].transpose(1, 2)

    def packed_weights(self):
        """The five matrices of the layer in the operand order of the fused kernels
        (``pack_weight``), rebuilt when a source weight changes:
        ``(w_fo, w_qkv, out_proj, ff[0], ff[2])``."""
        w_fo, w_qkv = self.fused_weights()
        srcs = (w_fo, w_qkv, self.attn_rows.out_proj.weight, self.ff[0].weight, self.ff[2].weight)
        key = tuple((p.data_ptr(), p._version, p.dtype, p.device) for p in srcs)
        cached = getattr(self, "_packed_cache", None)
        if cached is None or cached[0] != key:
            cached = (key, tuple(pack_weight(p) for p in srcs))
            self._packed_cache = cached
        return cached[1]

    def _fusable(self, x_row: Tensor) -> bool:
        return layer_fusable(x_row, x_row.shape[-1], self.ff[0].out_features)

    def fused_for(self, t: Tensor) -> bool:
        """Whether tensors of ``t``'s dtype and device go through this layer's fused kernels."""
        return layer_fusable(t, self.norm1.normalized_shape[0], self.ff[0].out_features)

    def pre_attention(self, x_row: Tensor):
        """Everything before the row-attention call: ``(y, q, k, v)`` with ``y`` the normed
        feature stage ``[B,N,D]`` and q, k, v ``[B,H,N,Dh]`` views of one ``[B,N,3D]`` tensor.
        One launch where the fused kernel covers the layer, otherwise two GEMMs and norm1."""
        if not self._fusable(x_row):
            y = self.feature_stage(x_row)
            return (y,) + tuple(self.qkv_heads(y))
        p_fo, p_qkv = self.packed_weights()[:2]
        B, N, D = x_row.shape
        a = self.attn_rows
        y, qkv = layer_pre(x_row, p_fo, self.norm1, p_qkv)
        qkv = qkv.view(B, N, 3, a.n_heads, a.head_dim)
        return (y.view(B, N, D), qkv[:, :, 0].transpose(1, 2), qkv[:, :, 1].transpose(1, 2),
                qkv[:, :, 2].transpose(1, 2))

    def finish(self, x_row: Tensor, attn_heads: Tensor) -> Tensor:
        """``out_proj`` on ``[B,H,N,Dh]`` attention output, then norm2 / FFN / norm3
        (inference.py:825-831); one launch where the fused kernel covers the layer."""
        B, H, N, Dh = attn_heads.shape
        D = H * Dh
        # unmerged partials (attention_kernels.AttentionPartials) go to the kernel as they are
        attn2d = attn_heads if hasattr(attn_heads, "desc") else attn_heads.transpose(1, 2).reshape(B * N, D)
        if self._fusable(x_row):
            p_o, p_1, p_2 = self.packed_weights()[2:]
            return layer_post(attn2d, x_row, p_o, self.norm2, p_1, self.ff[0].bias, p_2, self.ff[2].bias,
                              self.norm3).view(B, N, D)
        if hasattr(attn_heads, "desc"):
            raise ValueError("attention partials need a layer the fused kernels cover")
        x_row = add_layer_norm(x_row, torch.mm(attn2d, self.attn_rows.out_proj.weight.t()).view(B, N, D), None, self.norm2)
        return self.feed_forward(x_row)

    def finish_then_pre(self, x_row: Tensor, attn_heads: Tensor, next_layer: "TwoStageTransformerLayer"):
        """``next_layer.pre_attention(self.finish(x_row, attn_heads))``: ``(y, q, k, v)`` of the
        next layer.  One launch when both layers are covered by the fused kernels and have the
        same widths; the layer output between them is then never written to memory."""
        same = (next_layer.ff[0].out_features == self.ff[0].out_features
                and next_layer.attn_rows.n_heads == self.attn_rows.n_heads)
        if not (same and self._fusable(x_row) and next_layer._fusable(x_row)):
            return next_layer.pre_attention(self.finish(x_row, attn_heads))
        B, H, N, Dh = attn_heads.shape
        D = H * Dh
        attn2d = attn_heads if hasattr(attn_heads, "desc") else attn_heads.transpose(1, 2).reshape(B * N, D)
        p_o, p_1, p_2 = self.packed_weights()[2:]
        n_fo, n_qkv = next_layer.packed_weights()[:2]
        y, qkv = layer_post_pre(attn2d, x_row, p_o, self.norm2, p_1, self.ff[0].bias, p_2, self.ff[2].bias,
                                self.norm3, n_fo, next_layer.norm1, n_qkv)
        qkv = qkv.view(B, N, 3, H, Dh)
        return (y.view(B, N, D), qkv[:, :, 0].transpose(1, 2), qkv[:, :, 1].transpose(1, 2),
                qkv[:, :, 2].transpose(1, 2))

    def feed_forward(self, x_row: Tensor) -> Tensor:
        """``norm3(x + ff(x))`` with bias+GELU and bias+residual+norm fused around the two GEMMs."""
        lin1, lin2 = self.ff[0], self.ff[2]
        x2d = x_row.reshape(-1, x_row.shape[-1])
        h = bias_gelu(torch.mm(x2d, lin1.weight.t()), lin1.bias)
        return add_layer_norm(x_row, torch.mm(h, lin2.weight.t()).view_as(x_row), lin2.bias, self.norm3)

    def _forward_recording(self, x_row: Tensor, mask_rows) -> Tuple[Tensor, Tuple[Tensor, Tensor]]:
        """The layer on ``[B,R,D]`` rows as differentiable PyTorch modules around the device row
        attention (model.py:100-126 with C = 1): what a training step records."""
        af = self.attn_features
        # one key per query: the softmax weight is exactly 1 and the attention output is
        # out_proj(v_proj(x)); q_proj and k_proj get the exact zero gradients autograd gives them
        # in the reference (their parameters stay in the optimiser's bookkeeping)
        feat = af.out_proj(af.v_proj(x_row)) + 0.0 * (af.q_proj.weight.sum() + af.k_proj.weight.sum())
        x_row = self.norm1(feat + x_row)
        attn, kv = self.attn_rows(x_row, x_row, x_row, mask_rows)
        x_row = self.norm2(attn + x_row)
        return self.norm3(x_row + self.ff(x_row)), kv

    def forward(self, x: Tensor, mask_features, mask_rows) -> Tuple[Tensor, Tuple[Tensor, Tensor]]:
        """``[B,R,C,D]`` under a dense mask (the bidirectional context pass, inference only) or the
        training row mask.  Under the row mask, while gradients are recorded, the layer runs as
        differentiable modules."""
        B, R, C, D = x.shape
        if C != 1:
            raise NotImplementedError("only the single-column layout (C = 1) is used by this model")
        if (isinstance(mask_rows, RowMask) and torch.is_grad_enabled()
                and (x.requires_grad or any(p.requires_grad for p in self.parameters()))):
            out, kv = self._forward_recording(x.squeeze(2), mask_rows)
            return out.unsqueeze(2), kv
        x_row = self.feature_stage(x.squeeze(2))
        attn, kv = self.attn_rows(x_row, x_row, x_row, mask_rows)
        x_row = add_layer_norm(x_row, attn, None, self.norm2)
        return self.feed_forward(x_row).unsqueeze(2), kv


class TwoStageTransformer(nn.Module):
    def __init__(self, d_model: int, n_heads: int, n_layers: int, d_ff: int):
        super().__init__()
        self.d_model = d_model
        self.layers = nn.ModuleList([TwoStageTransformerLayer(d_model, n_heads, d_ff) for _ in range(n_layers)])
        self.norm = nn.LayerNorm(d_model)

    def forward(self, x: Tensor, mask_features: DenseMask, mask_rows: DenseMask) -> Tuple[Tensor, List[Tuple[Tensor, Tensor]]]:
        kvs = []
        for layer in self.layers:
            x, kv = layer(x, mask_features, mask_rows)
            kvs.append(kv)
        if torch.is_grad_enabled() and x.requires_grad:
            return self.norm(x), kvs
        return add_layer_norm(x, None, None, self.norm), kvs


class MixtureGaussianHead(nn.Module):
    """Mixture-of-Gaussians regression head (model.py:150-272)."""

    def __init__(self, d_model: int, d_ff: int, dim_y: int = 1, num_components: int = 5, std_min: float = 1e-3):
        super().__init__()
        self.dim_y = dim_y
        self.num_components = num_components
        self.std_min = std_min
        self.head = nn.Sequential(nn.Linear(d_model, d_ff), nn.GELU(), nn.Linear(d_ff, num_components * dim_y * 3))
        self.mean_bias = nn.Parameter(torch.linspace(-1.0, 1.0, num_components))
        delta = 1.0 / (num_components - 1)
        self.std_bias = nn.Parameter(torch.full((num_components,), math.log(math.expm1(delta))))
        self.weight_bias = nn.Parameter(torch.zeros(num_components))

    def _parameterize(self, z: Tensor) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
        """``[B,T,D] -> mean, std, weight, log_weight`` each ``[B,T,K,dim_y]``; the raw
        output is laid out ``(K, dim_y, 3)`` (model.py:195-196)."""
        B, T, _ = z.shape
        raw = self.head(z).view(B, T, self.num_components, self.dim_y, 3)
        bias = lambda p: p.view(1, 1, -1, 1)  # noqa: E731
        mean = raw[..., 0] + bias(self.mean_bias)
        std = F.softplus(raw[..., 1] + bias(self.std_bias)).clamp(max=2.0) + self.std_min
        log_weight = F.log_softmax(raw[..., 2] + bias(self.weight_bias), dim=2)
        return mean, std, log_weight.exp(), log_weight

    @staticmethod
    def _log_likelihood(y: Tensor, mean: Tensor, std: Tensor, log_weight: Tensor) -> Tensor:
        z = (y.unsqueeze(2) - mean) / std
        comp = -0.5 * (math.log(2 * math.pi) + z * z) - std.log() + log_weight
        return torch.logsumexp(comp, dim=2)

    def forward(self, z: Tensor, y: Optional[Tensor] = None, loss_mask: Optional[Tensor] = None):
        mean, std, weight, log_weight = self._parameterize(z)
        loss = None
        if y is not None:
            ll = self._log_likelihood(y, mean, std, log_weight)
            if loss_mask is not None:
                ll = ll.mean(-1) * loss_mask
                denom = loss_mask.sum().clamp(min=1)
            else:
                denom = ll.numel()
            loss = -ll.sum() / denom
        return loss, mean, std, weight

    def sample(self, z: Tensor, num_samples: int = 1) -> Tensor:
        """``[B,T,D] -> [B,T,num_samples,dim_y]``: pick a component per draw, then a normal."""
        mean, std, weight, _ = self._parameterize(z)
        B, T, K, Dy = mean.shape
        flat = lambda t: t.permute(0, 1, 3, 2).reshape(B * T * Dy, K)  # noqa: E731
        # Component = first k whose cumulative weight exceeds a uniform variate times the total
        # (the law of a multinomial draw, and the rule of the fused step tail).  The index is
        # clamped, so non-finite weights give non-finite samples instead of a device-side
        # index assertion.
        cdf = flat(weight).float().cumsum(dim=1)
        u = torch.rand((cdf.shape[0], num_samples), device=cdf.device, dtype=cdf.dtype) * cdf[:, -1:]
        idx = (u.unsqueeze(-1) >= cdf.unsqueeze(1)).sum(dim=-1).clamp_(max=K - 1)
        mu = torch.gather(flat(mean), 1, idx).view(B, T, Dy, num_samples)
        sd = torch.gather(flat(std), 1, idx).view(B, T, Dy, num_samples)
        return (mu + sd * torch.randn_like(mu)).permute(0, 1, 3, 2)

    def log_likelihood(self, z: Tensor, y: Tensor) -> Tensor:
        """``z [B,T,D]``, ``y [B,T,dim_y]`` -> ``[B,T]``."""
        mean, std, _, log_weight = self._parameterize(z)
        return self._log_likelihood(y, mean, std, log_weight).sum(dim=-1)


class ARTabPFN(nn.Module):
    """Container with the reference's constructor and attribute names (model.py:275-315)."""

    def __init__(self, d_model: int = 128, n_heads: int = 4, n_layers: int = 6, d_ff: int = 256,
                 num_features: int = 10, buffer_size: int = 8, num_components: int = 5):
        super().__init__()
        self.d_model = d_model
        self.num_features = num_features
        self.buffer_size = buffer_size
        self.embedder = Embedder(d_model)
        self.backbone = TwoStageTransformer(d_model, n_heads, n_layers, d_ff)
        self.head = MixtureGaussianHead(d_model, d_ff, dim_y=1, num_components=num_components)
        self.ar_tokens = nn.Parameter(torch.randn(buffer_size, d_model) * 0.02)

    def forward(self, x_context: Tensor, y_context: Tensor, x_buffer: Tensor, y_buffer: Tensor, x_target: Tensor,
                mask_features, mask_rows, y_target: Optional[Tensor] = None):
        """The training objective (model.py:317-369): context, buffer and target rows in one pass
        under the row mask of ``create_row_mask``; returns the mean negative log-likelihood of
        ``y_target`` (None without it).  The row attention runs on the device kernels in both
        directions: ``loss.backward()`` gives every parameter its gradient, as in the reference's
        training step (train.py:289-300).  Under ``torch.no_grad()`` the layers take the fused
        inference kernels instead."""
        ctx_emb = self.embedder.embed_context(x_context, y_context)
        buf_emb = self.embedder.embed_buffer(x_buffer, y_buffer) + self.ar_tokens[: x_buffer.size(1)]
        tgt_emb = self.embedder.embed_target(x_target)
        Nc, Nb = ctx_emb.size(1), buf_emb.size(1)
        embeddings = torch.cat([ctx_emb, buf_emb, tgt_emb], dim=1).unsqueeze(2)
        z, _ = self.backbone(embeddings, mask_features, mask_rows)
        z_target = z[:, Nc + Nb:, 0, :]
        if y_target is not None and y_target.dim() == 2:
            y_target = y_target.unsqueeze(-1)
        loss, _, _, _ = self.head(z_target, y_target)
        return loss

    # ---- checkpoints written by the reference's training loop (train.py:336-343): a dict
    # {"step": int, "model": state_dict}.  With `compile_model` the embedder and the head were
    # wrapped by torch.compile before the state_dict was taken (train.py:233-235), which puts an
    # "_orig_mod." segment into their keys.

    @staticmethod
    def clean_state_dict(state_dict):
        """The state_dict with every ``_orig_mod.`` path segment removed."""
        return {k.replace("_orig_mod.", ""): v for k, v in state_dict.items()}

    @classmethod
    def from_checkpoint(cls, checkpoint, n_heads: int, num_features: int = 10, map_location="cpu"):
        """Build the model a reference checkpoint was trained with and load it.

        ``checkpoint`` is a path (read with ``torch.load(..., weights_only=True)``), the loaded
        ``{"step", "model"}`` dict, or a bare state_dict.  Every size except the number of heads is
        read off the tensors.  Returns ``(model, step)``; ``step`` is None for a bare state_dict.
        """
        if not isinstance(checkpoint, dict):
            checkpoint = torch.load(checkpoint, map_location=map_location, weights_only=True)
        step = checkpoint.get("step") if "model" in checkpoint else None
        sd = cls.clean_state_dict(checkpoint["model"] if "model" in checkpoint else checkpoint)
        try:
            d_model = sd["embedder.x_embed.weight"].shape[0]
            d_ff = sd["backbone.layers.0.ff.0.weight"].shape[0]
            buffer_size = sd["ar_tokens"].shape[0]
            num_components = sd["head.mean_bias"].shape[0]
        except KeyError as err:
            raise ValueError(f"not an AR-TabPFN state_dict: missing {err}") from None
        n_layers = 1 + max(int(k.split(".")[2]) for k in sd if k.startswith("backbone.layers."))
        if d_model % n_heads:
            raise ValueError(f"d_model {d_model} is not divisible by n_heads {n_heads}")
        model = cls(d_model=d_model, n_heads=n_heads, n_layers=n_layers, d_ff=d_ff, num_features=num_features,
                    buffer_size=buffer_size, num_components=num_components)
        model.load_state_dict(sd, strict=True)
        return model, step
