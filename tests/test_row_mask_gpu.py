"""The training row mask as a tile schedule (``artab_row_mask_attention``), its backward pass
(``artab_row_mask_attention_backward``) and the training objective built on them, against the
oracle, a plain PyTorch statement and the loss the reference computed for the fixture
(attention.py:86-175, model.py:317-369, train.py:289-300)."""

import os

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from oracle import model_oracle as mo
from tests.helpers import max_abs, out_tol, randn, to_np

pytestmark = pytest.mark.gpu

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "tiny_model.npz")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize(
    "B,H,D,Nc,Nb,T,A",
    [
        (2, 2, 32, 7, 4, 16, None),      # the fixture's shape
        (3, 4, 32, 300, 8, 64, None),    # context longer than a query tile, four of eight chunks attend
        (2, 8, 32, 64, 32, 128, 4),      # every chunk attends
        (2, 8, 32, 64, 32, 128, 0),      # no target attends: buffer tiles are skipped for target rows
        (1, 2, 64, 100, 16, 96, None),   # head_dim 64
        (2, 2, 32, 1, 1, 2, None),       # the smallest legal problem
        (1, 4, 32, 513, 70, 280, 3),     # ragged everything: limits wrap inside a 32-row block
    ],
)
def test_row_mask_attention_matches_oracle(device, dtype, B, H, D, Nc, Nb, T, A):
    import ar_nanotabpfn_amd.attention_kernels as ak
    from ar_nanotabpfn_amd.attention import create_row_mask

    R = Nc + Nb + T
    q, k, v = (randn((B, H, R, D), s, dtype, 0.7) for s in (1, 2, 3))
    mask = create_row_mask(R, Nc, Nb, A, device=device)
    assert np.array_equal(mask.dense().numpy(), ao.row_mask(R, Nc, Nb, A))
    ref = ao.row_mask_attention(to_np(q), to_np(k), to_np(v), Nc, Nb, A)
    for use_mfma in (True, False):
        out = ak.row_mask_attention(q.to(device), k.to(device), v.to(device), Nc, Nb, mask.attending_chunks,
                                    use_triton=use_mfma)
        assert out.shape == (B, H, R, D)
        assert max_abs(to_np(out), ref) <= out_tol(dtype), f"use_mfma={use_mfma}"


def test_row_mask_attention_on_projection_views(device):
    """q, k, v as strided views of one [B,R,3,H,D] projection output, as the layer produces them."""
    import ar_nanotabpfn_amd.attention_kernels as ak

    B, H, D, Nc, Nb, T = 2, 4, 32, 130, 8, 48
    R = Nc + Nb + T
    qkv = randn((B, R, 3, H, D), 5, torch.bfloat16, 0.7).to(device)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
    out = ak.row_mask_attention(q, k, v, Nc, Nb, T // (2 * Nb))
    ref = ao.row_mask_attention(to_np(q), to_np(k), to_np(v), Nc, Nb)
    assert max_abs(to_np(out), ref) <= 2e-2


def test_row_mask_argument_errors(device):
    import ar_nanotabpfn_amd.attention_kernels as ak

    q = torch.zeros(1, 2, 10, 32, device=device, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ak.row_mask_attention(q, q, q, 0, 2, 1)      # no context
    with pytest.raises(ValueError):
        ak.row_mask_attention(q, q, q, 8, 4, 1)      # context + buffer exceed the rows
    with pytest.raises(ValueError):
        ak.row_mask_attention(q, q[:, :, :5], q, 4, 2, 1)


def test_training_forward_matches_reference_fixture(device):
    """The loss the reference computed (float32 model, CPU) through the device path."""
    from ar_nanotabpfn_amd.attention import create_dense_mask, create_row_mask
    from ar_nanotabpfn_amd.model import ARTabPFN

    data = np.load(FIXTURE, allow_pickle=False)
    sd = {k[3:]: torch.from_numpy(data[k]) for k in data.files if k.startswith("w::")}
    cfg = dict(zip(("d_model", "n_heads", "n_layers", "d_ff", "num_features", "buffer_size", "num_components"),
                   (int(v) for v in data["cfg"])))
    model = ARTabPFN(**cfg).eval()
    model.load_state_dict(sd, strict=True)
    model = model.to(device)
    t = lambda name: torch.from_numpy(data[name]).to(device)  # noqa: E731
    Nc, Nb, Nt = data["x_ctx"].shape[1], data["train_x_buf"].shape[1], data["train_x_tgt"].shape[1]
    feat = create_dense_mask(1, device=device)
    args = (t("x_ctx"), t("y_ctx"), t("train_x_buf"), t("train_y_buf"), t("train_x_tgt"))
    # once as a training step records it (differentiable modules around the device attention),
    # once under no_grad (the fused inference kernels)
    for recording in (True, False):
        with torch.set_grad_enabled(recording):
            loss = model(*args, feat, create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device), y_target=t("train_y_tgt"))
            loss3 = model(*args, feat, create_row_mask(Nc + Nb + Nt, Nc, Nb, attending_chunks=3, device=device),
                          y_target=t("train_y_tgt"))
            assert loss.requires_grad == recording
            assert abs(loss.item() - float(data["train_loss"])) <= 1e-4
            assert abs(loss3.item() - float(data["train_loss_attend3"])) <= 1e-4
            # no labels, no loss
            assert model(*args, feat, create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device)) is None


def test_training_forward_bf16_vs_oracle(device):
    """A bf16 model at a training-like shape (256 context, 32 buffer, 128 target rows): the loss
    against the float64 oracle on the same bf16 weights and inputs."""
    from ar_nanotabpfn_amd.attention import create_dense_mask, create_row_mask
    from ar_nanotabpfn_amd.model import ARTabPFN

    cfg = dict(d_model=128, n_heads=4, n_layers=3, d_ff=128, num_features=5, buffer_size=32, num_components=4)
    torch.manual_seed(0)
    model = ARTabPFN(**cfg).eval().to(device=device, dtype=torch.bfloat16)
    B, Nc, Nb, Nt = 4, 256, 32, 128
    g = torch.Generator().manual_seed(1)
    mk = lambda *s: torch.randn(*s, generator=g).to(device, torch.bfloat16)  # noqa: E731
    xc, yc, xb, yb, xt, yt = mk(B, Nc, 5), mk(B, Nc), mk(B, Nb, 5), mk(B, Nb), mk(B, Nt, 5), mk(B, Nt)
    loss = model(xc, yc, xb, yb, xt, create_dense_mask(1, device=device),
                 create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device), y_target=yt)
    sd = {k: v.detach().float().cpu().numpy() for k, v in model.state_dict().items()}
    ref, _ = mo.training_forward(mo.OracleModel(sd, cfg["n_heads"]), *(to_np(a) for a in (xc, yc, xb, yb, xt, yt)))
    print(f"\n[training forward bf16] loss {loss.item():.5f} vs exact {ref:.5f}")
    assert abs(loss.item() - ref) <= 2e-2


# ----------------------------------------------------------------------------- backward pass

def _grad_err(got, ref):
    """Largest deviation relative to the gradient's own scale (at least 1)."""
    return max_abs(to_np(got), ref) / max(1.0, float(np.abs(ref).max()))


def _grad_tol(dtype):
    # float32 arithmetic on float32 inputs; for 16-bit inputs P, dS, the saved output and the
    # results themselves are rounded to the input type (2^-9 relative for bf16)
    return 2e-5 if dtype == torch.float32 else 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize(
    "B,H,D,Nc,Nb,T,A",
    [
        (2, 2, 32, 7, 4, 16, None),      # the fixture's shape
        (3, 4, 32, 300, 8, 64, None),    # context longer than one workgroup's 128 rows
        (2, 8, 32, 64, 32, 128, 4),      # every chunk attends
        (2, 8, 32, 64, 32, 128, 0),      # no target attends
        (1, 2, 64, 100, 16, 96, None),   # head_dim 64
        (2, 2, 32, 1, 1, 2, None),       # the smallest legal problem
        (1, 4, 32, 513, 70, 280, 3),     # ragged everything: sections end inside 32-row tiles
        (2, 2, 32, 128, 0, 64, 0),       # no buffer rows at all
        (1, 2, 128, 40, 8, 32, None),    # head_dim 128: the float32-arithmetic kernels for every dtype
    ],
)
def test_row_mask_attention_backward_matches_oracle(device, dtype, B, H, D, Nc, Nb, T, A):
    import ar_nanotabpfn_amd.attention_kernels as ak
    from ar_nanotabpfn_amd.attention import create_row_mask

    R = Nc + Nb + T
    q, k, v, dout = (randn((B, H, R, D), s, dtype, 0.7) for s in (1, 2, 3, 4))
    chunks = create_row_mask(R, Nc, Nb, A, device=device).attending_chunks
    dq_ref, dk_ref, dv_ref = ao.row_mask_attention_backward(to_np(q), to_np(k), to_np(v), to_np(dout), Nc, Nb, A)
    _, lse_ref = ao.buffer_attention(to_np(q), to_np(k), to_np(v), mask=ao.row_mask(R, Nc, Nb, A)[None, None])
    qd, kd, vd, gd = (t.to(device) for t in (q, k, v, dout))
    for use_mfma in (True, False):
        out, lse = ak._row_mask_forward(qd, kd, vd, Nc, Nb, chunks, use_mfma, want_lse=True)
        # (the matrix-core forward rounds scale * log2(e) * q to the input type, the rounding model
        # of the reference kernel: a few 1e-3 on a score, which a 7-key row does not average out)
        assert max_abs(to_np(lse), lse_ref) <= (1e-5 if dtype == torch.float32 else 4e-3)
        dq, dk, dv = ak.row_mask_attention_backward(qd, kd, vd, out, gd, lse, Nc, Nb, chunks, use_triton=use_mfma)
        for name, got, ref in (("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
            assert got.shape == (B, H, R, D)
            assert _grad_err(got, ref) <= _grad_tol(dtype), f"{name} use_mfma={use_mfma}"
        # nobody sees a target key: exact zeros, whatever the arithmetic
        assert not dk[:, :, Nc + Nb:].any() and not dv[:, :, Nc + Nb:].any()


def test_row_mask_attention_autograd_on_projection_views(device):
    """q, k, v as strided views of one [B,R,3,H,D] leaf, as the layer's projections produce them:
    ``backward()`` fills the leaf's gradient with dq, dk, dv side by side."""
    import ar_nanotabpfn_amd.attention_kernels as ak

    B, H, D, Nc, Nb, T = 2, 4, 32, 130, 8, 48
    R = Nc + Nb + T
    qkv = randn((B, R, 3, H, D), 5, torch.bfloat16, 0.7).to(device).requires_grad_()
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
    dout = randn((B, H, R, D), 6, torch.bfloat16, 0.7).to(device)
    out = ak.row_mask_attention(q, k, v, Nc, Nb, T // (2 * Nb))
    assert out.requires_grad
    (out.float() * dout.float()).sum().backward()
    refs = ao.row_mask_attention_backward(to_np(q), to_np(k), to_np(v), to_np(dout), Nc, Nb)
    for i, ref in enumerate(refs):
        assert _grad_err(qkv.grad[:, :, i].transpose(1, 2), ref) <= 2e-2
    # without recorded gradients the same call is the plain forward
    with torch.no_grad():
        out2 = ak.row_mask_attention(q, k, v, Nc, Nb, T // (2 * Nb))
    assert not out2.requires_grad and torch.equal(out2, out.detach())


def test_row_mask_backward_argument_errors(device):
    import ar_nanotabpfn_amd.attention_kernels as ak

    q = torch.zeros(1, 2, 10, 32, device=device, dtype=torch.bfloat16)
    lse = torch.zeros(1, 2, 10, device=device)
    with pytest.raises(ValueError):
        ak.row_mask_attention_backward(q, q, q, q, q, lse[:, :, :5], 4, 2, 1)
    with pytest.raises(ValueError):
        ak.row_mask_attention_backward(q, q, q, q, q.float(), lse, 4, 2, 1)
    with pytest.raises(ValueError):
        ak.row_mask_attention_backward(q, q, q, q, q, lse, 0, 2, 1)


def _torch_row_attention(q, k, v, context_len, buffer_len, attending_chunks, use_triton=True):
    """Plain PyTorch statement of the same op (dense mask, float32 softmax): the reference the
    device path's parameter gradients are compared with."""
    from ar_nanotabpfn_amd.attention import RowMask

    R = q.shape[2]
    mask = RowMask(R, context_len, buffer_len, attending_chunks).dense(q.device)
    s = torch.matmul(q.float(), k.float().transpose(-1, -2)) * q.shape[-1] ** -0.5
    p = torch.softmax(s.masked_fill(~mask, float("-inf")), dim=-1)
    return torch.matmul(p, v.float()).to(q.dtype)


def _training_problem(device, dtype, cfg, B, Nc, Nb, Nt, seed=1):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(device, dtype)  # noqa: E731
    F_ = cfg["num_features"]
    return mk(B, Nc, F_), mk(B, Nc), mk(B, Nb, F_), mk(B, Nb), mk(B, Nt, F_), mk(B, Nt)


def test_training_step_gradients_match_torch_reference(device, monkeypatch):
    """``loss.backward()`` through the device row attention (float32 model) against the same model
    with the row attention as plain PyTorch: every parameter's gradient."""
    import ar_nanotabpfn_amd.attention_kernels as ak
    from ar_nanotabpfn_amd.attention import create_dense_mask, create_row_mask
    from ar_nanotabpfn_amd.model import ARTabPFN

    cfg = dict(d_model=64, n_heads=2, n_layers=2, d_ff=96, num_features=3, buffer_size=8, num_components=3)
    torch.manual_seed(0)
    model = ARTabPFN(**cfg).to(device)
    B, Nc, Nb, Nt = 3, 70, 8, 40
    xc, yc, xb, yb, xt, yt = _training_problem(device, torch.float32, cfg, B, Nc, Nb, Nt)
    masks = (create_dense_mask(1, device=device), create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device))

    def grads():
        model.zero_grad(set_to_none=True)
        loss = model(xc, yc, xb, yb, xt, *masks, y_target=yt)
        loss.backward()
        return loss.item(), {n: p.grad.clone() for n, p in model.named_parameters()}

    loss_dev, g_dev = grads()
    monkeypatch.setattr(ak, "row_mask_attention", _torch_row_attention)
    loss_ref, g_ref = grads()
    monkeypatch.undo()
    assert abs(loss_dev - loss_ref) <= 1e-5
    assert set(g_dev) == {n for n, _ in model.named_parameters()}  # nobody is left without a gradient
    for name, ref in g_ref.items():
        scale = max(1e-3, float(ref.abs().max()))
        assert float((g_dev[name] - ref).abs().max()) <= 2e-4 * scale, name
    # the feature attention has one key per query: its q and k projections get exact zeros
    for name in ("backbone.layers.0.attn_features.q_proj.weight", "backbone.layers.1.attn_features.k_proj.weight"):
        assert not g_dev[name].any()
    # the no-grad path (fused inference kernels) gives the same loss
    with torch.no_grad():
        assert abs(float(model(xc, yc, xb, yb, xt, *masks, y_target=yt)) - loss_dev) <= 1e-5


@pytest.mark.parametrize(
    "cfg,B,Nc,Nb,Nt",
    [
        (dict(d_model=128, n_heads=4, n_layers=2, d_ff=128, num_features=5, buffer_size=16, num_components=4),
         4, 200, 16, 96),
        # the model and batch shape of the reference's configs/train_tabular_online.yaml (12 layers there)
        (dict(d_model=128, n_heads=4, n_layers=4, d_ff=256, num_features=2, buffer_size=32, num_components=20),
         8, 64, 32, 512),
    ],
)
def test_training_step_under_bf16_autocast(device, monkeypatch, cfg, B, Nc, Nb, Nt):
    """The reference trains under bf16 autocast (train.py:289-292): q, k, v reach the row attention
    as bf16 and take the matrix-core kernels in both directions.  Parameter gradients against the
    plain PyTorch statement under the same autocast, and a few optimiser steps."""
    import ar_nanotabpfn_amd.attention_kernels as ak
    from ar_nanotabpfn_amd.attention import create_dense_mask, create_row_mask
    from ar_nanotabpfn_amd.model import ARTabPFN

    torch.manual_seed(0)
    model = ARTabPFN(**cfg).to(device)
    xc, yc, xb, yb, xt, yt = _training_problem(device, torch.float32, cfg, B, Nc, Nb, Nt)
    masks = (create_dense_mask(1, device=device), create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device))
    calls = []
    real_backward = ak.row_mask_attention_backward
    monkeypatch.setattr(ak, "row_mask_attention_backward",
                        lambda *a, **kw: calls.append(a[0].dtype) or real_backward(*a, **kw))

    def grads():
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = model(xc, yc, xb, yb, xt, *masks, y_target=yt)
        loss.backward()
        return loss.item(), torch.cat([p.grad.flatten() for p in model.parameters()])

    loss_dev, g_dev = grads()
    assert calls == [torch.bfloat16] * cfg["n_layers"]
    with monkeypatch.context() as m:
        m.setattr(ak, "row_mask_attention", _torch_row_attention)
        loss_ref, g_ref = grads()
    cos = float(torch.dot(g_dev, g_ref) / (g_dev.norm() * g_ref.norm()))
    rel = float((g_dev - g_ref).norm() / g_ref.norm())
    print(f"\n[bf16 autocast training step] loss {loss_dev:.5f} vs {loss_ref:.5f}, gradient cosine {cos:.6f}, "
          f"relative difference {rel:.4f}")
    assert abs(loss_dev - loss_ref) <= 2e-2 and cos >= 0.999 and rel <= 5e-2

    opt = torch.optim.AdamW(model.parameters(), lr=2e-3)
    losses = []
    for _ in range(8):
        opt.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = model(xc, yc, xb, yb, xt, *masks, y_target=yt)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(np.isfinite(losses)) and losses[-1] < losses[0] - 0.05, losses


def test_dense_attention_refuses_to_backpropagate(device):
    """The dense (prefill) attention is inference-only: its forward works wherever it is called,
    a gradient that reaches it raises instead of silently stopping."""
    from ar_nanotabpfn_amd.attention import MultiheadAttention, create_dense_mask

    attn = MultiheadAttention(64, 2).to(device=device, dtype=torch.bfloat16)
    x = torch.zeros(1, 8, 64, device=device, dtype=torch.bfloat16)
    out, _ = attn(x, x, x, create_dense_mask(8, device=device))
    with pytest.raises(NotImplementedError):
        out.float().sum().backward()
    with torch.no_grad():
        out2, _ = attn(x, x, x, create_dense_mask(8, device=device))
    assert torch.equal(out2, out.detach())


def test_row_mask_attending_chunks_beyond_the_targets(device):
    """More attending chunks than there are target rows (up to the largest int) mean "every chunk
    attends": same output and gradients as the exact count."""
    import ar_nanotabpfn_amd.attention_kernels as ak

    B, H, D, Nc, Nb, T = 2, 2, 32, 40, 8, 64
    R = Nc + Nb + T
    q, k, v, dout = (randn((B, H, R, D), s, torch.bfloat16, 0.7).to(device) for s in (1, 2, 3, 4))
    want, lse = ak._row_mask_forward(q, k, v, Nc, Nb, T // Nb, True, want_lse=True)
    grads = ak.row_mask_attention_backward(q, k, v, want, dout, lse, Nc, Nb, T // Nb)
    for chunks in (T // Nb + 5, 2 ** 31 - 1):
        out, lse2 = ak._row_mask_forward(q, k, v, Nc, Nb, chunks, True, want_lse=True)
        assert torch.equal(out, want) and torch.equal(lse2, lse)
        for g, w in zip(ak.row_mask_attention_backward(q, k, v, out, dout, lse2, Nc, Nb, chunks), grads):
            assert torch.equal(g, w)


def test_row_mask_backward_at_the_reference_training_shape(device):
    """The largest shape of the reference's training defaults (train.py:44-64: batch 64 here, 4 heads
    of 32, 1024 context + 32 buffer + 512 target rows), where the oracle is too slow for the whole
    batch: the oracle on two datasets, and for all of them what does not depend on size — the
    matrix-core kernels against the float32-arithmetic ones, key gradients summing to zero, value
    gradients summing to the sum of the output gradients, zeros for the target keys."""
    import ar_nanotabpfn_amd.attention_kernels as ak

    B, H, D, Nc, Nb, T = 64, 4, 32, 1024, 32, 512
    R, A = Nc + Nb + T, T // (2 * Nb)
    qkv = randn((B, R, 3, H, D), 11, torch.bfloat16, 0.7).to(device)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
    dout = randn((B, R, H, D), 12, torch.bfloat16, 0.7).to(device).transpose(1, 2)
    out, lse = ak._row_mask_forward(q, k, v, Nc, Nb, A, True, want_lse=True)
    dq, dk, dv = ak.row_mask_attention_backward(q, k, v, out, dout, lse, Nc, Nb, A)
    pq, pk, pv = ak.row_mask_attention_backward(q, k, v, out, dout, lse, Nc, Nb, A, use_triton=False)
    for name, a, b in (("dq", dq, pq), ("dk", dk, pk), ("dv", dv, pv)):
        scale = max(1.0, float(b.float().abs().max()))
        assert float((a.float() - b.float()).abs().max()) <= 2e-2 * scale, name
    refs = ao.row_mask_attention_backward(*(to_np(t[:2]) for t in (q, k, v, dout)), Nc, Nb, A)
    for name, got, ref in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        assert _grad_err(got[:2], ref) <= 2e-2, name
    assert not dk[:, :, Nc + Nb:].any() and not dv[:, :, Nc + Nb:].any()
    # sums over 1056 keys of 16-bit results: the rounding of each term is what is left
    dk_sum = dk.float().sum(dim=2).abs().max()
    assert float(dk_sum) <= 2e-2 * float(dk.float().abs().sum(dim=2).max())
    dv_sum, do_sum = dv.float().sum(dim=2), dout.float().sum(dim=2)
    assert float((dv_sum - do_sum).abs().max()) <= 1e-2 * float(dout.float().abs().sum(dim=2).max())
