"""The training row mask as a tile schedule (``artab_row_mask_attention``) and the forward-only
training pass built on it, against the oracle and the loss the reference computed for the
fixture (attention.py:86-175, model.py:317-369)."""

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
    loss = model(*args, feat, create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device), y_target=t("train_y_tgt"))
    assert abs(float(loss) - float(data["train_loss"])) <= 1e-4
    loss3 = model(*args, feat, create_row_mask(Nc + Nb + Nt, Nc, Nb, attending_chunks=3, device=device),
                  y_target=t("train_y_tgt"))
    assert abs(float(loss3) - float(data["train_loss_attend3"])) <= 1e-4
    assert model(*args, feat, create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device)) is None  # no labels, no loss


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
    print(f"\n[training forward bf16] loss {float(loss):.5f} vs exact {ref:.5f}")
    assert abs(float(loss) - ref) <= 2e-2
