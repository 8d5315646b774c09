"""Writes ``tiny_model.npz``: a seeded tiny AR-TabPFN ``state_dict``, inputs, and the
outputs the reference implementation computes for them on the CPU.

The fixture pins what only the reference's source fixes — embedder wiring (marker
indices, mean over features), post-norm order, head raw layout, AR-token indexing —
for the numpy oracle and, through it, for the device path.  It is made in the build
container only (the reference checkout is not available elsewhere):

    python tests/golden/make_tiny_model_fixture.py /root/reference

Contents: weights (float32), x/y context and targets, teacher-forced log-density for
the per-dataset ("flex_attention") and shared ("triton_shared_context") backends, and
the per-step target representation of a decode with prescribed buffer values under
the reference's sampling rule for AR tokens, and the training forward (context, buffer and
target rows in one pass under ``create_row_mask``): its loss and the target rows' output.
"""

import os
import sys

import numpy as np
import torch


def main(ref_root: str) -> None:
    sys.path.insert(0, ref_root)
    from ar_tabpfn.model.inference import ARTabPFNPredictor  # noqa: E402
    from ar_tabpfn.model.model import ARTabPFN  # noqa: E402

    torch.manual_seed(0)
    cfg = dict(d_model=32, n_heads=2, n_layers=2, d_ff=48, num_features=3, buffer_size=4, num_components=3)
    model = ARTabPFN(**cfg).eval()
    # non-trivial norms / biases so that a swapped norm or a dropped bias is visible
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name or name.endswith("bias") or "marker" in name:
                p.add_(0.2 * torch.randn(p.shape, generator=g))

    B, Nc, Nt, F = 3, 7, 5, 3
    g = torch.Generator().manual_seed(2)
    x_ctx = torch.randn(B, Nc, F, generator=g)
    y_ctx = torch.randn(B, Nc, generator=g)
    x_tgt = torch.randn(B, Nt, F, generator=g)
    y_tgt = torch.randn(B, Nt, generator=g)

    out = {f"w::{k}": v.detach().numpy() for k, v in model.state_dict().items()}
    out.update(x_ctx=x_ctx.numpy(), y_ctx=y_ctx.numpy(), x_tgt=x_tgt.numpy(), y_tgt=y_tgt.numpy())
    out["cfg"] = np.array([cfg[k] for k in ("d_model", "n_heads", "n_layers", "d_ff", "num_features", "buffer_size", "num_components")])

    def clear(model):
        for layer in model.backbone.layers:
            for a in ("k_cache", "v_cache", "k_ctx_cache", "v_ctx_cache", "k_buf_cache", "v_buf_cache"):
                if hasattr(layer, a):
                    delattr(layer, a)

    with torch.no_grad():
        pred = ARTabPFNPredictor.from_trained_model(model, backend="flex_attention")
        out["ll_per_dataset"] = pred.evaluate_joint_density(x_ctx, y_ctx, x_tgt, y_tgt).numpy()
        clear(model)

        # shared backend: context of batch entry 0 is used for every trajectory
        x_sh, y_sh = x_ctx[0:1].expand(B, -1, -1).contiguous(), y_ctx[0:1].expand(B, -1).contiguous()
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            pred_s = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
        out["ll_shared"] = pred_s.evaluate_joint_density(x_sh, y_sh, x_tgt, y_tgt).numpy()
        clear(model)

        # decode with prescribed buffer values (construction of tests/test_triton_gpu.py:126-165)
        for name, p, xc, yc in (("per_dataset", pred, x_ctx, y_ctx), ("shared", pred_s, x_sh, y_sh)):
            p.init_kv_cache(B, Nt if name == "shared" else Nc + Nt, xc.device, xc.dtype)
            p.prefill_context(xc, yc)
            zs = []
            for t in range(Nt):
                emb_t = p.embedder.embed_target(x_tgt[:, t : t + 1])
                if t == 0:
                    emb, commit = emb_t, 0
                else:
                    emb_b = p.embedder.embed_buffer(x_tgt[:, t - 1 : t], y_tgt[:, t - 1 : t])
                    emb_b = emb_b + p.ar_tokens[t % p.ar_tokens.shape[0]]
                    emb, commit = torch.cat([emb_b, emb_t], dim=1), 1
                zs.append(p.transformer_decode(emb, commit=commit)[:, -1:])
            out[f"z_decode_{name}"] = torch.cat(zs, dim=1).numpy()
            clear(model)

        # training forward under the row mask (model.py:317-369, attention.py:86-175): buffer_size
        # buffer rows, 4 * buffer_size target rows (two of the four chunks attend to the buffer)
        from ar_tabpfn.model.attention import create_dense_mask, create_row_mask  # noqa: E402

        Nb, Ntr = cfg["buffer_size"], 4 * cfg["buffer_size"]
        g = torch.Generator().manual_seed(3)
        x_buf, y_buf = torch.randn(B, Nb, F, generator=g), torch.randn(B, Nb, generator=g)
        x_trn, y_trn = torch.randn(B, Ntr, F, generator=g), torch.randn(B, Ntr, generator=g)
        mask_rows = create_row_mask(Nc + Nb + Ntr, Nc, Nb, device="cpu")
        mask_feat = create_dense_mask(1, device="cpu")
        loss = model(x_ctx, y_ctx, x_buf, y_buf, x_trn, mask_feat, mask_rows, y_target=y_trn)
        out.update(train_x_buf=x_buf.numpy(), train_y_buf=y_buf.numpy(), train_x_tgt=x_trn.numpy(),
                   train_y_tgt=y_trn.numpy(), train_loss=np.array(float(loss)))
        # the same pass with three attending chunks
        mask3 = create_row_mask(Nc + Nb + Ntr, Nc, Nb, attending_chunks=3, device="cpu")
        out["train_loss_attend3"] = np.array(float(model(x_ctx, y_ctx, x_buf, y_buf, x_trn, mask_feat, mask3, y_target=y_trn)))

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny_model.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
