"""The PyTorch-CPU restatement of the reference's op sequence (oracle/torch_cpu_path.py: the CPU
baseline that bench.py times) against the numpy oracle and against the vectors the reference
itself computed (tests/golden/tiny_model.npz).  CPU only."""

import os

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from oracle import model_oracle as mo
from oracle import torch_cpu_path as tp
from tests.test_oracle import _data, tiny_state_dict

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "tiny_model.npz")


def _t(a, dtype=torch.float64):
    return torch.as_tensor(np.asarray(a), dtype=dtype)


def _r(seed, *shape):
    return np.random.default_rng(seed).normal(size=shape)


def test_context_buffer_merge_match_the_numpy_oracle():
    B, H, Nc, Nb, D = 3, 2, 13, 5, 8
    q, kc, vc = _r(1, B, H, 2, D), _r(2, H, Nc, D), _r(3, H, Nc, D)
    kb, vb = _r(4, B, H, Nb, D), _r(5, B, H, Nb, D)
    out, lse = tp.pytorch_context_attention(_t(q), _t(kc), _t(vc))
    ref_out, ref_lse = ao.context_attention(q, kc, vc)
    np.testing.assert_allclose(out.numpy(), ref_out, atol=1e-12)
    np.testing.assert_allclose(lse.numpy(), ref_lse, atol=1e-5)  # the reference takes it of scores.float()
    mask = np.random.default_rng(6).random((B, H, 2, Nb)) < 0.5
    mask[0, 0, 0] = False  # a row that sees nothing: out 0, lse -inf (triton_kernels.py:598-611)
    ob, lb = tp.pytorch_buffer_attention(_t(q), _t(kb), _t(vb), mask=torch.as_tensor(mask))
    rob, rlb = ao.buffer_attention(q, kb, vb, mask=mask)
    np.testing.assert_allclose(ob.numpy(), rob, atol=1e-12)
    assert np.isneginf(lb.numpy()[0, 0, 0]) and np.all(ob.numpy()[0, 0, 0] == 0)
    np.testing.assert_allclose(lb.numpy()[np.isfinite(rlb)], rlb[np.isfinite(rlb)], atol=1e-5)
    merged = tp.merge_attention_outputs(out, lse.double(), ob, lb.double())
    np.testing.assert_allclose(merged.numpy(), ao.merge_attention_outputs(ref_out, ref_lse, rob, rlb), atol=1e-6)
    hyb = tp.hybrid_attention(_t(q), _t(kc), _t(vc), _t(kb), _t(vb))
    np.testing.assert_allclose(hyb.numpy(), ao.hybrid_attention(q, kc, vc, kb, vb), atol=1e-6)
    empty = tp.hybrid_attention(_t(q), _t(kc), _t(vc), _t(kb[:, :, :0]), _t(vb[:, :, :0]))
    np.testing.assert_allclose(empty.numpy(), ref_out, atol=1e-12)


@pytest.mark.parametrize("Nt", [1, 2, 7])
def test_teacher_forcing_masks_and_attention_match_the_numpy_oracle(Nt):
    assert np.array_equal(tp.teacher_forcing_buffer_mask(Nt).numpy(), ao.teacher_forcing_buffer_mask(Nt))
    for cached in (0, 5):
        assert np.array_equal(tp.teacher_forcing_mask(cached, Nt).numpy(), ao.teacher_forcing_mask(cached, Nt))
    B, H, Nc, D = 2, 2, 9, 8
    q, kc, vc = _r(7, B, H, 2 * Nt, D), _r(8, H, Nc, D), _r(9, H, Nc, D)
    kb, vb = _r(10, B, H, Nt, D), _r(11, B, H, Nt, D)
    out = tp.hybrid_teacher_forcing_attention(_t(q), _t(kc), _t(vc), _t(kb), _t(vb), Nt)
    np.testing.assert_allclose(out.numpy(), ao.hybrid_teacher_forcing_attention(q, kc, vc, kb, vb, Nt), atol=1e-6)
    with pytest.raises(ValueError):
        tp.hybrid_teacher_forcing_attention(_t(q), _t(kc), _t(vc), _t(kb), _t(vb), Nt + 1)


def test_masked_dense_attention_matches_the_numpy_oracle():
    B, H, R, D = 2, 2, 6, 8
    q, k, v = _r(12, B, H, R, D), _r(13, B, H, R + 3, D), _r(14, B, H, R + 3, D)
    mask = np.tril(np.ones((R, R + 3), dtype=bool), k=2)
    out = tp.masked_dense_attention(_t(q, torch.float32), _t(k, torch.float32), _t(v, torch.float32), torch.as_tensor(mask))
    ref, _ = ao.masked_full_attention(q, k, v, mask=mask)
    np.testing.assert_allclose(out.numpy(), ref, atol=2e-6)


def test_predictor_matches_the_numpy_oracle_on_both_backends():
    sd = tiny_state_dict(seed=4)
    om = mo.OracleModel(sd, n_heads=2)
    tm = tp.TorchCpuModel({k: _t(v) for k, v in sd.items()}, n_heads=2, dtype=torch.float64)
    B, Nc, Nt, F = 3, 6, 4, 3
    xc, yc, xt, yt = _data(5, B, Nc, Nt, F)
    ll_p = tp.TorchCpuPredictor(tm, "per_dataset").evaluate_joint_density(_t(xc), _t(yc), _t(xt), _t(yt))
    np.testing.assert_allclose(ll_p.numpy(), mo.OraclePredictor(om, "per_dataset").evaluate_joint_density(xc, yc, xt, yt),
                               atol=1e-5)  # the dense path scores in float32, as flex's host fallback does
    xc[:], yc[:] = xc[0], yc[0]
    ll_s = tp.TorchCpuPredictor(tm, "shared").evaluate_joint_density(_t(xc), _t(yc), _t(xt), _t(yt))
    np.testing.assert_allclose(ll_s.numpy(), mo.OraclePredictor(om, "shared").evaluate_joint_density(xc, yc, xt, yt), atol=1e-5)
    # step-wise decode with prescribed buffer values (tests/test_triton_gpu.py:126-165), sampling rule
    p = tp.TorchCpuPredictor(tm, "shared")
    p.init_kv_cache(B, Nt, context_len=Nc)
    p.prefill_context(_t(xc), _t(yc))
    zs = []
    bs = tm.ar_tokens.shape[0]
    for t in range(Nt):
        tgt = tm.embed_target(_t(xt[:, t:t + 1]))
        if t == 0:
            emb, commit = tgt, 0
        else:
            emb = torch.cat([tm.embed_buffer(_t(xt[:, t - 1:t]), _t(yt[:, t - 1:t])) + tm.ar_tokens[t % bs], tgt], dim=1)
            commit = 1
        zs.append(p.transformer_decode(emb, commit)[:, -1:])
    ref = mo.OraclePredictor(om, "shared").fixed_buffer_decode(xc, yc, xt, yt, ar_rule="sampling")
    np.testing.assert_allclose(torch.cat(zs, dim=1).numpy(), ref, atol=1e-5)
    assert p.buffer_len == Nt - 1
    with pytest.raises(ValueError):
        for _ in range(3):
            p.transformer_decode(emb, 1)


def test_predictor_matches_the_vectors_the_reference_computed():
    data = np.load(FIXTURE, allow_pickle=False)
    sd = {k[3:]: torch.as_tensor(data[k]) for k in data.files if k.startswith("w::")}
    tm = tp.TorchCpuModel(sd, int(data["cfg"][1]), dtype=torch.float32)
    f = lambda name: torch.as_tensor(data[name], dtype=torch.float32)  # noqa: E731
    ll = tp.TorchCpuPredictor(tm, "per_dataset").evaluate_joint_density(f("x_ctx"), f("y_ctx"), f("x_tgt"), f("y_tgt"))
    np.testing.assert_allclose(ll.numpy(), data["ll_per_dataset"], atol=1e-4, rtol=0)
    B = data["x_ctx"].shape[0]
    xc, yc = f("x_ctx")[0:1].expand(B, -1, -1), f("y_ctx")[0:1].expand(B, -1)
    ll = tp.TorchCpuPredictor(tm, "shared").evaluate_joint_density(xc, yc, f("x_tgt"), f("y_tgt"))
    np.testing.assert_allclose(ll.numpy(), data["ll_shared"], atol=1e-4, rtol=0)


def test_head_sample_follows_the_mixture():
    sd = tiny_state_dict(seed=2)
    tm = tp.TorchCpuModel({k: _t(v) for k, v in sd.items()}, n_heads=2, dtype=torch.float32)
    torch.manual_seed(0)
    z = torch.randn(1, 1, 16).expand(4000, 1, 16).contiguous()
    y = tm.head_sample(z)
    assert y.shape == (4000, 1, 1, 1)
    mean, std, w, _ = tm.head_parameterize(z[:1])
    mix_mean = float((w * mean).sum())
    assert abs(float(y.mean()) - mix_mean) < 0.1


def test_bf16_run_stays_close_to_float32():
    """The baseline is timed in bfloat16 as well; its values are only sanity-checked."""
    sd = tiny_state_dict(seed=3)
    B, Nc, Nt, F = 2, 8, 3, 2
    xc, yc, xt, yt = _data(9, B, Nc, Nt, F)
    lls = []
    for dt in (torch.float32, torch.bfloat16):
        tm = tp.TorchCpuModel({k: _t(v) for k, v in sd.items()}, n_heads=2, dtype=dt)
        lls.append(tp.TorchCpuPredictor(tm, "shared").evaluate_joint_density(_t(xc, dt), _t(yc, dt), _t(xt, dt), _t(yt, dt)).float())
    assert torch.isfinite(lls[1]).all() and float((lls[0] - lls[1]).abs().max()) < 0.5
