"""Pins the numpy oracle: closed forms and invariants the reference's own tests hold,
library routines, and brute-force loops — chosen so that a dropped term, a wrong
sign/index or a transposed operand fails at least one of them.  CPU only."""

import math

import numpy as np
import pytest
import scipy.special
import scipy.stats

from oracle import attention_oracle as ao
from oracle import model_oracle as mo


def rng(seed):
    return np.random.default_rng(seed)


# ----- attention vs brute-force loops and library routines ------------------------------------


@pytest.mark.parametrize("Lq,N,D", [(1, 1, 1), (2, 5, 3), (3, 7, 4)])
def test_context_attention_vs_python_loops(Lq, N, D):
    r = rng(0)
    q, k, v = r.normal(size=(Lq, D)), r.normal(size=(N, D)), r.normal(size=(N, D))
    out, lse = ao.context_attention(q[None, None], k[None], v[None])
    lo, ll = ao.loops_attention(q.tolist(), k.tolist(), v.tolist())
    np.testing.assert_allclose(out[0, 0], np.array(lo), atol=1e-12)
    np.testing.assert_allclose(lse[0, 0], np.array(ll), atol=1e-12)


def test_context_attention_vs_scipy_and_ragged_shapes():
    """B=37 and N_CTX=100 are the ragged cases of tests/test_triton_kernel.py:68-102."""
    r = rng(1)
    for B, H, Nc, D in [(37, 4, 64, 32), (32, 4, 100, 32)]:
        q, k, v = r.normal(size=(B, H, 1, D)), r.normal(size=(H, Nc, D)), r.normal(size=(H, Nc, D))
        out, lse = ao.context_attention(q, k, v)
        for b in (0, B - 1):
            for h in range(H):
                s = (k[h] @ q[b, h, 0]) / math.sqrt(D)  # [Nc]
                np.testing.assert_allclose(lse[b, h, 0], scipy.special.logsumexp(s), atol=1e-12)
                np.testing.assert_allclose(out[b, h, 0], scipy.special.softmax(s) @ v[h], atol=1e-12)


def test_context_attention_operand_roles():
    """One-hot construction: a transposed/exchanged operand cannot pass.  With q = e_0
    scaled hard and k_j = j-th basis direction, the softmax picks key 0 and returns v_0."""
    D, N = 4, 3
    q = np.zeros((1, 1, 1, D))
    q[..., 0] = 200.0
    k = np.eye(N, D)[None]
    v = np.arange(N * D, dtype=float).reshape(1, N, D)
    out, lse = ao.context_attention(q, k, v)
    np.testing.assert_allclose(out[0, 0, 0], v[0, 0], atol=1e-9)
    np.testing.assert_allclose(lse[0, 0, 0], 200.0 / math.sqrt(D), atol=1e-9)


def test_scale_default_and_override():
    r = rng(2)
    q, k, v = r.normal(size=(1, 1, 2, 8)), r.normal(size=(1, 6, 8)), r.normal(size=(1, 6, 8))
    a, la = ao.context_attention(q, k, v)
    b, lb = ao.context_attention(q * 8 ** -0.5, k, v, scale=1.0)
    np.testing.assert_allclose(a, b, atol=1e-12)
    np.testing.assert_allclose(la, lb, atol=1e-12)


def test_per_dataset_context_equals_loop_over_batch():
    r = rng(3)
    B, H, Lq, Nc, D = 3, 2, 4, 9, 8
    q, k, v = r.normal(size=(B, H, Lq, D)), r.normal(size=(B, H, Nc, D)), r.normal(size=(B, H, Nc, D))
    out, lse = ao.context_attention(q, k, v)
    for b in range(B):
        ob, lb = ao.context_attention(q[b : b + 1], k[b], v[b])
        np.testing.assert_allclose(out[b], ob[0], atol=1e-12)
        np.testing.assert_allclose(lse[b], lb[0], atol=1e-12)


def test_buffer_attention_mask_vs_python_loops_and_empty_rows():
    r = rng(4)
    Lq, N, D = 4, 6, 3
    q, k, v = r.normal(size=(Lq, D)), r.normal(size=(N, D)), r.normal(size=(N, D))
    mask = r.random((Lq, N)) < 0.5
    mask[2] = False  # a row with no visible key
    out, lse = ao.buffer_attention(q[None, None], k[None, None], v[None, None], mask=mask[None, None])
    lo, ll = ao.loops_attention(q.tolist(), k.tolist(), v.tolist(), mask=mask.tolist())
    np.testing.assert_allclose(out[0, 0], np.array(lo), atol=1e-12)
    np.testing.assert_allclose(lse[0, 0], np.array(ll), atol=1e-12)
    assert np.all(out[0, 0, 2] == 0) and np.isneginf(lse[0, 0, 2])


# ----- merge: the closed forms the reference's tests hold -----------------------------------------


def test_merge_dominant_source():
    """tests/test_triton_kernel.py:345-364: lse 10 vs -10 -> out_ctx (atol 1e-4)."""
    r = rng(5)
    a, b = r.normal(size=(8, 4, 1, 32)), r.normal(size=(8, 4, 1, 32))
    out = ao.merge_attention_outputs(a, np.full((8, 4, 1), 10.0), b, np.full((8, 4, 1), -10.0))
    np.testing.assert_allclose(out, a, atol=1e-4)
    w = 1.0 / (1.0 + math.exp(-20.0))
    np.testing.assert_allclose(out, w * a + (1 - w) * b, atol=1e-14)


def test_merge_equal_sources():
    """tests/test_triton_kernel.py:366-382: equal lse -> arithmetic mean."""
    r = rng(6)
    a, b = r.normal(size=(8, 4, 1, 32)), r.normal(size=(8, 4, 1, 32))
    out = ao.merge_attention_outputs(a, np.full((8, 4, 1), 5.0), b, np.full((8, 4, 1), 5.0))
    np.testing.assert_allclose(out, (a + b) / 2, atol=1e-14)


def test_merge_equals_attention_over_concatenated_keys():
    """tests/test_triton_kernel.py:204-240 (B,H,Lq,D = 16,4,1,32; N_CTX,N_BUF = 64,16)."""
    r = rng(7)
    B, H, Lq, D, Nc, Nb = 16, 4, 1, 32, 64, 16
    q = r.normal(size=(B, H, Lq, D))
    kc, vc = r.normal(size=(H, Nc, D)), r.normal(size=(H, Nc, D))
    kb, vb = r.normal(size=(B, H, Nb, D)), r.normal(size=(B, H, Nb, D))
    oc, lc = ao.context_attention(q, kc, vc)
    ob, lb = ao.buffer_attention(q, kb, vb)
    merged = ao.merge_attention_outputs(oc, lc, ob, lb)
    k_full = np.concatenate([np.broadcast_to(kc[None], (B, H, Nc, D)), kb], axis=2)
    v_full = np.concatenate([np.broadcast_to(vc[None], (B, H, Nc, D)), vb], axis=2)
    full, lse_full = ao.masked_full_attention(q, k_full, v_full)
    np.testing.assert_allclose(merged, full, atol=1e-12)
    np.testing.assert_allclose(np.logaddexp(lc, lb), lse_full, atol=1e-12)
    np.testing.assert_allclose(ao.hybrid_attention(q, kc, vc, kb, vb), full, atol=1e-12)


def test_merge_with_masked_buffer():
    """tests/test_triton_kernel.py:242-282: only the first 4 buffer keys visible."""
    r = rng(8)
    B, H, Lq, D, Nc, Nb = 8, 4, 1, 32, 32, 8
    q = r.normal(size=(B, H, Lq, D))
    kc, vc = r.normal(size=(H, Nc, D)), r.normal(size=(H, Nc, D))
    kb, vb = r.normal(size=(B, H, Nb, D)), r.normal(size=(B, H, Nb, D))
    bm = np.zeros((B, H, Lq, Nb), dtype=bool)
    bm[..., :4] = True
    merged = ao.hybrid_attention(q, kc, vc, kb, vb, buf_mask=bm)
    k_full = np.concatenate([np.broadcast_to(kc[None], (B, H, Nc, D)), kb], axis=2)
    v_full = np.concatenate([np.broadcast_to(vc[None], (B, H, Nc, D)), vb], axis=2)
    fm = np.ones((B, H, Lq, Nc + Nb), dtype=bool)
    fm[..., Nc:] = bm
    full, _ = ao.masked_full_attention(q, k_full, v_full, mask=fm)
    np.testing.assert_allclose(merged, full, atol=1e-12)


def test_merge_split_invariance_commutativity_and_neutral_element():
    r = rng(9)
    B, H, Lq, D, N = 3, 2, 2, 8, 24
    q, k, v = r.normal(size=(B, H, Lq, D)), r.normal(size=(H, N, D)), r.normal(size=(H, N, D))
    full, lse = ao.context_attention(q, k, v)
    o1, l1 = ao.context_attention(q, k[:, :7], v[:, :7])
    o2, l2 = ao.context_attention(q, k[:, 7:], v[:, 7:])
    np.testing.assert_allclose(ao.merge_attention_outputs(o1, l1, o2, l2), full, atol=1e-12)
    np.testing.assert_allclose(ao.merge_attention_outputs(o2, l2, o1, l1), full, atol=1e-12)
    ninf = np.full(l1.shape, -np.inf)
    np.testing.assert_array_equal(ao.merge_attention_outputs(o1, l1, np.zeros_like(o1), ninf), o1)
    assert np.isnan(ao.merge_attention_outputs(o1, ninf, o1, ninf)).all()  # 0/0 as in the reference formula


def test_hybrid_empty_buffer_is_context_only():
    """tests/test_triton_kernel.py:319-339."""
    r = rng(10)
    q, k, v = r.normal(size=(32, 4, 1, 32)), r.normal(size=(4, 64, 32)), r.normal(size=(4, 64, 32))
    kb = np.empty((32, 4, 0, 32))
    oc, _ = ao.context_attention(q, k, v)
    np.testing.assert_array_equal(ao.hybrid_attention(q, k, v, kb, kb), oc)


# ----- masks -----------------------------------------------------------------------------------------


@pytest.mark.parametrize("Nt", [1, 2, 3, 16, 37])
def test_teacher_forcing_masks_agree_and_count(Nt):
    """Two independent statements in the reference (triton_kernels.py:627-633 and
    inference.py:543-568) must describe one mask; Nt^2 visible buffer pairs."""
    m_buf = ao.teacher_forcing_buffer_mask(Nt)[0, 0]
    for Nc in (0, 5):
        m_full = ao.teacher_forcing_mask(Nc, Nt)
        assert m_full.shape == (2 * Nt, Nc + 2 * Nt)
        assert m_full[:, :Nc].all()
        np.testing.assert_array_equal(m_full[:, Nc : Nc + Nt], m_buf)
        assert not m_full[:, Nc + Nt :].any()  # target keys never visible
    assert m_buf.sum() == Nt * Nt
    assert not m_buf[Nt].any()  # target 0 sees no buffer
    # row-by-row restatement: buffer i sees j <= i, target i sees j < i
    for i in range(Nt):
        assert m_buf[i].tolist() == [j <= i for j in range(Nt)]
        assert m_buf[Nt + i].tolist() == [j < i for j in range(Nt)]


def test_target0_has_no_buffers():
    """tests/test_triton_kernel.py:135-151."""
    r = rng(11)
    B, H, Nt, D = 4, 2, 3, 16
    q, kb, vb = r.normal(size=(B, H, 2 * Nt, D)), r.normal(size=(B, H, Nt, D)), r.normal(size=(B, H, Nt, D))
    out, lse = ao.teacher_forcing_buffer_attention(q, kb, vb, Nt)
    assert np.all(out[:, :, Nt] == 0) and np.isneginf(lse[:, :, Nt]).all()
    with pytest.raises(ValueError):
        ao.teacher_forcing_buffer_attention(q[:, :, :-1], kb, vb, Nt)
    with pytest.raises(ValueError):
        ao.teacher_forcing_buffer_attention(q, kb[:, :, :-1], vb[:, :, :-1], Nt)


@pytest.mark.parametrize("Nt,Nc", [(4, 5), (1, 3)])
def test_hybrid_teacher_forcing_matches_masked_full(Nt, Nc):
    """tests/test_triton_kernel.py:157-198 (B,H,Nt,D = 2,3,4,16; N_CTX = 5) and Nt=1."""
    r = rng(12)
    B, H, D = 2, 3, 16
    q = r.normal(size=(B, H, 2 * Nt, D))
    kc, vc = r.normal(size=(H, Nc, D)), r.normal(size=(H, Nc, D))
    kb, vb = r.normal(size=(B, H, Nt, D)), r.normal(size=(B, H, Nt, D))
    hyb = ao.hybrid_teacher_forcing_attention(q, kc, vc, kb, vb, Nt)
    pad = r.normal(size=(B, H, Nt, D))  # target keys: values must not matter
    k_full = np.concatenate([np.broadcast_to(kc[None], (B, H, Nc, D)), kb, pad], axis=2)
    v_full = np.concatenate([np.broadcast_to(vc[None], (B, H, Nc, D)), vb, pad], axis=2)
    full, _ = ao.masked_full_attention(q, k_full, v_full, mask=ao.teacher_forcing_mask(Nc, Nt)[None, None])
    np.testing.assert_allclose(hyb, full, atol=1e-12)


def test_decode_mask_closed_form_and_decode_step():
    """inference.py:512-519: for num_new=2 both rows see kv < num_cached+1; for num_new=1
    the target sees kv < num_cached.  decode_step_attention == masked attention over the
    per-trajectory full cache."""
    assert ao.decode_mask(5, 1).tolist() == [[True] * 5 + [False]]
    assert ao.decode_mask(5, 2).tolist() == [[True] * 6 + [False], [True] * 6 + [False]]
    r = rng(13)
    B, H, D, Nc, nb = 3, 2, 8, 6, 4
    q = r.normal(size=(B, H, 2, D))
    kc, vc = r.normal(size=(H, Nc, D)), r.normal(size=(H, Nc, D))
    kb, vb = r.normal(size=(B, H, nb, D)), r.normal(size=(B, H, nb, D))
    kn, vn = r.normal(size=(B, H, 2, D)), r.normal(size=(B, H, 2, D))
    out, k_all, v_all = ao.decode_step_attention(q, kc, vc, kb, vb, kn[:, :, :1], vn[:, :, :1])
    assert k_all.shape[2] == nb + 1
    k_full = np.concatenate([np.broadcast_to(kc[None], (B, H, Nc, D)), kb, kn], axis=2)
    v_full = np.concatenate([np.broadcast_to(vc[None], (B, H, Nc, D)), vb, vn], axis=2)
    full, _ = ao.masked_full_attention(q, k_full, v_full, mask=ao.decode_mask(Nc + nb, 2)[None, None])
    np.testing.assert_allclose(out, full, atol=1e-12)
    out1, _, _ = ao.decode_step_attention(q[:, :, 1:], kc, vc, kb, vb)
    full1, _ = ao.masked_full_attention(
        q[:, :, 1:], k_full[:, :, : Nc + nb + 1], v_full[:, :, : Nc + nb + 1], mask=ao.decode_mask(Nc + nb, 1)[None, None]
    )
    np.testing.assert_allclose(out1, full1, atol=1e-12)


# ----- model pieces ----------------------------------------------------------------------------------


def tiny_state_dict(seed=0, d_model=16, n_heads=2, n_layers=2, d_ff=24, buffer_size=4, K=3):
    r = rng(seed)
    sd = {}

    def lin(name, out_f, in_f, bias=True):
        sd[f"{name}.weight"] = r.normal(size=(out_f, in_f)) / math.sqrt(in_f)
        if bias:
            sd[f"{name}.bias"] = r.normal(size=(out_f,)) * 0.1

    lin("embedder.x_embed", d_model, 1)
    lin("embedder.y_embed", d_model, 1)
    sd["embedder.marker_embed.weight"] = r.normal(size=(3, d_model))
    for i in range(n_layers):
        p = f"backbone.layers.{i}"
        for a in ("attn_features", "attn_rows"):
            for w in ("q_proj", "k_proj", "v_proj", "out_proj"):
                lin(f"{p}.{a}.{w}", d_model, d_model, bias=False)
        lin(f"{p}.ff.0", d_ff, d_model)
        lin(f"{p}.ff.2", d_model, d_ff)
        for n in ("norm1", "norm2", "norm3"):
            sd[f"{p}.{n}.weight"] = 1 + 0.1 * r.normal(size=(d_model,))
            sd[f"{p}.{n}.bias"] = 0.1 * r.normal(size=(d_model,))
    sd["backbone.norm.weight"] = 1 + 0.1 * r.normal(size=(d_model,))
    sd["backbone.norm.bias"] = 0.1 * r.normal(size=(d_model,))
    lin("head.head.0", d_ff, d_model)
    lin("head.head.2", K * 3, d_ff)
    sd["head.mean_bias"] = np.linspace(-1, 1, K)
    sd["head.std_bias"] = np.full(K, math.log(math.exp(1.0 / (K - 1)) - 1))
    sd["head.weight_bias"] = np.zeros(K)
    sd["ar_tokens"] = 0.02 * r.normal(size=(buffer_size, d_model))
    return sd


def test_head_log_likelihood_vs_scipy_mixture():
    sd = tiny_state_dict()
    m = mo.OracleModel(sd, n_heads=2)
    r = rng(1)
    z, y = r.normal(size=(2, 3, 16)), r.normal(size=(2, 3))
    ll = m.head_log_likelihood(z, y)
    mean, std, lw = m.head_parameterize(z)
    K = mean.shape[2]
    assert std.max() <= 2.0 + 1e-3 + 1e-12 and std.min() >= 1e-3
    np.testing.assert_allclose(np.exp(lw).sum(axis=2), 1.0, atol=1e-12)
    # raw layout view(B,T,K,1,3): component k reads outputs 3k, 3k+1, 3k+2 (model.py:195-196)
    h = mo._gelu(z @ sd["head.head.0.weight"].T + sd["head.head.0.bias"]) @ sd["head.head.2.weight"].T + sd["head.head.2.bias"]
    np.testing.assert_allclose(mean[..., 0], h[..., 0::3] + sd["head.mean_bias"], atol=1e-12)
    for b in range(2):
        for t in range(3):
            comp = [scipy.stats.norm.logpdf(y[b, t], mean[b, t, k, 0], std[b, t, k, 0]) + lw[b, t, k, 0] for k in range(K)]
            np.testing.assert_allclose(ll[b, t], scipy.special.logsumexp(comp), atol=1e-10)


def test_layer_norm_and_gelu_textbook():
    r = rng(2)
    x = r.normal(size=(5, 7))
    w, b = r.normal(size=7), r.normal(size=7)
    y = mo._layer_norm(x, w, b)
    ref = (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True) + 1e-5) * w + b
    np.testing.assert_allclose(y, ref, atol=1e-12)
    np.testing.assert_allclose(mo._gelu(x), x * scipy.stats.norm.cdf(x), atol=1e-12)


def _data(seed, B, Nc, Nt, F):
    r = rng(seed)
    return r.normal(size=(B, Nc, F)), r.normal(size=(B, Nc)), r.normal(size=(B, Nt, F)), r.normal(size=(B, Nt))


def test_predictor_decode_equals_teacher_forcing_under_one_ar_rule():
    """Step-wise decode with prescribed buffer values reproduces rows Nt+t of the
    teacher-forced pass when buffer row j carries ar_tokens[j % bs] in both."""
    sd = tiny_state_dict(buffer_size=3)
    m = mo.OracleModel(sd, n_heads=2)
    B, Nc, Nt, F = 2, 7, 5, 2
    xc, yc, xt, yt = _data(3, B, Nc, Nt, F)
    xc[1], yc[1] = xc[0], yc[0]
    p = mo.OraclePredictor(m, "shared")
    z_steps = p.fixed_buffer_decode(xc, yc, xt, yt, ar_rule="teacher_forcing")
    assert p.buffer_len == Nt - 1
    p2 = mo.OraclePredictor(m, "shared")
    p2.init_kv_cache(B, Nt)
    p2.prefill_context(xc, yc)
    buf = m.embed_buffer(xt, yt) + m.ar_tokens[np.arange(Nt) % 3]
    z_tf = p2.teacher_forcing_decode(np.concatenate([buf, m.embed_target(xt)], axis=1), Nt)
    np.testing.assert_allclose(z_steps, z_tf[:, Nt:], atol=1e-10)
    # the reference's sampling rule is offset by one token (inference.py:359 vs :408-409)
    z_samp = mo.OraclePredictor(m, "shared").fixed_buffer_decode(xc, yc, xt, yt, ar_rule="sampling")
    np.testing.assert_allclose(z_samp[:, 0], z_steps[:, 0], atol=1e-12)
    assert np.abs(z_samp[:, 1:] - z_steps[:, 1:]).max() > 1e-6


def test_predictor_shared_equals_per_dataset_when_contexts_are_identical():
    """The comparison of tests/test_triton_gpu.py:200-252 and
    tests/test_triton_joint_density.py:163-210, on the oracle."""
    sd = tiny_state_dict(seed=4)
    m = mo.OracleModel(sd, n_heads=2)
    B, Nc, Nt, F = 3, 6, 4, 3
    xc, yc, xt, yt = _data(5, B, Nc, Nt, F)
    xc[:], yc[:] = xc[0], yc[0]
    ll_s = mo.OraclePredictor(m, "shared").evaluate_joint_density(xc, yc, xt, yt)
    ll_p = mo.OraclePredictor(m, "per_dataset").evaluate_joint_density(xc, yc, xt, yt)
    np.testing.assert_allclose(ll_s, ll_p, atol=1e-10)
    z_s = mo.OraclePredictor(m, "shared").fixed_buffer_decode(xc, yc, xt, yt)
    z_p = mo.OraclePredictor(m, "per_dataset").fixed_buffer_decode(xc, yc, xt, yt)
    np.testing.assert_allclose(z_s, z_p, atol=1e-10)


def test_predictor_context_permutation_invariance_and_overflow():
    sd = tiny_state_dict(seed=6)
    m = mo.OracleModel(sd, n_heads=2)
    B, Nc, Nt, F = 2, 9, 3, 2
    xc, yc, xt, yt = _data(7, B, Nc, Nt, F)
    perm = rng(0).permutation(Nc)
    a = mo.OraclePredictor(m, "per_dataset").evaluate_joint_density(xc, yc, xt, yt)
    b = mo.OraclePredictor(m, "per_dataset").evaluate_joint_density(xc[:, perm], yc[:, perm], xt, yt)
    np.testing.assert_allclose(a, b, atol=1e-10)
    assert a.shape == (B, Nt) and np.isfinite(a).all()
    p = mo.OraclePredictor(m, "shared")
    p.init_kv_cache(B, 0)
    p.prefill_context(xc, yc)
    emb = np.zeros((B, 2, 16))
    with pytest.raises(ValueError):
        p.transformer_decode(emb, commit=1)
    with pytest.raises(ValueError):
        p.transformer_decode(np.zeros((B, 3, 16)), commit=0)


def test_feature_stage_equals_single_key_attention():
    """C=1 feature attention: softmax over one key is 1, so the block is
    out_proj(v_proj(x)); check against an explicit single-key attention."""
    sd = tiny_state_dict(seed=8)
    m = mo.OracleModel(sd, n_heads=2)
    x = rng(9).normal(size=(2, 3, 16))
    H, Dh = 2, 8
    xf = x.reshape(6, 1, 16)
    q = (xf @ sd["backbone.layers.0.attn_features.q_proj.weight"].T).reshape(6, 1, H, Dh).transpose(0, 2, 1, 3)
    k = (xf @ sd["backbone.layers.0.attn_features.k_proj.weight"].T).reshape(6, 1, H, Dh).transpose(0, 2, 1, 3)
    v = (xf @ sd["backbone.layers.0.attn_features.v_proj.weight"].T).reshape(6, 1, H, Dh).transpose(0, 2, 1, 3)
    att, _ = ao.dense_self_attention(q, k, v)
    att = att.transpose(0, 2, 1, 3).reshape(6, 1, 16) @ sd["backbone.layers.0.attn_features.out_proj.weight"].T
    ref = mo._layer_norm(att + xf, sd["backbone.layers.0.norm1.weight"], sd["backbone.layers.0.norm1.bias"])
    np.testing.assert_allclose(m.feature_stage(0, x).reshape(6, 1, 16), ref, atol=1e-12)


# ----- training row mask (attention.py:86-175) ---------------------------------------------------------


def _row_mask_by_regions(C, B, T, attending_chunks=None):
    """The second statement of the mask that the reference holds: region by region, as
    tests/visualize_masks.py:57-85 composes it for its figure."""
    total = C + B + T
    if attending_chunks is None:
        attending_chunks = T // (2 * B)
    M, N = np.meshgrid(np.arange(total), np.arange(total), indexing="ij")
    q_ctx, k_ctx = M < C, N < C
    q_buf, k_buf = (M >= C) & (M < C + B), (N >= C) & (N < C + B)
    q_tgt = M >= C + B
    causal = M >= N
    tgt_buf = q_tgt & k_buf & ((M - C - B) < attending_chunks * B) & ((N - C) <= (M - C - B) % max(B, 1))
    return (q_ctx & k_ctx) | (q_buf & k_buf & causal) | (q_tgt & k_ctx) | (q_buf & k_ctx) | tgt_buf


@pytest.mark.parametrize("C,B,T,A", [(7, 4, 16, None), (1, 1, 2, None), (5, 3, 12, 0), (5, 3, 12, 4), (64, 8, 32, 1), (3, 8, 16, None)])
def test_row_mask_two_statements_agree(C, B, T, A):
    m = ao.row_mask(C + B + T, C, B, A)
    assert m.shape == (C + B + T, C + B + T)
    assert np.array_equal(m, _row_mask_by_regions(C, B, T, A))
    a = T // (2 * B) if A is None else A
    # closed-form pair count: everyone sees the context; buffers are causal among themselves;
    # each of the first min(a*B, T) target rows sees (offset mod B) + 1 buffers
    n_att = min(a * B, T)
    full, rest = divmod(n_att, B)
    expect = (C + B + T) * C + B * (B + 1) // 2 + full * B * (B + 1) // 2 + rest * (rest + 1) // 2
    assert int(m.sum()) == expect
    assert not m[:, C + B:].any()          # nobody sees a target key, not even itself
    assert not m[:C, C:].any()             # the context sees the context only


def test_row_mask_tiny_case_by_hand():
    # rows: c0 c1 | b0 b1 | t0 t1 t2 t3, one attending chunk (targets t0, t1)
    X, o = True, False
    expect = np.array([
        [X, X, o, o, o, o, o, o],
        [X, X, o, o, o, o, o, o],
        [X, X, X, o, o, o, o, o],
        [X, X, X, X, o, o, o, o],
        [X, X, X, o, o, o, o, o],   # t0: buffers <= 0
        [X, X, X, X, o, o, o, o],   # t1: buffers <= 1
        [X, X, o, o, o, o, o, o],   # t2: outside the attending region
        [X, X, o, o, o, o, o, o],
    ])
    assert np.array_equal(ao.row_mask(8, 2, 2, 1), expect)
    assert np.array_equal(ao.row_mask(8, 2, 2), expect)  # default: 4 // (2 * 2) = 1


def test_row_mask_attention_equals_per_row_softmax():
    rng = np.random.default_rng(0)
    C, B, T, D = 5, 3, 6, 8
    R = C + B + T
    q, k, v = (rng.standard_normal((2, 2, R, D)) for _ in range(3))
    out = ao.row_mask_attention(q, k, v, C, B)
    m = ao.row_mask(R, C, B)
    for r in (0, C, C + B - 1, C + B, C + B + 2, R - 1):
        keys = np.nonzero(m[r])[0]
        s = np.einsum("bhd,bhkd->bhk", q[:, :, r], k[:, :, keys]) / np.sqrt(D)
        p = scipy.special.softmax(s, axis=-1)
        assert np.abs(out[:, :, r] - np.einsum("bhk,bhkd->bhd", p, v[:, :, keys])).max() <= 1e-12


@pytest.mark.parametrize("C,B,T,A", [(5, 3, 6, None), (7, 4, 12, 1), (3, 2, 9, 3), (6, 0, 4, 0), (1, 5, 5, 1)])
def test_row_mask_attention_backward_by_finite_differences(C, B, T, A):
    """The analytic gradients against central differences of the forward oracle: for random
    directions (eq, ek, ev) the derivative of sum(out * dout) along them must equal
    <dq, eq> + <dk, ek> + <dv, ev>, direction by direction."""
    rng = np.random.default_rng(10 * C + B)
    D = 8
    R = C + B + T
    q, k, v, dout = (rng.standard_normal((2, 2, R, D)) for _ in range(4))
    dq, dk, dv = ao.row_mask_attention_backward(q, k, v, dout, C, B, A)
    f = lambda q_, k_, v_: (ao.row_mask_attention(q_, k_, v_, C, B, A) * dout).sum()  # noqa: E731
    eps = 1e-5
    for grad, which in ((dq, 0), (dk, 1), (dv, 2)):
        for _ in range(3):
            e = rng.standard_normal(q.shape)
            args_p, args_m = [q, k, v], [q, k, v]
            args_p[which] = args_p[which] + eps * e
            args_m[which] = args_m[which] - eps * e
            numeric = (f(*args_p) - f(*args_m)) / (2 * eps)
            analytic = (grad * e).sum()
            assert abs(numeric - analytic) <= 1e-7 * (1 + abs(analytic)), (which, numeric, analytic)


def test_row_mask_attention_backward_invariants():
    rng = np.random.default_rng(3)
    C, B, T, D = 6, 4, 10, 8
    R = C + B + T
    q, k, v, dout = (rng.standard_normal((2, 3, R, D)) for _ in range(4))
    dq, dk, dv = ao.row_mask_attention_backward(q, k, v, dout, C, B)
    # one vector added to every key shifts all scores of a row alike: the output does not move
    assert np.abs(dk.sum(axis=2)).max() <= 1e-12
    # every row of P sums to one
    assert np.abs(dv.sum(axis=2) - dout.sum(axis=2)).max() <= 1e-12
    # nobody sees a target key
    assert np.all(dk[:, :, C + B:] == 0) and np.all(dv[:, :, C + B:] == 0)
    # an explicit scale is honoured: scale s on (q, k) equals scale 1 on (s q, k), with dq scaled back
    dq1, dk1, dv1 = ao.row_mask_attention_backward(0.3 * q, k, v, dout, C, B, scale=1.0)
    dq2, dk2, dv2 = ao.row_mask_attention_backward(q, k, v, dout, C, B, scale=0.3)
    assert np.abs(0.3 * dq1 - dq2).max() <= 1e-12 and np.abs(dk1 - dk2).max() <= 1e-12
    assert np.abs(dv1 - dv2).max() <= 1e-12


def test_round_bf16_matches_torch_cast():
    """The oracle's bfloat16 rounding against torch's cast: random values over many exponents,
    exact ties (both parities of the kept mantissa bit), signed zeros, subnormals of bfloat16."""
    import torch

    rng = np.random.default_rng(0)
    x = (rng.standard_normal(20000) * np.exp2(rng.integers(-30, 30, 20000))).astype(np.float32)
    ties = np.array([0x3F808000, 0x3F818000, 0xBF808000, 0x3F80FFFF, 0x00008000, 0x00018000, 0x00000000, 0x80000000],
                    dtype=np.uint32).view(np.float32)
    x = np.concatenate([x, ties])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    got = ao.round_bf16(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_same_dtype_context_attention_is_near_the_exact_one():
    """The bfloat16-arithmetic evaluation of pytorch_context_attention stays within the tolerances
    stated for 16-bit outputs at the scale the targets are stated for (entries ~N(0,1)/8), and is
    an evaluation of the same function (not of something else) at unit scale."""
    rng = np.random.default_rng(1)
    B, H, Lq, Nc, D = 3, 2, 2, 300, 32
    for s, tol_o, tol_l in ((0.125, 2e-2, 1e-3), (1.0, 6e-2, 5e-2)):
        q, k, v = (ao.round_bf16(rng.standard_normal(sh) * s) for sh in ((B, H, Lq, D), (H, Nc, D), (H, Nc, D)))
        o1, l1 = ao.context_attention_same_dtype(q, k, v)
        o0, l0 = ao.context_attention(q, k, v)
        assert np.abs(o1 - o0).max() <= tol_o and np.abs(l1 - l0).max() <= tol_l
