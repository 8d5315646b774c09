"""Host-side checks that need no GPU: the shared library loads and exports every symbol
the header declares, argument validation returns before any launch, the package's
module tree has the reference's names, and the host logic raises the reference's errors."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    from ar_nanotabpfn_amd import _lib

    if not _lib.library_built():
        pytest.skip("libartab_attention.so not built (run __graft_entry__.build())")
    return _lib


def _declared(header_name):
    header = open(os.path.join(ROOT, "include", header_name)).read()
    return set(re.findall(r"\b(artab_[a-z_]+)\s*\(", header)) - {"artab_view"}


def _exported(path):
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True, text=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def test_library_exports_every_declared_symbol():
    L = _lib()
    declared = _declared("artab_attention.h")
    assert declared == set(L.SIGNATURES), (declared ^ set(L.SIGNATURES))
    lib = L.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.artab_version() == L.ABI_VERSION == 7
    assert lib.artab_status_string(0) == b"ok"


def test_drop_in_library_exports_nothing_but_the_declared_abi():
    """The drop-in library exports exactly the functions of include/artab_attention.h: no
    benchmark aid, no C++ symbol.  The benchmark library adds those of include/artab_bench.h."""
    L = _lib()
    assert _exported(L.LIB_PATH) == _declared("artab_attention.h")
    bench_only = _declared("artab_bench.h")
    assert bench_only == set(L.BENCH_SIGNATURES)
    assert _exported(L.BENCH_LIB_PATH) == _declared("artab_attention.h") | bench_only
    for name in bench_only:
        assert not hasattr(L.load(), name)


def test_tuning_overrides_are_explicit_and_restorable(monkeypatch):
    """Route overrides are set through the ABI; the environment is read when the library is
    loaded and never again."""
    L = _lib()
    lib = L.load()
    assert lib.artab_tuning_set(b"ARTAB_NO_SUCH_KEY", 1, 1) == L.ARTAB_ERR_UNSUPPORTED
    for key in L.TUNING_KEYS:
        assert L.tuning.get(key) is None or key in os.environ
    monkeypatch.setenv("ARTAB_SMALL", "0")  # after the load: must not be seen
    if "ARTAB_SMALL" not in os.environ or L.tuning.get("ARTAB_SMALL") is None:
        assert L.tuning.get("ARTAB_SMALL") is None
    with L.tuning(ARTAB_TILE_ROWS=32, ARTAB_DENSE_BELOW=0):
        assert L.tuning.get("ARTAB_TILE_ROWS") == 32 and L.tuning.get("ARTAB_DENSE_BELOW") == 0
        with L.tuning(ARTAB_TILE_ROWS=None):
            assert L.tuning.get("ARTAB_TILE_ROWS") is None
        assert L.tuning.get("ARTAB_TILE_ROWS") == 32
    assert L.tuning.get("ARTAB_TILE_ROWS") is None and L.tuning.get("ARTAB_DENSE_BELOW") is None


def test_workspace_query_is_host_only():
    lib = _lib().load()
    assert lib.artab_workspace_bytes(1024, 8, 2, 16384, 32, 0) > 0
    assert lib.artab_workspace_bytes(1024, 8, 2, 16384, 32, 2) == 0  # float32: portable kernel, no workspace
    assert lib.artab_workspace_bytes(0, 8, 2, 16384, 32, 0) == 0


def test_argument_validation_returns_before_launch():
    L = _lib()
    lib = L.load()
    v = L.ArtabView(0x1000, 64, 32, 32)  # never dereferenced: every call below fails validation
    r = ctypes.byref
    # decode: Lq outside {1,2}
    rc = lib.artab_decode_attention(r(v), r(v), r(v), r(v), r(v), None, None, r(v), 2, 2, 3, 8, 0, None, 4, 32, 0.0, 0,
                                    None, 0, 0, None)
    assert rc == L.ARTAB_ERR_BAD_SHAPE and b"Lq" in lib.artab_last_error()
    # decode: cache full
    rc = lib.artab_decode_attention(r(v), r(v), r(v), r(v), r(v), r(v), r(v), r(v), 2, 2, 2, 8, 4, None, 4, 32, 0.0, 0,
                                    None, 0, 0, None)
    assert rc == L.ARTAB_ERR_CAPACITY
    # context attention: empty context, unknown dtype, NULL q, oversized head_dim
    assert lib.artab_context_attention(r(v), r(v), r(v), r(v), None, 1, 1, 1, 0, 32, 0.0, 0, None, 0, 0, None) == L.ARTAB_ERR_BAD_SHAPE
    assert lib.artab_context_attention(r(v), r(v), r(v), r(v), None, 1, 1, 1, 4, 32, 0.0, 7, None, 0, 0, None) == L.ARTAB_ERR_UNSUPPORTED
    assert lib.artab_context_attention(None, r(v), r(v), r(v), None, 1, 1, 1, 4, 32, 0.0, 0, None, 0, 0, None) == L.ARTAB_ERR_NULL_POINTER
    assert lib.artab_context_attention(r(v), r(v), r(v), r(v), None, 1, 1, 1, 4, 512, 0.0, 0, None, 0, 0, None) == L.ARTAB_ERR_UNSUPPORTED
    # MFMA requested for a float32 problem
    assert lib.artab_context_attention(r(v), r(v), r(v), r(v), None, 1, 1, 1, 4, 32, 0.0, 2, None, 0, L.IMPL_MFMA, None) == L.ARTAB_ERR_UNSUPPORTED
    # prefill: cache given for only one of k/v
    assert lib.artab_prefill_attention(r(v), r(v), r(v), r(v), r(v), None, 1, 1, 1, 4, 32, 0.0, 0, 0, None) == L.ARTAB_ERR_NULL_POINTER
    # merge without lse
    assert lib.artab_merge_attention_outputs(r(v), None, r(v), None, r(v), 1, 1, 1, 32, 0, None) == L.ARTAB_ERR_NULL_POINTER
    # empty problems are a no-op success
    assert lib.artab_context_attention(r(v), r(v), r(v), r(v), None, 0, 1, 1, 4, 32, 0.0, 0, None, 0, 0, None) == 0
    # row-mask backward: no context, sections longer than the rows, missing statistics, MFMA for float32
    bwd = lambda lse, delta, B, R, Nc, Nb, dtype, impl: lib.artab_row_mask_attention_backward(  # noqa: E731
        r(v), r(v), r(v), r(v), r(v), lse, delta, r(v), r(v), r(v), B, 2, R, Nc, Nb, 1, 32, 0.0, dtype, impl, None)
    assert bwd(0x1000, 0x1000, 1, 10, 0, 2, 0, 0) == L.ARTAB_ERR_BAD_SHAPE
    assert bwd(0x1000, 0x1000, 1, 10, 8, 4, 0, 0) == L.ARTAB_ERR_BAD_SHAPE
    assert bwd(None, 0x1000, 1, 10, 4, 2, 0, 0) == L.ARTAB_ERR_NULL_POINTER
    assert bwd(0x1000, None, 1, 10, 4, 2, 0, 0) == L.ARTAB_ERR_NULL_POINTER
    assert bwd(0x1000, 0x1000, 1, 10, 4, 2, 2, L.IMPL_MFMA) == L.ARTAB_ERR_UNSUPPORTED
    assert bwd(0x1000, 0x1000, 0, 10, 4, 2, 0, 0) == 0


def test_status_to_exception_mapping():
    L = _lib()
    with pytest.raises(ValueError):
        L.check(L.ARTAB_ERR_BAD_SHAPE)
    with pytest.raises(ValueError):
        L.check(L.ARTAB_ERR_CAPACITY)
    with pytest.raises(RuntimeError):
        L.check(L.ARTAB_ERR_UNSUPPORTED)
    L.check(0)


def test_cpu_tensors_are_rejected_not_silently_computed():
    import ar_nanotabpfn_amd.attention_kernels as ak

    q, k = torch.zeros(1, 1, 1, 32), torch.zeros(1, 4, 32)
    for call in (
        lambda: ak.context_attention(q, k, k),
        lambda: ak.hybrid_attention(q, k, k, torch.zeros(1, 1, 2, 32), torch.zeros(1, 1, 2, 32)),
        lambda: ak.merge_attention_outputs(q, torch.zeros(1, 1, 1), q, torch.zeros(1, 1, 1)),
        lambda: ak.prefill_attention(q, q, q),
    ):
        with pytest.raises(RuntimeError):
            call()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "ar_nanotabpfn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".h", ".hip")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("no oracle", ""), f"{f} mentions the oracle"


def test_model_tree_and_state_dict_keys():
    from ar_nanotabpfn_amd.model import ARTabPFN

    torch.manual_seed(0)
    m = ARTabPFN(d_model=32, n_heads=2, n_layers=2, d_ff=48, num_features=3, buffer_size=4, num_components=3)
    keys = set(m.state_dict())
    assert {"embedder.x_embed.weight", "embedder.marker_embed.weight", "backbone.layers.1.attn_rows.out_proj.weight",
            "backbone.layers.0.attn_features.q_proj.weight", "backbone.layers.0.ff.2.bias", "backbone.layers.1.norm3.weight",
            "backbone.norm.bias", "head.head.2.weight", "head.mean_bias", "head.std_bias", "head.weight_bias",
            "ar_tokens"} <= keys
    assert len(keys) == 15 + 2 * 18
    assert m.ar_tokens.shape == (4, 32) and m.head.head[2].out_features == 9
    a = m.backbone.layers[0].attn_rows
    assert (a.n_heads, a.head_dim, a.scale) == (2, 16, 16 ** -0.5)
    # the training forward exists (forward only) and runs on the device kernels: CPU tensors raise
    from ar_nanotabpfn_amd.attention import create_dense_mask, create_row_mask

    rm = create_row_mask(2 + 4 + 16, 2, 4, device="cpu")
    assert (rm.num_rows, rm.context_len, rm.buffer_len, rm.attending_chunks) == (22, 2, 4, 2)  # 16 // (2 * 4)
    assert create_row_mask(22, 2, 4, device="cpu") is rm  # cached, as in attention.py:113-121
    z = torch.zeros
    with pytest.raises(RuntimeError):
        m(z(1, 2, 3), z(1, 2), z(1, 4, 3), z(1, 4), z(1, 16, 3), create_dense_mask(1, "cpu"), rm, y_target=z(1, 16))


def test_reference_checkpoint_format_loads(tmp_path):
    """The reference's training loop saves {"step", "model"} (train.py:336-343); with compile_model
    the embedder and the head carry an "_orig_mod." segment in their keys (train.py:233-235).
    from_checkpoint reads the sizes off the tensors, strips the segment and loads strictly."""
    from ar_nanotabpfn_amd.model import ARTabPFN

    torch.manual_seed(3)
    src = ARTabPFN(d_model=64, n_heads=4, n_layers=3, d_ff=96, num_features=2, buffer_size=7, num_components=4)
    sd = {}
    for k, v in src.state_dict().items():
        top, rest = k.split(".", 1) if "." in k else (k, "")
        sd[f"{top}._orig_mod.{rest}" if top in ("embedder", "head") else k] = v.clone()
    assert any("_orig_mod" in k for k in sd)
    path = tmp_path / "step_10.pt"
    torch.save({"step": 10, "model": sd}, path)

    model, step = ARTabPFN.from_checkpoint(str(path), n_heads=4, num_features=2)
    assert step == 10
    assert (model.d_model, model.buffer_size, len(model.backbone.layers)) == (64, 7, 3)
    assert model.head.mean_bias.shape[0] == 4 and model.backbone.layers[0].ff[0].out_features == 96
    for (ka, va), (kb, vb) in zip(src.state_dict().items(), model.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)
    # a bare state_dict works too; a foreign one is refused
    model2, step2 = ARTabPFN.from_checkpoint(src.state_dict(), n_heads=4)
    assert step2 is None and torch.equal(model2.ar_tokens, src.ar_tokens)
    with pytest.raises(ValueError):
        ARTabPFN.from_checkpoint({"w": torch.zeros(1)}, n_heads=4)
    with pytest.raises(ValueError):
        ARTabPFN.from_checkpoint(src.state_dict(), n_heads=5)


def test_embedder_mean_over_features_and_markers():
    from ar_nanotabpfn_amd.model import Embedder

    torch.manual_seed(1)
    e = Embedder(8)
    x, y = torch.randn(2, 3, 4), torch.randn(2, 3)
    per_feature = e.x_embed(x.unsqueeze(-1)).mean(dim=2)  # the reference's order of operations
    want = per_feature + e.y_embed(y.unsqueeze(-1)) + e.marker_embed.weight[1]
    torch.testing.assert_close(e.embed_context(x, y), want, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(e.embed_buffer(x, y), want - e.marker_embed.weight[1] + e.marker_embed.weight[2], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(e.embed_target(x), per_feature + e.marker_embed.weight[0], atol=1e-6, rtol=1e-6)


def test_head_against_torch_distributions():
    from ar_nanotabpfn_amd.model import MixtureGaussianHead

    torch.manual_seed(2)
    h = MixtureGaussianHead(16, 24, num_components=4)
    z, y = torch.randn(2, 5, 16), torch.randn(2, 5, 1)
    mean, std, weight, log_weight = h._parameterize(z)
    mix = torch.distributions.MixtureSameFamily(
        torch.distributions.Categorical(probs=weight[..., 0]),
        torch.distributions.Normal(mean[..., 0], std[..., 0]),
    )
    torch.testing.assert_close(h.log_likelihood(z, y), mix.log_prob(y[..., 0]), atol=1e-5, rtol=1e-5)
    assert std.min() >= 1e-3 and std.max() <= 2.0 + 1e-3
    s = h.sample(z, num_samples=3)
    assert s.shape == (2, 5, 3, 1)
    loss, *_ = h(z, y)
    torch.testing.assert_close(loss, -h.log_likelihood(z, y).mean(), atol=1e-6, rtol=1e-6)


def test_predictor_host_errors_and_state():
    """Conditions the reference raises before touching the attention kernels."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor
    from ar_nanotabpfn_amd.model import ARTabPFN

    m = ARTabPFN(d_model=32, n_heads=2, n_layers=1, d_ff=32, buffer_size=4, num_components=3)
    with pytest.raises(ValueError, match="Unsupported backend"):
        ARTabPFNPredictor.from_trained_model(m, backend="cuda_graphs")
    p = ARTabPFNPredictor.from_trained_model(m, backend="triton_shared_context")
    assert p.backend == "triton_shared_context" and p.ar_tokens is m.ar_tokens and p.embedder is m.embedder
    p.init_kv_cache(3, 0)  # device/dtype default to the backbone's parameters (inference.py:99-102)
    layer = m.backbone.layers[0]
    assert layer.k_ctx_cache.shape == (2, 0, 16) and layer.k_buf_cache.shape == (3, 2, 0, 16)
    assert layer.k_buf_cache.dtype == torch.float32
    with pytest.raises(ValueError, match="buffer cache exceeded"):
        p.transformer_decode(torch.zeros(3, 2, 32), commit=1)
    with pytest.raises(ValueError, match="N=1"):
        p.transformer_decode(torch.zeros(3, 3, 32), commit=0)
    with pytest.raises(ValueError, match="2\\*num_targets"):
        p._teacher_forcing_decode_shared(torch.zeros(3, 5, 32), 2)
    p2 = ARTabPFNPredictor.from_trained_model(m)  # default backend: per-dataset full cache
    assert p2.backend == "flex_attention"
    p2.init_kv_cache(2, 7)
    assert layer.k_cache.shape == (2, 2, 7, 16) and p2.max_buffer_len == 0
    p2.seq_len = 5
    p2.clear_cache()
    assert (p2.seq_len, p2.context_len, p2.buffer_len) == (0, 0, 0)


def test_mask_descriptors_are_cached():
    from ar_nanotabpfn_amd import attention as att

    att.clear_mask_cache()
    a = att.create_dense_mask(5, "cpu")
    assert a is att.create_dense_mask(5, "cpu") and a.seq_len == 5
    assert att.create_context_self_attention_mask(9, "cpu").seq_len == 9
    att.clear_mask_cache()
    assert att.create_dense_mask(5, "cpu") is not a
    r = att.create_row_mask(10, 4, 2)  # target_len 4 -> 4 // (2 * 2) = 1 attending chunk
    assert r.attending_chunks == 1 and r is att.create_row_mask(10, 4, 2)
    dense = r.dense()
    assert dense.shape == (10, 10) and bool(dense[:, :4].all()) and not bool(dense[:, 6:].any())
    assert dense[6].tolist() == [True] * 5 + [False] * 5 and dense[8].tolist() == [True] * 4 + [False] * 6
