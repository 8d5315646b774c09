"""End-to-end parity of the predictor (model in PyTorch-ROCm, attention in HIP) against
the numpy oracle and the reference-made fixture.  Tolerance of the build's target:
1e-3 nats per target on the log-density."""

import os

import numpy as np
import pytest
import torch

from oracle import model_oracle as mo
from oracle import torch_attention_f32 as tref
from tests.helpers import max_abs, to_np

pytestmark = pytest.mark.gpu

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "tiny_model.npz")


def _build(cfg, device, dtype=torch.float32, seed=0):
    from ar_nanotabpfn_amd.model import ARTabPFN

    torch.manual_seed(seed)
    model = ARTabPFN(**cfg).eval()
    g = torch.Generator().manual_seed(seed + 1)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name or name.endswith("bias") or "marker" in name:
                p.add_(0.2 * torch.randn(p.shape, generator=g))
    return model.to(device=device, dtype=dtype)


def _oracle(model, n_heads):
    sd = {k: v.detach().float().cpu().numpy() for k, v in model.state_dict().items()}
    return mo.OracleModel(sd, n_heads)


def _gp_dataset(seed, B, Nc, Nt, lengthscale=0.5, noise=0.1):
    """configs[0] data: x ~ U(-1,1) in R^1, y from a GP with an RBF kernel; one dataset
    whose context is shared by all B trajectories."""
    r = np.random.default_rng(seed)
    x = r.uniform(-1, 1, size=(Nc + Nt, 1))
    K = np.exp(-0.5 * (x - x.T) ** 2 / lengthscale**2) + noise**2 * np.eye(Nc + Nt)
    y = np.linalg.cholesky(K) @ r.normal(size=Nc + Nt)
    rep = lambda a: np.repeat(a[None], B, axis=0).astype(np.float32)  # noqa: E731
    return rep(x[:Nc]), rep(y[:Nc]), rep(x[Nc:]), rep(y[Nc:])


def _t(a, device, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=dtype)


# ----- reference-made fixture through the device path ------------------------------------------


@pytest.fixture(scope="module")
def fx():
    data = np.load(FIXTURE, allow_pickle=False)
    sd = {k[3:]: torch.from_numpy(data[k]) for k in data.files if k.startswith("w::")}
    cfg = dict(zip(("d_model", "n_heads", "n_layers", "d_ff", "num_features", "buffer_size", "num_components"),
                   (int(v) for v in data["cfg"])))
    return data, sd, cfg


def _fixture_model(fx, device):
    from ar_nanotabpfn_amd.model import ARTabPFN

    data, sd, cfg = fx
    model = ARTabPFN(**cfg).eval()
    missing, unexpected = model.load_state_dict(sd, strict=True)
    assert not missing and not unexpected
    return model.to(device)


@pytest.mark.parametrize("backend,key", [("flex_attention", "ll_per_dataset"), ("triton_shared_context", "ll_shared")])
def test_log_density_matches_reference_fixture(device, fx, backend, key):
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    data, _, _ = fx
    model = _fixture_model(fx, device)
    B = data["x_ctx"].shape[0]
    xc, yc = data["x_ctx"], data["y_ctx"]
    if backend == "triton_shared_context":
        xc, yc = np.repeat(xc[0:1], B, axis=0), np.repeat(yc[0:1], B, axis=0)
    pred = ARTabPFNPredictor.from_trained_model(model, backend=backend)
    ll = pred.evaluate_joint_density(_t(xc, device), _t(yc, device), _t(data["x_tgt"], device), _t(data["y_tgt"], device))
    assert ll.shape == data[key].shape
    assert max_abs(to_np(ll), data[key]) <= 1e-4  # float32 model, float32 reference values


@pytest.mark.parametrize("backend,key", [("flex_attention", "z_decode_per_dataset"), ("triton_shared_context", "z_decode_shared")])
def test_fixed_buffer_decode_matches_reference_fixture(device, fx, backend, key):
    """Step-wise decode with prescribed buffer values (tests/test_triton_gpu.py:126-165)."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    data, _, _ = fx
    model = _fixture_model(fx, device)
    B, Nc = data["x_ctx"].shape[:2]
    Nt = data["x_tgt"].shape[1]
    xc, yc = data["x_ctx"], data["y_ctx"]
    if backend == "triton_shared_context":
        xc, yc = np.repeat(xc[0:1], B, axis=0), np.repeat(yc[0:1], B, axis=0)
    pred = ARTabPFNPredictor.from_trained_model(model, backend=backend)
    x_tgt, y_tgt = _t(data["x_tgt"], device), _t(data["y_tgt"], device)
    pred.init_kv_cache(B, Nt if backend == "triton_shared_context" else Nc + Nt, device, torch.float32)
    pred.prefill_context(_t(xc, device), _t(yc, device))
    zs = []
    for t in range(Nt):
        emb_t = pred.embedder.embed_target(x_tgt[:, t : t + 1])
        if t == 0:
            emb, commit = emb_t, 0
        else:
            emb_b = pred.embedder.embed_buffer(x_tgt[:, t - 1 : t], y_tgt[:, t - 1 : t])
            emb_b = emb_b + pred.ar_tokens[t % pred.ar_tokens.shape[0]]
            emb, commit = torch.cat([emb_b, emb_t], dim=1), 1
        zs.append(pred.transformer_decode(emb, commit=commit)[:, -1:])
    z = torch.cat(zs, dim=1)
    assert max_abs(to_np(z), data[key]) <= 1e-4
    assert pred.buffer_len == (Nt - 1 if backend == "triton_shared_context" else 0)
    assert pred.seq_len == Nc + Nt - 1


# ----- configs[0]: tiny float32 model, 64 context rows, 16 targets, 8 trajectories -----------------

CFG0 = dict(d_model=128, n_heads=4, n_layers=4, d_ff=256, num_features=1, buffer_size=32, num_components=5)


@pytest.mark.parametrize("backend,obackend", [("triton_shared_context", "shared"), ("flex_attention", "per_dataset")])
def test_config0_log_density_vs_oracle(device, backend, obackend):
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    model = _build(CFG0, device)
    xc, yc, xt, yt = _gp_dataset(1, B=8, Nc=64, Nt=16)
    pred = ARTabPFNPredictor.from_trained_model(model, backend=backend)
    ll = pred.evaluate_joint_density(_t(xc, device), _t(yc, device), _t(xt, device), _t(yt, device))
    ref = mo.OraclePredictor(_oracle(model, CFG0["n_heads"]), obackend).evaluate_joint_density(xc, yc, xt, yt)
    assert ll.shape == (8, 16) and torch.isfinite(ll).all()
    assert max_abs(to_np(ll), ref) <= 1e-3  # nats per target


def test_config0_sampling_shapes_and_cache_state(device):
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    model = _build(CFG0, device)
    xc, yc, xt, _ = _gp_dataset(1, B=8, Nc=64, Nt=16)
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    torch.manual_seed(0)
    y = pred.sample_sequence(_t(xc, device), _t(yc, device), _t(xt, device))
    assert y.shape == (8, 16) and torch.isfinite(y).all()
    assert pred.context_len == 64 and pred.buffer_len == 15 and pred.seq_len == 79
    layer = model.backbone.layers[0]
    assert layer.k_ctx_cache.shape == (4, 64, 32) and layer.k_buf_cache.shape == (8, 4, 16, 32)
    assert torch.all(layer.k_buf_cache[:, :, 15:] == 0)  # last slot never written
    assert not torch.all(layer.k_buf_cache[:, :, :15] == 0)
    # trajectories share the context but sample independently
    assert (y[0] - y[1]).abs().max() > 0


def test_config0_decode_equals_teacher_forcing(device):
    """With buffer row j carrying ar_tokens[j % bs] in both, the decode steps reproduce the
    target rows of the teacher-forced pass (the identity the two kernels must share)."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    model = _build(CFG0, device)
    xc, yc, xt, yt = (_t(a, device) for a in _gp_dataset(3, B=4, Nc=64, Nt=16))
    Nt = 16
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    pred.init_kv_cache(4, Nt, device, torch.float32)
    pred.prefill_context(xc, yc)
    z_tf = pred._teacher_forcing_decode_shared(pred._teacher_forcing_embedding(xt, yt), Nt)[:, Nt:]
    zs = []
    for t in range(Nt):
        emb_t = pred.embedder.embed_target(xt[:, t : t + 1])
        if t == 0:
            emb, commit = emb_t, 0
        else:
            emb_b = pred.embedder.embed_buffer(xt[:, t - 1 : t], yt[:, t - 1 : t]) + pred.ar_tokens[(t - 1) % 32]
            emb, commit = torch.cat([emb_b, emb_t], dim=1), 1
        zs.append(pred.transformer_decode(emb, commit)[:, -1:])
    assert max_abs(to_np(torch.cat(zs, dim=1)), to_np(z_tf)) <= 1e-4


def test_prefill_cache_matches_projections(device):
    """tests/test_inference_vs_forward.py:55-99: cached K/V equal the layer's own
    projections of its input, shape (B,H,Nc,Dh)."""
    from ar_nanotabpfn_amd.attention import create_dense_mask
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=32, n_heads=2, n_layers=2, d_ff=64, num_features=3, buffer_size=4, num_components=3)
    model = _build(cfg, device)
    B, Nc = 2, 10
    g = torch.Generator().manual_seed(5)
    xc, yc = torch.randn(B, Nc, 3, generator=g).to(device), torch.randn(B, Nc, generator=g).to(device)
    pred = ARTabPFNPredictor.from_trained_model(model)
    pred.init_kv_cache(B, Nc, device, torch.float32)
    pred.prefill_context(xc, yc)
    emb = model.embedder.embed_context(xc, yc).unsqueeze(2)
    _, kvs = model.backbone(emb, create_dense_mask(1, device), create_dense_mask(Nc, device))
    for layer, (k, v) in zip(model.backbone.layers, kvs):
        assert layer.k_cache.shape == (B, 2, Nc, 16)
        assert max_abs(to_np(layer.k_cache), to_np(k)) <= 1e-5
        assert max_abs(to_np(layer.v_cache), to_np(v)) <= 1e-5


# ----- bf16, configs[2]-like: same model, only the attention implementation differs -----------------

CFG2 = dict(d_model=256, n_heads=8, n_layers=12, d_ff=256, num_features=10, buffer_size=128, num_components=5)


def _mlp_prior(seed, B, N, F=10, width=64, noise=0.1):
    """configs[2] data: x ~ N(0,I), y = tanh-MLP(x) (F->64->64->1, W ~ N(0,1/fan_in), no
    bias) + N(0, 0.1^2); one independent MLP per dataset; y standardised by context stats."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, N, F, generator=g)
    w1 = torch.randn(B, F, width, generator=g) / F**0.5
    w2 = torch.randn(B, width, width, generator=g) / width**0.5
    w3 = torch.randn(B, width, 1, generator=g) / width**0.5
    y = (torch.tanh(torch.tanh(x @ w1) @ w2) @ w3).squeeze(-1) + noise * torch.randn(B, N, generator=g)
    return x, y


# Absolute bounds of the bf16 12-layer log-density against the exact (float64) evaluation of the
# same bf16 weights on the same bf16 inputs, nats per target.  Measured on MI355X (the values the
# test prints), product path: mean 1.13e-2 / 1.05e-2 / 1.17e-2 and max 0.154 / 0.168 / 0.619 at
# B=8 per-dataset / B=8 shared / B=64 per-dataset.  A float32-attention run of the same model
# (mean 1.15e-2 / 1.07e-2 / 1.18e-2, max 0.154 / 0.259 / 0.443) and a run with the fused layer
# kernels switched off (mean 1.21e-2 / 1.04e-2 / 1.17e-2, max 0.212 / 0.259 / 0.440) miss the
# exact value by the same amount: the floor is the 8-bit rounding of every activation, twelve
# layers deep, and the maximum over 8192 targets is the tail of a density with small std.
# The bounds leave a factor of about 1.7 over the largest value seen.
BF16_DLOGP_MEAN_MAX = 2.0e-2
BF16_DLOGP_P99_MAX = 2.0e-1
BF16_DLOGP_MAX_MAX = 1.0


@pytest.mark.parametrize("backend,B", [("flex_attention", 8), ("triton_shared_context", 8), ("flex_attention", 64)])
def test_bf16_log_density_hip_vs_float32_attention(device, backend, B, monkeypatch):
    """configs[2] (B=64 datasets x 512 context + 128 target rows, 12 layers, bf16) and its B=8
    cut on both cache layouts.  Four evaluations of one model on one input: HIP attention + fused
    layer kernels (the product path), HIP attention + unfused layers, float32 PyTorch attention +
    unfused layers, and the float64 oracle as arbiter."""
    import ar_nanotabpfn_amd.inference as inf
    import ar_nanotabpfn_amd.model as model_mod
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    Nc, Nt = 512, 128
    model = _build(CFG2, device, dtype=torch.bfloat16, seed=0)
    x, y = _mlp_prior(2, B, Nc + Nt)
    mu, sd = y[:, :Nc].mean(1, keepdim=True), y[:, :Nc].std(1, keepdim=True)
    y = (y - mu) / sd
    if backend == "triton_shared_context":
        x[:, :Nc], y[:, :Nc] = x[0:1, :Nc], y[0:1, :Nc]
    x, y = x.to(device, torch.bfloat16), y.to(device, torch.bfloat16)
    args = (x[:, :Nc], y[:, :Nc], x[:, Nc:], y[:, Nc:])
    pred = ARTabPFNPredictor.from_trained_model(model, backend=backend)
    assert all(layer.fused_for(x) for layer in model.backbone.layers)
    ll_hip = pred.evaluate_joint_density(*args).float()

    # the same HIP attention with the fused layer kernels switched off: an error inside them
    # cannot hide in both operands of the comparisons below
    monkeypatch.setattr(model_mod, "layer_fusable", lambda *a, **k: False)
    assert not any(layer.fused_for(x) for layer in model.backbone.layers)
    ll_unfused = ARTabPFNPredictor.from_trained_model(model, backend=backend).evaluate_joint_density(*args).float()

    class Ref:  # the same module namespace the predictor calls, float32 attention inside
        prefill_attention = staticmethod(tref.prefill_attention)
        decode_attention = staticmethod(tref.decode_attention)
        teacher_forcing_attention = staticmethod(tref.teacher_forcing_attention)
        hybrid_teacher_forcing_attention = staticmethod(tref.hybrid_teacher_forcing_attention)

    monkeypatch.setattr(inf, "ak", Ref)
    ll_ref = ARTabPFNPredictor.from_trained_model(model, backend=backend).evaluate_joint_density(*args).float()

    # arbiter: exact (float64) evaluation of the same bf16 weights on the same bf16 inputs
    obackend = "shared" if backend == "triton_shared_context" else "per_dataset"
    ll_true = mo.OraclePredictor(_oracle(model, CFG2["n_heads"]), obackend).evaluate_joint_density(
        *(to_np(a) for a in args)
    )
    err_hip = np.abs(to_np(ll_hip) - ll_true)
    err_unf = np.abs(to_np(ll_unfused) - ll_true)
    err_ref = np.abs(to_np(ll_ref) - ll_true)
    diff = (ll_hip - ll_ref).abs()
    print(f"\n[{backend} B={B}] |dlogp| per target vs exact: hip+fused mean {err_hip.mean():.3e} "
          f"p99 {np.quantile(err_hip, 0.99):.3e} max {err_hip.max():.3e}; "
          f"hip+unfused mean {err_unf.mean():.3e} max {err_unf.max():.3e}; "
          f"f32attn+unfused mean {err_ref.mean():.3e} max {err_ref.max():.3e}; "
          f"hip-vs-f32attn mean {diff.mean().item():.3e} max {diff.max().item():.3e}")
    assert torch.isfinite(ll_hip).all() and torch.isfinite(ll_unfused).all()
    # absolute: the product path against the exact value
    assert err_hip.mean() <= BF16_DLOGP_MEAN_MAX
    assert np.quantile(err_hip, 0.99) <= BF16_DLOGP_P99_MAX
    assert err_hip.max() <= BF16_DLOGP_MAX_MAX
    # relative: neither the HIP attention nor the fused layer kernels add anything to the floor
    # that a float32-attention / unfused run of the same bf16 model shows
    assert err_hip.mean() <= 1.25 * err_ref.mean() + 1e-3
    assert err_hip.max() <= 1.5 * err_ref.max() + 1e-2
    assert err_hip.mean() <= 1.25 * err_unf.mean() + 1e-3
    assert err_unf.mean() <= 1.25 * err_ref.mean() + 1e-3
    assert diff.mean().item() <= 2.5e-2


@pytest.mark.parametrize("backend", ["flex_attention", "triton_shared_context"])
def test_config2_shape_float32_log_density_within_1e3_nats(device, backend):
    """The configs[2] shape (512 context + 128 target rows, 12 layers, d_model 256, 8 heads) with a
    float32 model, B=8 datasets, through the device path against the float64 oracle: the case in
    which the end-to-end tolerance of 1e-3 nats per target is well defined (a bf16 model misses the
    exact value by 1e-2 whatever computes its attention: test_bf16_log_density_hip_vs_float32_attention).
    The comparison the reference makes between its two backends at 5e-3
    (tests/test_triton_joint_density.py:163-210), here against the exact value."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    B, Nc, Nt = 8, 512, 128
    model = _build(CFG2, device, dtype=torch.float32, seed=0)
    x, y = _mlp_prior(2, B, Nc + Nt)
    y = (y - y[:, :Nc].mean(1, keepdim=True)) / y[:, :Nc].std(1, keepdim=True)
    if backend == "triton_shared_context":
        x[:, :Nc], y[:, :Nc] = x[0:1, :Nc], y[0:1, :Nc]
    x, y = x.to(device), y.to(device)
    args = (x[:, :Nc], y[:, :Nc], x[:, Nc:], y[:, Nc:])
    ll = ARTabPFNPredictor.from_trained_model(model, backend=backend).evaluate_joint_density(*args)
    obackend = "shared" if backend == "triton_shared_context" else "per_dataset"
    ll_true = mo.OraclePredictor(_oracle(model, CFG2["n_heads"]), obackend).evaluate_joint_density(*(to_np(a) for a in args))
    err = np.abs(to_np(ll) - ll_true)
    print(f"\n[{backend}] float32 configs[2] shape, B={B}: |dlogp| per target mean {err.mean():.3e} max {err.max():.3e}")
    assert ll.shape == (B, Nt) and torch.isfinite(ll).all()
    assert err.max() <= 1e-3


def test_torch_attention_ref_against_oracle(device):
    """The float32 PyTorch restatement used above equals the numpy oracle."""
    from oracle import attention_oracle as ao
    from tests.helpers import randn

    B, H, Nt, Nc, D = 2, 2, 5, 9, 16
    q = randn((B, H, 2 * Nt, D), 1, torch.float32)
    kc, vc = randn((H, Nc, D), 2, torch.float32), randn((H, Nc, D), 3, torch.float32)
    kb, vb = randn((B, H, Nt, D), 4, torch.float32), randn((B, H, Nt, D), 5, torch.float32)
    out = tref.teacher_forcing_attention(q, kc, vc, kb, vb, Nt)
    ref = ao.hybrid_teacher_forcing_attention(to_np(q), to_np(kc), to_np(vc), to_np(kb), to_np(vb), Nt)
    assert max_abs(to_np(out), ref) <= 1e-5
    cache_k, cache_v = torch.zeros(B, H, 8, D), torch.zeros(B, H, 8, D)
    cache_k[:, :, :3], cache_v[:, :, :3] = kb[:, :, :3], vb[:, :, :3]
    out = tref.decode_attention(q[:, :, :2], kc, vc, cache_k, cache_v, 3, kb[:, :, 3:4], vb[:, :, 3:4])
    ref, _, _ = ao.decode_step_attention(to_np(q[:, :, :2]), to_np(kc), to_np(vc), to_np(kb[:, :, :3]),
                                         to_np(vb[:, :, :3]), to_np(kb[:, :, 3:4]), to_np(vb[:, :, 3:4]))
    assert max_abs(to_np(out), ref) <= 1e-5
    assert torch.equal(cache_k[:, :, 3], kb[:, :, 3])


# ----- recorded HIP graph vs Python loop -------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_graph_replayed_sampling_equals_python_loop(device, dtype, monkeypatch):
    """The recorded step must do exactly what the Python loop does.  Sampling is made
    deterministic (mixture mean of the heaviest component) so the two runs can be compared;
    several calls in a row exercise graph reuse with fresh inputs."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor
    from ar_nanotabpfn_amd.model import MixtureGaussianHead

    def det_sample(self, z, num_samples=1):
        mean, std, weight, _ = self._parameterize(z)
        idx = weight.argmax(dim=2, keepdim=True)
        return torch.gather(mean, 2, idx).permute(0, 1, 3, 2) + 0.1 * torch.gather(std, 2, idx).permute(0, 1, 3, 2)

    monkeypatch.setattr(MixtureGaussianHead, "sample", det_sample)
    cfg = dict(d_model=64, n_heads=2, n_layers=3, d_ff=64, num_features=3, buffer_size=5, num_components=4)
    model = _build(cfg, device, dtype=dtype)
    B, Nc, Nt = 16, 40, 9
    pred_g = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    for seed in (0, 1, 2):
        g = torch.Generator().manual_seed(seed)
        xc = torch.randn(1, Nc, 3, generator=g).expand(B, -1, -1).to(device, dtype)
        yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, dtype)
        xt = torch.randn(B, Nt, 3, generator=g).to(device, dtype)
        pred_g.use_hip_graph = True
        y_graph = pred_g.sample_sequence(xc, yc, xt)
        caches_g = [(l.k_buf_cache.clone(), l.v_buf_cache.clone()) for l in model.backbone.layers]
        assert pred_g.buffer_len == Nt - 1 and pred_g.seq_len == Nc + Nt - 1
        pred_g.use_hip_graph = False
        y_loop = pred_g.sample_sequence(xc, yc, xt)
        assert y_graph.shape == (B, Nt) and torch.isfinite(y_graph).all()
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert max_abs(to_np(y_graph), to_np(y_loop)) <= tol
        for (kg, vg), l in zip(caches_g, model.backbone.layers):
            assert max_abs(to_np(kg), to_np(l.k_buf_cache)) <= tol and max_abs(to_np(vg), to_np(l.v_buf_cache)) <= tol
    assert pred_g._graph_state is not None and pred_g._graph_state.graph is not None


def test_graph_sampling_in_concurrent_groups_equals_one_group(device, monkeypatch):
    """Trajectories sampled as several groups, each replaying its own recorded step on its own
    stream with its own scratch memory, against all of them in one group: same values, same
    caches (deterministic head; bf16; the groups are uneven on purpose)."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor
    from ar_nanotabpfn_amd.model import MixtureGaussianHead

    def det_sample(self, z, num_samples=1):
        mean, std, weight, _ = self._parameterize(z)
        idx = weight.argmax(dim=2, keepdim=True)
        return torch.gather(mean, 2, idx).permute(0, 1, 3, 2) + 0.1 * torch.gather(std, 2, idx).permute(0, 1, 3, 2)

    monkeypatch.setattr(MixtureGaussianHead, "sample", det_sample)
    cfg = dict(d_model=128, n_heads=4, n_layers=3, d_ff=128, num_features=3, buffer_size=5, num_components=4)
    model = _build(cfg, device, dtype=torch.bfloat16)
    B, Nc, Nt = 70, 2100, 9  # long enough for a split context (partials in per-group scratch)
    g = torch.Generator().manual_seed(5)
    xc = torch.randn(1, Nc, 3, generator=g).expand(B, -1, -1).to(device, torch.bfloat16)
    yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, torch.bfloat16)
    xt = torch.randn(B, Nt, 3, generator=g).to(device, torch.bfloat16)
    results = {}
    for chains in (1, 3):
        pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
        pred.fuse_step_tail = False  # the deterministic head stands in for the sampler
        pred.decode_chains, pred.min_chain_batch = chains, 8
        for _ in range(2):  # second call: recorded graphs are reused
            y = pred.sample_sequence(xc, yc, xt)
        assert len(pred._graph_state.chains) == chains
        results[chains] = (y, [(l.k_buf_cache.clone(), l.v_buf_cache.clone()) for l in model.backbone.layers])
    y1, c1 = results[1]
    y3, c3 = results[3]
    assert y3.shape == (B, Nt) and torch.isfinite(y3).all()
    assert max_abs(to_np(y1), to_np(y3)) <= 2e-2
    for (k1, v1), (k3, v3) in zip(c1, c3):
        assert max_abs(to_np(k1), to_np(k3)) <= 2e-2 and max_abs(to_np(v1), to_np(v3)) <= 2e-2


def test_graph_sampling_with_random_head_is_finite_and_varied(device):
    """The real sampler (multinomial + normal draws) inside the recorded graph: every
    replay must draw fresh numbers."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    model = _build(CFG0, device)
    xc, yc, xt, _ = _gp_dataset(1, B=8, Nc=64, Nt=16)
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    torch.manual_seed(0)
    y1 = pred.sample_sequence(_t(xc, device), _t(yc, device), _t(xt, device))
    y2 = pred.sample_sequence(_t(xc, device), _t(yc, device), _t(xt, device))
    assert torch.isfinite(y1).all() and torch.isfinite(y2).all()
    assert (y1 - y2).abs().max() > 0          # a second call draws different samples
    assert (y1[0] - y1[1]).abs().max() > 0    # trajectories differ
    assert y1.std(dim=0).min() > 0            # every step drew fresh numbers across trajectories


# ----- error behaviour -------------------------------------------------------------------------------


def test_predictor_errors(device):
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=32, n_heads=2, n_layers=1, d_ff=32, num_features=2, buffer_size=4, num_components=3)
    model = _build(cfg, device)
    with pytest.raises(ValueError):
        ARTabPFNPredictor.from_trained_model(model, backend="nope")
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    pred.init_kv_cache(2, 1, device, torch.float32)
    pred.prefill_context(torch.zeros(2, 5, 2, device=device), torch.zeros(2, 5, device=device))
    emb = torch.zeros(2, 2, 32, device=device)
    pred.transformer_decode(emb, commit=1)
    with pytest.raises(ValueError):  # buffer cache full (inference.py:247-250)
        pred.transformer_decode(emb, commit=1)
    with pytest.raises(ValueError):  # N not in {1,2} (inference.py:765-768)
        pred.transformer_decode(torch.zeros(2, 3, 32, device=device), commit=0)
    with pytest.raises(ValueError):  # N != 2*Nt (inference.py:855-856)
        pred._teacher_forcing_decode_shared(torch.zeros(2, 5, 32, device=device), 2)


def test_graph_sampling_with_fused_step_tail_equals_python_loop(device, monkeypatch):
    """The recorded step with the one-launch tail (norm + head + draw + next embedding) against the
    Python loop of autoregressive_decode.  Both are made deterministic the same way: component 0
    (uniform variate 0) and a fixed normal variate."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor
    from ar_nanotabpfn_amd.model import MixtureGaussianHead

    def det_sample(self, z, num_samples=1):
        mean, std, _, _ = self._parameterize(z)
        return (mean[:, :, 0:1] + 0.3 * std[:, :, 0:1]).permute(0, 1, 3, 2)

    def det_variates(rand_u, rand_n):
        rand_u.zero_()
        rand_n.fill_(0.3)

    monkeypatch.setattr(MixtureGaussianHead, "sample", det_sample)
    monkeypatch.setattr(ARTabPFNPredictor, "_draw_step_variates", staticmethod(det_variates))
    cfg = dict(d_model=128, n_heads=4, n_layers=3, d_ff=128, num_features=3, buffer_size=5, num_components=4)
    model = _build(cfg, device, dtype=torch.bfloat16)
    B, Nc, Nt = 48, 40, 9
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    for seed in (0, 1):
        g = torch.Generator().manual_seed(seed)
        xc = torch.randn(1, Nc, 3, generator=g).expand(B, -1, -1).to(device, torch.bfloat16)
        yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, torch.bfloat16)
        xt = torch.randn(B, Nt, 3, generator=g).to(device, torch.bfloat16)
        pred.use_hip_graph = True
        y_graph = pred.sample_sequence(xc, yc, xt)
        assert pred._graph_state.tail is not None
        caches_g = [(l.k_buf_cache.clone(), l.v_buf_cache.clone()) for l in model.backbone.layers]
        pred.use_hip_graph = False
        y_loop = pred.sample_sequence(xc, yc, xt)
        assert y_graph.shape == (B, Nt) and torch.isfinite(y_graph).all()
        # small differences feed back through the sampled values: a few bf16 ulps per step
        assert max_abs(to_np(y_graph), to_np(y_loop)) <= 6e-2
        for (kg, vg), l in zip(caches_g, model.backbone.layers):
            assert max_abs(to_np(kg), to_np(l.k_buf_cache)) <= 6e-2 and max_abs(to_np(vg), to_np(l.v_buf_cache)) <= 6e-2
        pred.fuse_step_tail = False
        pred.use_hip_graph = True
        y_unfused = pred.sample_sequence(xc, yc, xt)
        assert pred._graph_state.tail is None
        assert max_abs(to_np(y_unfused), to_np(y_loop)) <= 6e-2
        pred.fuse_step_tail = True


def test_graph_sampling_fused_tail_law(device):
    """Real variates: two calls differ, trajectories differ, and the first-step marginal of the
    fused path agrees with the Python loop's in mean and spread (same context, many trajectories)."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=128, n_heads=4, n_layers=2, d_ff=128, num_features=1, buffer_size=8, num_components=5)
    model = _build(cfg, device, dtype=torch.bfloat16)
    xc, yc, xt, _ = _gp_dataset(1, B=1, Nc=32, Nt=4)
    B = 4096
    xc, yc, xt = (_t(np.repeat(a, B, axis=0), device).to(torch.bfloat16) for a in (xc, yc, xt))
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    torch.manual_seed(0)
    y1 = pred.sample_sequence(xc, yc, xt).float()
    assert pred._graph_state.tail is not None
    y2 = pred.sample_sequence(xc, yc, xt).float()
    pred.use_hip_graph = False
    y3 = pred.sample_sequence(xc, yc, xt).float()
    assert torch.isfinite(y1).all() and (y1 - y2).abs().max() > 0 and (y1[0] - y1[1]).abs().max() > 0
    for col in range(1, 4):  # columns 1.. come from the fused tail in y1/y2, from head.sample in y3
        s = float(y3[:, col].std())
        assert abs(float(y1[:, col].mean() - y3[:, col].mean())) <= 6 * s / B ** 0.5 + 1e-2
        assert abs(float(y1[:, col].std()) - s) <= 0.1 * s + 1e-2


def test_layer_by_layer_methods_equal_the_fused_stack(device):
    """The reference-named per-layer methods (one layer = pre, attention, finish) against the
    predictor's own pass over the stack, which fuses layer boundaries: teacher forcing on the
    shared layout and one decode step, bf16."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=128, n_heads=4, n_layers=3, d_ff=128, num_features=2, buffer_size=4, num_components=3)
    model = _build(cfg, device, dtype=torch.bfloat16)
    B, Nc, Nt = 6, 48, 5
    g = torch.Generator().manual_seed(3)
    xc = torch.randn(1, Nc, 2, generator=g).expand(B, -1, -1).to(device, torch.bfloat16)
    yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, torch.bfloat16)
    xt = torch.randn(B, Nt, 2, generator=g).to(device, torch.bfloat16)
    yt = torch.randn(B, Nt, generator=g).to(device, torch.bfloat16)
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    pred.init_kv_cache(B, Nt, device, torch.bfloat16)
    pred.prefill_context(xc, yc)
    emb = pred._teacher_forcing_embedding(xt, yt)
    z_stack = pred._teacher_forcing_decode_shared(emb, Nt)
    x = emb
    for layer in model.backbone.layers:
        x = pred._layer_teacher_forcing_shared(layer, x, Nt)
    z_layers = model.backbone.norm(x)
    assert max_abs(to_np(z_stack), to_np(z_layers)) <= 2e-2

    # one [buffer, target] decode step, twice from the same cache state
    step = torch.cat([model.embedder.embed_buffer(xt[:, 0:1], yt[:, 0:1]) + model.ar_tokens[1],
                      model.embedder.embed_target(xt[:, 1:2])], dim=1)
    z1 = pred.transformer_decode(step, commit=1)
    caches = [(l.k_buf_cache.clone(), l.v_buf_cache.clone()) for l in model.backbone.layers]
    pred.buffer_len = 0
    x = step
    for layer in model.backbone.layers:
        x = pred._layer_decode_with_cache_shared(layer, x, 1)
    z2 = model.backbone.norm(x)
    assert max_abs(to_np(z1), to_np(z2)) <= 2e-2
    for (kc, vc), l in zip(caches, model.backbone.layers):
        assert max_abs(to_np(kc[:, :, 0]), to_np(l.k_buf_cache[:, :, 0])) <= 2e-2


def test_graph_sampling_ordered_by_counters_equals_event_ordered(device):
    """The recorded decode step with its two streams ordered by device-side counters against the
    same step ordered by events: same variates in, same predictions and caches out (bf16, the
    fused step tail, several steps per graph and a one-step remainder)."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=128, n_heads=4, n_layers=3, d_ff=128, num_features=3, buffer_size=5, num_components=4)
    model = _build(cfg, device, dtype=torch.bfloat16)
    B, Nc, Nt = 70, 2100, 11
    g = torch.Generator().manual_seed(5)
    xc = torch.randn(1, Nc, 3, generator=g).expand(B, -1, -1).to(device, torch.bfloat16)
    yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, torch.bfloat16)
    xt = torch.randn(B, Nt, 3, generator=g).to(device, torch.bfloat16)
    results = {}
    for ordered in (False, True):
        pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
        pred.counter_ordering = ordered
        for _ in range(2):  # second call: recorded graphs are reused
            torch.manual_seed(11)
            y = pred.sample_sequence(xc, yc, xt)
        st = pred._graph_state.chains[0]
        if ordered:
            if st.order is None:
                pytest.skip("the two streams are served by one hardware queue here")
            assert pred.counter_ordering and st.order.failed() == 0
            # one signal per layer and step: two calls of sample_sequence, and the one replay of
            # each recorded graph (one step, steps_per_graph steps) when they were recorded
            n_steps = 2 * (Nt - 1) + 1 + pred.steps_per_graph
            assert st.graph_many is not None
            assert st.order.state[0].item() == st.order.state[32].item() == n_steps * len(model.backbone.layers)
        else:
            assert st.order is None
        results[ordered] = (y, [(l.k_buf_cache.clone(), l.v_buf_cache.clone()) for l in model.backbone.layers])
    (y0, c0), (y1, c1) = results[False], results[True]
    assert y1.shape == (B, Nt) and torch.isfinite(y1).all()
    assert torch.equal(y0, y1)
    for (k0, v0), (k1, v1) in zip(c0, c1):
        assert torch.equal(k0, k1) and torch.equal(v0, v1)


def test_graph_sampling_falls_back_to_events_when_a_counter_wait_times_out(device, monkeypatch):
    """A wait on the counters that timed out voids the run (forced from the host: the check
    reports one failure): the predictor must record the step again with event ordering, sample
    afresh and keep using events."""
    from ar_nanotabpfn_amd import attention_kernels as ak
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=128, n_heads=4, n_layers=2, d_ff=128, num_features=3, buffer_size=5, num_components=4)
    model = _build(cfg, device, dtype=torch.bfloat16)
    B, Nc, Nt = 40, 600, 7
    g = torch.Generator().manual_seed(6)
    xc = torch.randn(1, Nc, 3, generator=g).expand(B, -1, -1).to(device, torch.bfloat16)
    yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, torch.bfloat16)
    xt = torch.randn(B, Nt, 3, generator=g).to(device, torch.bfloat16)

    ref = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    ref.counter_ordering = False
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    pred.sample_sequence(xc, yc, xt)  # records the step with counter ordering where the device allows
    if pred._graph_state.chains[0].order is None:
        pytest.skip("counter ordering is not in use on this device")
    calls = {"n": 0}
    real_failed = ak.QueueOrder.failed

    def failed_once(self):
        calls["n"] += 1
        return 1 if calls["n"] == 1 else real_failed(self)

    monkeypatch.setattr(ak.QueueOrder, "failed", failed_once)
    y = pred.sample_sequence(xc, yc, xt)
    assert calls["n"] == 1
    assert pred.counter_ordering is False and pred._graph_state.chains[0].order is None
    assert y.shape == (B, Nt) and torch.isfinite(y).all()
    # same variates in -> same values as a predictor that used events from the start
    torch.manual_seed(3)
    y_ref = ref.sample_sequence(xc, yc, xt)
    torch.manual_seed(3)
    y_again = pred.sample_sequence(xc, yc, xt)
    assert torch.equal(y_ref, y_again)


def test_graph_sampling_target_only_last_layer_changes_nothing_that_is_read(device):
    """The sampling loop lets the last layer finish the target row only.  Against the same loop
    with both rows finished: predictions agree to bf16 rounding (the target query of the last
    context pass is tiled and split differently when it stands alone) and the caches — which
    take the buffer row's K/V from in front of the attention call — are the same in every layer
    but for the propagation of those roundings through the next step's buffer row."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=128, n_heads=4, n_layers=3, d_ff=128, num_features=3, buffer_size=5, num_components=4)
    model = _build(cfg, device, dtype=torch.bfloat16)
    B, Nc, Nt = 70, 2100, 9
    g = torch.Generator().manual_seed(8)
    xc = torch.randn(1, Nc, 3, generator=g).expand(B, -1, -1).to(device, torch.bfloat16)
    yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, torch.bfloat16)
    xt = torch.randn(B, Nt, 3, generator=g).to(device, torch.bfloat16)
    results = {}
    for cut in (False, True):
        pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
        pred.target_only_last_layer = cut
        torch.manual_seed(21)
        y = pred.sample_sequence(xc, yc, xt)
        results[cut] = (y, [(l.k_buf_cache.clone(), l.v_buf_cache.clone()) for l in model.backbone.layers])
    (y0, c0), (y1, c1) = results[False], results[True]
    assert y1.shape == (B, Nt) and torch.isfinite(y1).all()
    # step 1 (first replayed step) starts from identical state: only the last context pass differs
    assert max_abs(to_np(y0[:, :2]), to_np(y1[:, :2])) <= 2e-2
    # later steps feed earlier samples back; a sampled value moves with the rounding of its mean
    assert max_abs(to_np(y0), to_np(y1)) <= 0.25
    for (k0, v0), (k1, v1) in zip(c0, c1):
        assert max_abs(to_np(k0[:, :, :1]), to_np(k1[:, :, :1])) <= 2e-2  # the row appended by step 1
        assert max_abs(to_np(v0[:, :, :1]), to_np(v1[:, :, :1])) <= 2e-2


@pytest.mark.parametrize("ordered", [True, False], ids=["counters", "events"])
def test_graph_sampling_with_one_launch_step_boundary_equals_three_launches(device, ordered):
    """The recorded decode step whose boundary (last layer's tail, head, draw, next embedding,
    first layer's head of the next step) is one launch against the same step with the three
    launches: same variates in, the same predictions and caches out, bit for bit (bf16, several
    steps per graph and a remainder, both orderings of the two streams, graphs reused by a second
    call)."""
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    cfg = dict(d_model=128, n_heads=4, n_layers=3, d_ff=128, num_features=3, buffer_size=5, num_components=4)
    model = _build(cfg, device, dtype=torch.bfloat16)
    B, Nc, Nt = 70, 2100, 11
    g = torch.Generator().manual_seed(6)
    xc = torch.randn(1, Nc, 3, generator=g).expand(B, -1, -1).to(device, torch.bfloat16)
    yc = torch.randn(1, Nc, generator=g).expand(B, -1).to(device, torch.bfloat16)
    xt = torch.randn(B, Nt, 3, generator=g).to(device, torch.bfloat16)
    results = {}
    for fused in (False, True):
        pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
        pred.counter_ordering = ordered
        pred.fuse_step_boundary = fused
        for n in (Nt, 4, Nt):  # a shorter run in between: the state of a run must not leak into the next
            torch.manual_seed(13)
            y = pred.sample_sequence(xc, yc, xt[:, :n])
        st = pred._graph_state.chains[0]
        assert (st.boundary is not None) == fused
        if st.order is not None:
            assert st.order.failed() == 0
        results[fused] = (y, [(l.k_buf_cache.clone(), l.v_buf_cache.clone()) for l in model.backbone.layers])
    (y0, c0), (y1, c1) = results[False], results[True]
    assert y1.shape == (B, Nt) and torch.isfinite(y1).all()
    assert torch.equal(y0, y1)
    for (k0, v0), (k1, v1) in zip(c0, c1):
        assert torch.equal(k0, k1) and torch.equal(v0, v1)
