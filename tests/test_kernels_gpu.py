"""Parity of every C-ABI entry point (through the Python mirror) against the numpy
oracle on identical seeded inputs.  Tolerances: 2e-2 max-abs on 16-bit outputs,
1e-3 on float32 LSE; 1e-5 for float32 inputs (the reference's own kernel-vs-PyTorch
tolerance, tests/test_triton_kernel.py:51-66)."""

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from tests.helpers import lse_tol, max_abs, out_tol, randn, to_np

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _ak():
    import ar_nanotabpfn_amd.attention_kernels as ak

    return ak


def _ctx_inputs(B, H, Lq, Nc, D, dtype, seed=42, scale=1.0, per_batch=False):
    q = randn((B, H, Lq, D), seed, dtype, scale)
    kshape = (B, H, Nc, D) if per_batch else (H, Nc, D)
    k = randn(kshape, seed + 1, dtype, scale)
    v = randn(kshape, seed + 2, dtype, scale)
    return q, k, v


# ----- context attention (reference grid: tests/test_triton_kernel.py:28-129) -----------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_mfma", [True, False])
@pytest.mark.parametrize(
    "B,H,Lq,Nc,D",
    [
        (1, 4, 1, 32, 32),
        (16, 8, 1, 64, 64),
        (64, 4, 1, 128, 32),
        (128, 8, 1, 256, 64),
        (37, 4, 1, 64, 32),  # batch not divisible by any tile
        (32, 4, 1, 100, 32),  # context not divisible by any tile
        (8, 2, 5, 64, 32),  # multi-query
        (1, 2, 2, 32, 32),
        (3, 2, 7, 333, 128),
        (5, 3, 3, 70, 16),  # head_dim only the portable kernel covers
    ],
)
def test_context_attention_matches_oracle(device, dtype, use_mfma, B, H, Lq, Nc, D):
    ak = _ak()
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, dtype)
    out, lse = ak.context_attention(q.to(device), k.to(device), v.to(device), use_triton=use_mfma)
    ref_out, ref_lse = ao.context_attention(to_np(q), to_np(k), to_np(v))
    assert out.shape == (B, H, Lq, D) and out.dtype == dtype
    assert lse.shape == (B, H, Lq) and lse.dtype == torch.float32
    tol_o, tol_l = out_tol(dtype), lse_tol(dtype)
    if dtype == torch.float32:
        tol_o = tol_l = 2e-5  # randn-scale scores up to ~20: float32 rounding of the scores themselves
    else:
        # unit-variance q,k give peaked softmaxes (a handful of keys carry the mass).  The
        # MFMA kernel sums the 16-bit-rounded probabilities it feeds to the PV product, so
        # the LSE carries their rounding: <= 2^-9 relative for a one-key softmax, shrinking
        # as 1/sqrt(#effective keys).  At the 1/sqrt(64)-scaled inputs the 1e-3 target is
        # stated for (test_decode_attention_config1_shape etc.) the error is ~1e-5.
        tol_l = 2.5e-3
    assert max_abs(to_np(out), ref_out) <= tol_o
    assert max_abs(to_np(lse), ref_lse) <= tol_l


@pytest.mark.parametrize("use_mfma", [True, False])
@pytest.mark.parametrize("B,H,Lq,Nc,D,scale", [(256, 8, 1, 1024, 64, 0.125), (37, 4, 2, 700, 32, 0.125), (9, 2, 2, 333, 32, 1.0)])
def test_context_attention_vs_same_dtype_reference(device, use_mfma, B, H, Lq, Nc, D, scale):
    """Secondary comparison: against pytorch_context_attention evaluated the way torch evaluates it
    on bfloat16 tensors (scores, probabilities and output rounded to bfloat16; float32 LSE of the
    rounded scores, triton_kernels.py:558-565).  Looser by construction: at the 1/8-scaled inputs
    of configs[1] both references are far inside 2e-2 / 1e-3; at unit scale the rounded scores
    alone move the LSE by up to 2^-8 of a score of ~10."""
    ak = _ak()
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, torch.bfloat16, seed=11, scale=scale)
    out, lse = ak.context_attention(q.to(device), k.to(device), v.to(device), use_triton=use_mfma)
    ref_out, ref_lse = ao.context_attention_same_dtype(to_np(q), to_np(k), to_np(v))
    tol_o, tol_l = (2e-2, 1e-3) if scale < 1.0 else (6e-2, 5e-2)
    assert max_abs(to_np(out), ref_out) <= tol_o
    assert max_abs(to_np(lse), ref_lse) <= tol_l


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_context_attention_per_dataset_context(device, dtype):
    ak = _ak()
    B, H, Lq, Nc, D = 6, 4, 9, 150, 32
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, dtype, per_batch=True, scale=0.5)
    out, lse = ak.context_attention(q.to(device), k.to(device), v.to(device))
    ref_out, ref_lse = ao.context_attention(to_np(q), to_np(k), to_np(v))
    assert max_abs(to_np(out), ref_out) <= out_tol(dtype)
    assert max_abs(to_np(lse), ref_lse) <= lse_tol(dtype)


def test_context_attention_more_head_groups_than_one_grid_holds(device):
    """Per-dataset contexts with more than 65535 x 8 (dataset, head) pairs: the matrix-core kernel's
    grid counts blocks of eight pairs in its z dimension, so the call is spread over two launches.
    The first and the last datasets against the oracle, everything against the portable kernel."""
    ak = _ak()
    B, H, Lq, Nc, D = 66000, 8, 1, 32, 32
    g = torch.Generator(device=device).manual_seed(5)
    mk = lambda *shape: (torch.randn(*shape, generator=g, device=device) * 0.6).to(torch.bfloat16)
    q, k, v = mk(B, H, Lq, D), mk(B, H, Nc, D), mk(B, H, Nc, D)
    out, lse = ak.context_attention(q, k, v)
    out_p, lse_p = ak.context_attention(q, k, v, use_triton=False)
    assert float((out.float() - out_p.float()).abs().max()) <= 2e-2
    assert float((lse - lse_p).abs().max()) <= 2.5e-3
    for sl in (slice(0, 3), slice(B - 3, B)):
        ref_out, ref_lse = ao.context_attention(to_np(q[sl]), to_np(k[sl]), to_np(v[sl]))
        assert max_abs(to_np(out[sl]), ref_out) <= 2e-2
        assert max_abs(to_np(lse[sl]), ref_lse) <= 2.5e-3


def test_context_attention_first_tiles_from_leading_arguments(device):
    """The plain context launch over one shared context requests its first K/V tiles from leading
    scalar kernel arguments when K and V have the same strides, and from the argument struct like
    every other launch when they have not: the same numbers either way, and the oracle's."""
    ak = _ak()
    B, H, Lq, Nc, D = 512, 8, 2, 2048, 32
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, torch.bfloat16, scale=0.6)  # k, v: [H, Nc, D], shared
    qd, kd, vd = q.to(device), k.to(device), v.to(device)
    out_a, lse_a = ak.context_attention(qd, kd, vd)
    wide = torch.zeros(H, Nc, 2 * D, device=device, dtype=torch.bfloat16)
    wide[..., :D] = kd
    k_strided = wide[..., :D]  # rows twice as far apart as V's
    assert k_strided.stride(1) != vd.stride(1)
    out_b, lse_b = ak.context_attention(qd, k_strided, vd)
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    ref_out, ref_lse = ao.context_attention(to_np(q[:4]), to_np(k), to_np(v))
    assert max_abs(to_np(out_a[:4]), ref_out) <= 2e-2
    assert max_abs(to_np(lse_a[:4]), ref_lse) <= 1e-3


def test_context_attention_split_context_large(device):
    """Long context, few query rows: the split-context schedule with the LSE combine."""
    ak = _ak()
    B, H, Lq, Nc, D = 64, 8, 2, 4096, 32
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, torch.bfloat16, scale=0.6)
    out, lse = ak.context_attention(q.to(device), k.to(device), v.to(device))
    ref_out, ref_lse = ao.context_attention(to_np(q), to_np(k), to_np(v))
    assert max_abs(to_np(out), ref_out) <= 2e-2
    assert max_abs(to_np(lse), ref_lse) <= 1e-3


def test_context_attention_strided_q_view(device):
    """q arrives as the transposed view of a [B,N,H*Dh] projection (inference.py:781)."""
    ak = _ak()
    B, H, Lq, Nc, D = 9, 4, 2, 96, 32
    proj = randn((B, Lq, H * D), 7, torch.bfloat16)
    q = proj.view(B, Lq, H, D).transpose(1, 2)
    _, k, v = _ctx_inputs(B, H, Lq, Nc, D, torch.bfloat16)
    qd = proj.to(device).view(B, Lq, H, D).transpose(1, 2)
    assert not qd.is_contiguous()
    out, lse = ak.context_attention(qd, k.to(device), v.to(device))
    ref_out, ref_lse = ao.context_attention(to_np(q), to_np(k), to_np(v))
    assert max_abs(to_np(out), ref_out) <= 2e-2
    assert max_abs(to_np(lse), ref_lse) <= 2.5e-3  # unit-variance scores: see test_context_attention_matches_oracle
    # the output's transposed reshape must be a view (free for out_proj)
    flat = out.transpose(1, 2).reshape(B, Lq, H * D)
    assert flat.data_ptr() == out.data_ptr()


# ----- decode step ------------------------------------------------------------------------------


def _decode_case(device, dtype, B, H, Lq, Nc, D, n_buf, cap, with_new, use_mfma, scale=1.0, seed=3, overlapped=False):
    ak = _ak()
    side = torch.cuda.Stream(device=device) if overlapped else None
    q, k_ctx, v_ctx = _ctx_inputs(B, H, Lq, Nc, D, dtype, seed=seed, scale=scale)
    k_cache = randn((B, H, cap, D), seed + 10, dtype, scale)
    v_cache = randn((B, H, cap, D), seed + 11, dtype, scale)
    k_new = randn((B, H, 1, D), seed + 12, dtype, scale) if with_new else None
    v_new = randn((B, H, 1, D), seed + 13, dtype, scale) if with_new else None
    kc_d, vc_d = k_cache.to(device), v_cache.to(device)
    out = ak.decode_attention(
        q.to(device), k_ctx.to(device), v_ctx.to(device), kc_d, vc_d, n_buf,
        k_new.to(device) if with_new else None, v_new.to(device) if with_new else None, use_triton=use_mfma,
        side_stream=side,
    )
    ref, k_all, v_all = ao.decode_step_attention(
        to_np(q), to_np(k_ctx), to_np(v_ctx), to_np(k_cache[:, :, :n_buf]), to_np(v_cache[:, :, :n_buf]),
        to_np(k_new) if with_new else None, to_np(v_new) if with_new else None,
    )
    tol = out_tol(dtype) if dtype != torch.float32 else 2e-5
    assert max_abs(to_np(out), ref) <= tol
    # cache after the call: appended row in place, everything else untouched (bit-exact)
    exp_k, exp_v = k_cache.clone(), v_cache.clone()
    if with_new:
        exp_k[:, :, n_buf] = k_new[:, :, 0]
        exp_v[:, :, n_buf] = v_new[:, :, 0]
    assert torch.equal(kc_d.cpu(), exp_k) and torch.equal(vc_d.cpu(), exp_v)


@pytest.fixture(params=[1, 0], ids=["one-launch", "general-route"])
def small_route(request, tuning):
    """Small decode problems take a single-launch kernel (ARTAB_SMALL, on by default); with it
    switched off the same call goes through the context pass, the buffer pass and their merge."""
    tuning(ARTAB_SMALL=request.param)
    return request.param


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_mfma", [True, False])
@pytest.mark.parametrize(
    "B,H,Lq,Nc,D,n_buf,cap,with_new",
    [
        (8, 4, 1, 64, 32, 0, 16, False),  # first target: context only
        (8, 4, 2, 64, 32, 0, 16, True),  # second step: buffer is just the new row
        (8, 4, 2, 64, 32, 5, 16, True),
        (8, 4, 2, 64, 32, 15, 16, True),  # last slot
        (8, 4, 1, 64, 32, 7, 16, False),  # target only over committed buffers
        (8, 4, 1, 64, 32, 6, 16, True),   # target query alone, with the step's buffer row appended (last layer of a step)
        (33, 8, 2, 100, 64, 19, 64, True),
        (5, 2, 2, 300, 128, 70, 80, True),
        (4, 3, 2, 50, 16, 9, 12, True),  # portable-only head_dim
        (9, 2, 1, 31, 32, 0, 4, False),  # context shorter than one key block
        (37, 3, 2, 1000, 64, 33, 48, True),  # ragged trajectory group, ragged last key block
        (64, 8, 2, 2048, 64, 63, 64, True),  # the largest context the one-launch kernel takes at head_dim 64
        (11, 5, 1, 257, 32, 40, 41, True),  # one key block more than the wavefronts share evenly
    ],
)
def test_decode_attention_matches_oracle(device, small_route, dtype, use_mfma, B, H, Lq, Nc, D, n_buf, cap, with_new):
    _decode_case(device, dtype, B, H, Lq, Nc, D, n_buf, cap, with_new, use_mfma)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "B,H,Lq,Nc,D,n_buf,cap,with_new",
    [
        (8, 4, 1, 64, 32, 0, 16, False),  # nothing for the buffer pass to do: plain schedule
        (8, 4, 2, 64, 32, 0, 16, True),   # the new row alone
        (8, 4, 2, 64, 32, 3, 16, True),   # exactly one 4-key chunk
        (8, 4, 2, 64, 32, 15, 16, True),  # last slot
        (8, 4, 1, 64, 32, 7, 16, False),  # target only over committed buffers, ragged last chunk
        (8, 4, 1, 64, 32, 6, 16, True),   # target query alone, buffer row appended by the streaming pass
        (70, 8, 1, 4096, 32, 11, 16, True),  # the same with a split context
        (5, 3, 2, 200, 32, 22, 40, True),  # 15 pairs: one ragged task
        (33, 8, 2, 100, 64, 19, 64, True),  # other head dims: register-staged buffer pass
        (5, 2, 2, 300, 128, 70, 80, True),
        (128, 8, 2, 8192, 32, 100, 128, True),  # split context + streamed buffer partial + combine
        (600, 8, 2, 1024, 32, 37, 64, True),  # more tasks than workgroups: several tasks per wavefront
        (4, 3, 2, 50, 16, 9, 12, True),  # portable-only head_dim: side stream is ignored
    ],
)
def test_decode_attention_overlapped_matches_oracle(device, small_route, dtype, B, H, Lq, Nc, D, n_buf, cap, with_new):
    """Buffer pass on a side stream next to the context pass, then the combine launch (small
    problems take the one-launch kernel instead unless it is switched off)."""
    _decode_case(device, dtype, B, H, Lq, Nc, D, n_buf, cap, with_new, True, scale=0.6, overlapped=True)


@pytest.fixture(params=["0", "100000", "20", None], ids=["16-row-chunks", "4-row-chunks", "switch-at-20-rows", "by-length"])
def stream_chunk_shape(request, tuning):
    """The streaming buffer pass reads 4 rows of 16 pairs or 16 rows of 4 pairs per request and
    picks by buffer length (ARTAB_STREAM_SHORT: the longest buffer that takes the first shape)."""
    tuning(ARTAB_SMALL=0)
    if request.param is not None:
        tuning(ARTAB_STREAM_SHORT=int(request.param))
    return request.param


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "B,H,Lq,Nc,D,n_buf,cap,with_new",
    [
        (8, 4, 2, 64, 32, 0, 16, True),    # the new row alone: one lane group of a 16-row chunk has a key
        (8, 4, 1, 64, 32, 1, 16, False),   # one committed row, one query
        (8, 4, 2, 64, 32, 3, 16, True),    # 4 rows
        (8, 4, 2, 64, 32, 4, 16, True),    # 5 rows: the second lane group holds the new row alone
        (8, 4, 2, 64, 32, 15, 16, True),   # exactly one 16-row chunk, new row in its last lane
        (8, 4, 2, 64, 32, 16, 32, True),   # 17 rows: the new row alone in a second chunk
        (8, 4, 1, 64, 32, 16, 32, False),  # 16 committed rows, nothing to append
        (7, 5, 2, 128, 32, 31, 48, True),  # 35 pairs (ragged for both shapes), two full chunks
        (7, 5, 2, 128, 32, 32, 48, True),
        (7, 5, 1, 128, 32, 47, 48, True),  # last slot of the cache, three chunks
        (5, 3, 2, 200, 32, 22, 40, True),  # 15 pairs
        (1, 1, 2, 64, 32, 20, 32, True),   # a single pair
        (3, 2, 2, 64, 32, 77, 100, True),  # steady steps between a task's first and last chunk
        (128, 8, 2, 2048, 32, 100, 128, True),
        (600, 8, 2, 1024, 32, 37, 64, True),  # several tasks per wavefront with either shape
        (600, 8, 1, 1024, 32, 9, 64, True),   # ... of one chunk each
        (300, 8, 2, 512, 32, 255, 256, True),  # the longest buffer
    ],
)
def test_decode_attention_stream_chunk_shapes(device, stream_chunk_shape, dtype, B, H, Lq, Nc, D, n_buf, cap, with_new):
    """The streaming buffer pass (beside the context pass) in both of its chunk shapes."""
    _decode_case(device, dtype, B, H, Lq, Nc, D, n_buf, cap, with_new, True, scale=0.6, overlapped=True)


@pytest.mark.parametrize("n_buf", [5, 150])
def test_decode_attention_wave_priorities_do_not_change_results(device, tuning, n_buf):
    """The two passes of an overlapped call choose their wave priorities from the buffer length
    (ARTAB_STREAM_CALM: the buffer pass stays at the base priority up to that many rows;
    ARTAB_CTX_YIELD: the context pass runs a step lower from that many rows on).  Priorities decide
    who is issued first, never what is computed: every setting must give the same bits."""
    ak = _ak()
    tuning(ARTAB_SMALL=0)
    dtype, B, H, Nc, D, cap = torch.bfloat16, 96, 8, 4096, 32, 160
    q, k_ctx, v_ctx = (t.to(device) for t in _ctx_inputs(B, H, 2, Nc, D, dtype, seed=11, scale=0.6))
    kb, vb = randn((B, H, cap, D), 12, dtype, 0.6).to(device), randn((B, H, cap, D), 13, dtype, 0.6).to(device)
    kn, vn = randn((B, H, 1, D), 14, dtype, 0.6).to(device), randn((B, H, 1, D), 15, dtype, 0.6).to(device)
    side = torch.cuda.Stream(device=device)
    outs = []
    for calm, give_way in ((None, None), (0, 0), (1000, 1), (0, 1), (1000, 0)):
        tuning(ARTAB_STREAM_CALM=calm, ARTAB_CTX_YIELD=give_way)
        outs.append(ak.decode_attention(q, k_ctx, v_ctx, kb.clone(), vb.clone(), n_buf, kn, vn, side_stream=side))
        torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    ref, _, _ = ao.decode_step_attention(to_np(q), to_np(k_ctx), to_np(v_ctx), to_np(kb[:, :, :n_buf]),
                                         to_np(vb[:, :, :n_buf]), to_np(kn), to_np(vn))
    assert max_abs(to_np(outs[0]), ref) <= 2e-2


def test_decode_attention_overlapped_device_length_in_graph(device):
    """The overlapped call recorded into a graph (fork/join inside the capture) with the buffer
    length in device memory: every replay appends one row and must equal the eager plain call."""
    ak = _ak()
    dtype, B, H, Nc, D, cap = torch.bfloat16, 64, 8, 2048, 32, 8
    q, k_ctx, v_ctx = (t.to(device) for t in _ctx_inputs(B, H, 2, Nc, D, dtype, seed=1, scale=0.6))
    k_cache, v_cache = randn((B, H, cap, D), 2, dtype, 0.6).to(device), randn((B, H, cap, D), 3, dtype, 0.6).to(device)
    k_ref, v_ref = k_cache.clone(), v_cache.clone()
    k_new, v_new = randn((B, H, 1, D), 4, dtype, 0.6).to(device), randn((B, H, 1, D), 5, dtype, 0.6).to(device)
    nbuf = torch.zeros(1, dtype=torch.int32, device=device)
    side = torch.cuda.Stream(device=device)
    out_static = torch.empty_like(q)

    def step():
        out_static.copy_(ak.decode_attention(q, k_ctx, v_ctx, k_cache, v_cache, cap - 1, k_new, v_new,
                                             n_buf_device=nbuf, side_stream=side))
        nbuf.add_(1)

    warm = torch.cuda.Stream(device=device)
    warm.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(warm):
        step()
    torch.cuda.current_stream(device).wait_stream(warm)
    nbuf.zero_()
    k_cache.copy_(k_ref)
    v_cache.copy_(v_ref)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    nbuf.zero_()
    k_cache.copy_(k_ref)
    v_cache.copy_(v_ref)
    for n in range(6):
        graph.replay()
        torch.cuda.synchronize()
        expect = ak.decode_attention(q, k_ctx, v_ctx, k_ref, v_ref, n, k_new, v_new)  # plain, eager, appends to the copy
        assert int(nbuf.item()) == n + 1
        assert max_abs(to_np(out_static), to_np(expect)) <= 2e-2
        assert torch.equal(k_cache, k_ref) and torch.equal(v_cache, v_ref)


def _full_size_decode(device, B, H, Nc, n_buf, cap, seed):
    """One decode step at a BASELINE shape (Dh=32, Lq=2, bf16).  Inputs are drawn on the device
    (the buffer cache alone is up to 0.5 GB); the oracle sees a sample of the trajectories, every
    head of them; the cache is compared whole and bit-exact; the schedules of the step (buffer
    pass after the context pass, beside it, merge left to the caller, streams ordered by counters)
    must agree on every row to within the rounding of the 16-bit partial outputs."""
    ak = _ak()
    dtype, D, Lq = torch.bfloat16, 32, 2
    g = torch.Generator(device=device).manual_seed(seed)

    def draw(*shape):
        return (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * 0.6).to(dtype)

    q, k_ctx, v_ctx = draw(B, H, Lq, D), draw(H, Nc, D), draw(H, Nc, D)
    k_cache, v_cache = draw(B, H, cap, D), draw(B, H, cap, D)
    k_new, v_new = draw(B, H, 1, D), draw(B, H, 1, D)
    exp_k, exp_v = k_cache.clone(), v_cache.clone()
    exp_k[:, :, n_buf] = k_new[:, :, 0]
    exp_v[:, :, n_buf] = v_new[:, :, 0]
    side = torch.cuda.Stream(device=device)

    outs = []
    for kwargs in (dict(), dict(side_stream=side), dict(side_stream=side, leave_partials=True)):
        kc, vc = k_cache.clone(), v_cache.clone()
        out = ak.decode_attention(q, k_ctx, v_ctx, kc, vc, n_buf, k_new, v_new, **kwargs)
        if hasattr(out, "desc"):  # unmerged partial slots: the stand-alone merge of the library
            assert out.desc.n_slots >= 2
            out = out.merged()
        torch.cuda.synchronize()
        assert torch.equal(kc, exp_k) and torch.equal(vc, exp_v)
        outs.append(out.float())
    for other in outs[1:]:
        assert float((outs[0] - other).abs().max()) <= 2e-2
    # fourth schedule: the two streams ordered by device-side counters (one fork, one join) —
    # the same launches as the third, so the merged result must be the same bit for bit
    main = torch.cuda.current_stream(device)
    side2, concurrent = ak.concurrent_stream(device, main)
    if concurrent:
        order = ak.QueueOrder(device)
        kc, vc = k_cache.clone(), v_cache.clone()
        side2.wait_stream(main)
        parts = ak.decode_attention(q, k_ctx, v_ctx, kc, vc, n_buf, k_new, v_new, side_stream=side2,
                                    leave_partials=True, order=order)
        out = parts.merged()
        main.wait_stream(side2)
        torch.cuda.synchronize()
        assert order.failed() == 0
        assert torch.equal(kc, exp_k) and torch.equal(vc, exp_v)
        assert torch.equal(out.float(), outs[2])

    sample = sorted({0, 1, B // 2 - 1, B // 2, B - 2, B - 1, (7 * seed + 13) % B, (31 * seed + 5) % B})
    idx = torch.tensor(sample, device=device)
    ref, _, _ = ao.decode_step_attention(
        to_np(q[idx]), to_np(k_ctx), to_np(v_ctx), to_np(k_cache[idx][:, :, :n_buf]), to_np(v_cache[idx][:, :, :n_buf]),
        to_np(k_new[idx]), to_np(v_new[idx]),
    )
    for out in outs:
        assert max_abs(to_np(out[idx]), ref) <= 2e-2


@pytest.mark.parametrize("n_buf", [0, 37, 255])
def test_decode_attention_config3_full_size(device, n_buf):
    """BASELINE configs[3] layer-step: B=1024 trajectories, 8 heads, N_ctx=16384, buffer up to 256."""
    _full_size_decode(device, 1024, 8, 16384, n_buf, 256, seed=3 + n_buf)


def test_context_pass_tile_loop_forms_agree_bit_for_bit(device, tuning):
    """Beside a buffer pass the context pass runs the bulk of its tile loop as straight-line code
    while the committed buffer is short and tile by tile beyond (``ARTAB_DENSE_BELOW`` rows, read
    with the length on the device): the same products in the same order, so the partial slots are
    identical whichever form ran (configs[3] shape, 37 buffer rows, limit forced to either side)."""
    ak = _ak()
    B, H, Nc, D, Lq, n_buf, cap = 1024, 8, 16384, 32, 2, 37, 64
    g = torch.Generator(device=device).manual_seed(21)
    draw = lambda *shape: (torch.randn(*shape, generator=g, device=device) * 0.6).to(torch.bfloat16)  # noqa: E731
    q, k_ctx, v_ctx = draw(B, H, Lq, D), draw(H, Nc, D), draw(H, Nc, D)
    k_cache, v_cache, k_new, v_new = draw(B, H, cap, D), draw(B, H, cap, D), draw(B, H, 1, D), draw(B, H, 1, D)
    nbuf = torch.tensor([n_buf], device=device, dtype=torch.int32)
    side = torch.cuda.Stream(device=device)
    outs = []
    for limit in ("1", "100000"):
        tuning(ARTAB_DENSE_BELOW=int(limit))
        parts = ak.decode_attention(q, k_ctx, v_ctx, k_cache.clone(), v_cache.clone(), cap - 1, k_new, v_new,
                                    side_stream=side, leave_partials=True, n_buf_device=nbuf)
        outs.append(parts.merged())
        torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("n_buf", [1, 130, 255])
def test_decode_attention_config4_full_size(device, n_buf):
    """BASELINE configs[4] layer-step: B=2048 trajectories, 16 heads, N_ctx=4096, buffer up to 256."""
    _full_size_decode(device, 2048, 16, 4096, n_buf, 256, seed=4 + n_buf)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,Lq,Nc,D,n_buf,cap", [(6, 4, 2, 70, 32, 0, 90), (6, 4, 2, 70, 32, 9, 90), (5, 2, 1, 33, 64, 4, 40),
                                                   (5, 2, 1, 33, 64, 0, 40),
                                                   (3, 2, 2, 257, 128, 30, 300), (64, 8, 2, 512, 32, 100, 640)])
def test_decode_attention_per_trajectory_cache(device, dtype, B, H, Lq, Nc, D, n_buf, cap):
    """Per-dataset layout (inference.py:687-744): every trajectory has its own context, stored in
    front of its buffer rows in one cache [B,H,cap,D].  The context view and the buffer view are
    then one run of rows, which the streaming buffer kernel reads as it is (16-bit types); the new
    row is appended at slot Nc + n_buf."""
    ak = _ak()
    cache_k, cache_v = randn((B, H, cap, D), 21, dtype, 0.7), randn((B, H, cap, D), 22, dtype, 0.7)
    q = randn((B, H, Lq, D), 23, dtype, 0.7)
    k_new = randn((B, H, 1, D), 24, dtype, 0.7) if Lq == 2 else None
    v_new = randn((B, H, 1, D), 25, dtype, 0.7) if Lq == 2 else None
    kc_d, vc_d = cache_k.to(device), cache_v.to(device)
    out = ak.decode_attention(
        q.to(device), kc_d[:, :, :Nc], vc_d[:, :, :Nc], kc_d[:, :, Nc:], vc_d[:, :, Nc:], n_buf,
        k_new.to(device) if Lq == 2 else None, v_new.to(device) if Lq == 2 else None)
    keys = torch.cat([cache_k[:, :, : Nc + n_buf]] + ([k_new] if Lq == 2 else []), dim=2)
    vals = torch.cat([cache_v[:, :, : Nc + n_buf]] + ([v_new] if Lq == 2 else []), dim=2)
    ref, _ = ao.context_attention(to_np(q), to_np(keys), to_np(vals))
    tol = out_tol(dtype) if dtype != torch.float32 else 2e-5
    assert max_abs(to_np(out), ref) <= tol
    exp_k, exp_v = cache_k.clone(), cache_v.clone()
    if Lq == 2:
        exp_k[:, :, Nc + n_buf] = k_new[:, :, 0]
        exp_v[:, :, Nc + n_buf] = v_new[:, :, 0]
    assert torch.equal(kc_d.cpu(), exp_k) and torch.equal(vc_d.cpu(), exp_v)


@pytest.mark.parametrize("n_buf", [1, 2, 17, 33, 64])
def test_decode_attention_config1_shape(device, small_route, n_buf):
    """BASELINE configs[1]: H=8, Dh=64, Nc=1024, B=256, entries ~N(0,1)/8, N_buf swept."""
    _decode_case(device, torch.bfloat16, 256, 8, 1, 1024, 64, n_buf, 64, False, True, scale=0.125, seed=0)


def test_decode_attention_long_context_split(device):
    """Many context slices + buffer pass + merge (the configs[3] schedule, smaller)."""
    _decode_case(device, torch.bfloat16, 128, 8, 2, 8192, 32, 100, 128, True, True, scale=0.6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Lq,Nc,D", [(64, 2, 8192, 32), (40, 1, 4200, 64), (300, 2, 2048, 32)])
@pytest.mark.parametrize("cache", ["none", "zero-rows"])
def test_decode_attention_split_context_without_any_buffer(device, dtype, B, Lq, Nc, D, cache):
    """A shared context long enough to be cut into slices, no committed buffer row and no new
    row, with no cache at all or one that holds zero rows: the call is context attention
    (tests/test_triton_kernel.py:319-339 on the split route) and must not touch the cache."""
    ak = _ak()
    H = 8
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, dtype, seed=11, scale=0.5)
    kb = None if cache == "none" else torch.empty(B, H, 0, D, dtype=dtype, device=device)
    out = ak.decode_attention(q.to(device), k.to(device), v.to(device), kb, kb, 0)
    ref, _ = ao.context_attention(to_np(q), to_np(k), to_np(v))
    assert out.shape == (B, H, Lq, D) and out.dtype == dtype
    assert max_abs(to_np(out), ref) <= out_tol(dtype)


def test_hybrid_attention_empty_buffer_is_context_only(device):
    """tests/test_triton_kernel.py:319-339."""
    ak = _ak()
    B, H, Lq, Nc, D = 32, 4, 1, 64, 32
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, torch.float32)
    kb = torch.empty(B, H, 0, D)
    out = ak.hybrid_attention(q.to(device), k.to(device), v.to(device), kb.to(device), kb.to(device), use_triton=False)
    ref, _ = ao.context_attention(to_np(q), to_np(k), to_np(v))
    assert max_abs(to_np(out), ref) <= 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hybrid_attention_matches_full_attention(device, dtype):
    """tests/test_triton_kernel.py:288-317: hybrid == one softmax over cat(ctx, buffer)."""
    ak = _ak()
    B, H, Lq, D, Nc, Nb = 64, 4, 1, 32, 128, 32
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, dtype)
    kb, vb = randn((B, H, Nb, D), 50, dtype), randn((B, H, Nb, D), 51, dtype)
    out = ak.hybrid_attention(q.to(device), k.to(device), v.to(device), kb.to(device), vb.to(device))
    k_full = np.concatenate([np.broadcast_to(to_np(k)[None], (B, H, Nc, D)), to_np(kb)], axis=2)
    v_full = np.concatenate([np.broadcast_to(to_np(v)[None], (B, H, Nc, D)), to_np(vb)], axis=2)
    ref, _ = ao.masked_full_attention(to_np(q), k_full, v_full)
    assert max_abs(to_np(out), ref) <= (2e-5 if dtype == torch.float32 else 2e-2)


def test_hybrid_attention_with_buffer_mask(device):
    """tests/test_triton_kernel.py:242-282: masked buffer + merge == masked full attention."""
    ak = _ak()
    B, H, Lq, D, Nc, Nb = 8, 4, 1, 32, 32, 8
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, torch.float32)
    kb, vb = randn((B, H, Nb, D), 50, torch.float32), randn((B, H, Nb, D), 51, torch.float32)
    mask = torch.zeros(B, H, Lq, Nb, dtype=torch.bool)
    mask[..., :4] = True
    out = ak.hybrid_attention(
        q.to(device), k.to(device), v.to(device), kb.to(device), vb.to(device), buf_mask=mask.to(device)
    )
    k_full = np.concatenate([np.broadcast_to(to_np(k)[None], (B, H, Nc, D)), to_np(kb)], axis=2)
    v_full = np.concatenate([np.broadcast_to(to_np(v)[None], (B, H, Nc, D)), to_np(vb)], axis=2)
    full_mask = np.ones((B, H, Lq, Nc + Nb), dtype=bool)
    full_mask[..., Nc:] = mask.numpy()
    ref, _ = ao.masked_full_attention(to_np(q), k_full, v_full, mask=full_mask)
    assert max_abs(to_np(out), ref) <= 2e-5


# ----- buffer attention / merge -------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
def test_buffer_attention_masked_rows(device, dtype):
    """Target 0 sees no buffer: out 0, lse -inf (tests/test_triton_kernel.py:135-151)."""
    ak = _ak()
    B, H, Nt, D = 4, 2, 3, 16
    q = randn((B, H, 2 * Nt, D), 1, dtype)
    kb, vb = randn((B, H, Nt, D), 2, dtype), randn((B, H, Nt, D), 3, dtype)
    out, lse = ak.pytorch_teacher_forcing_buffer_attention(q.to(device), kb.to(device), vb.to(device), Nt)
    ref_out, ref_lse = ao.teacher_forcing_buffer_attention(to_np(q), to_np(kb), to_np(vb), Nt)
    assert torch.all(out[:, :, Nt] == 0)
    assert torch.isneginf(lse[:, :, Nt]).all()
    assert max_abs(to_np(out), ref_out) <= (2e-5 if dtype == torch.float32 else 2e-2)
    assert max_abs(to_np(lse), ref_lse) <= (2e-5 if dtype == torch.float32 else 1e-3)


def test_buffer_attention_shape_errors(device):
    ak = _ak()
    q = torch.zeros(2, 2, 6, 16, device=device)
    kb = torch.zeros(2, 2, 3, 16, device=device)
    with pytest.raises(ValueError):
        ak.pytorch_teacher_forcing_buffer_attention(q, kb, kb, 4)
    with pytest.raises(ValueError):
        ak.pytorch_teacher_forcing_buffer_attention(q[:, :, :4], kb, kb, 2)


def test_merge_closed_forms(device):
    """tests/test_triton_kernel.py:345-382."""
    ak = _ak()
    B, H, Lq, D = 8, 4, 1, 32
    a, b = randn((B, H, Lq, D), 1, torch.float32), randn((B, H, Lq, D), 2, torch.float32)
    hi = torch.full((B, H, Lq), 10.0)
    lo = torch.full((B, H, Lq), -10.0)
    out = ak.merge_attention_outputs(a.to(device), hi.to(device), b.to(device), lo.to(device))
    assert max_abs(to_np(out), to_np(a)) <= 1e-4
    eq = torch.full((B, H, Lq), 5.0)
    out = ak.merge_attention_outputs(a.to(device), eq.to(device), b.to(device), eq.to(device))
    assert max_abs(to_np(out), (to_np(a) + to_np(b)) / 2) <= 1e-5
    ninf = torch.full((B, H, Lq), float("-inf"))
    out = ak.merge_attention_outputs(a.to(device), eq.to(device), b.to(device), ninf.to(device))
    assert torch.equal(out.cpu(), a)


@pytest.mark.parametrize("dtype", DTYPES)
def test_merge_matches_oracle(device, dtype):
    ak = _ak()
    B, H, Lq, D = 5, 3, 4, 32
    a, b = randn((B, H, Lq, D), 1, dtype), randn((B, H, Lq, D), 2, dtype)
    la, lb = randn((B, H, Lq), 3, torch.float32, 3.0), randn((B, H, Lq), 4, torch.float32, 3.0)
    out = ak.merge_attention_outputs(a.to(device), la.to(device), b.to(device), lb.to(device))
    ref = ao.merge_attention_outputs(to_np(a), to_np(la), to_np(b), to_np(lb))
    assert max_abs(to_np(out), ref) <= (1e-5 if dtype == torch.float32 else 2e-2)


# ----- teacher forcing ------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_mfma", [True, False])
@pytest.mark.parametrize("per_batch", [False, True])
@pytest.mark.parametrize(
    "B,H,Nt,Nc,D",
    [
        (2, 3, 4, 5, 16),  # tests/test_triton_kernel.py:157-198
        (2, 2, 1, 40, 32),  # Nt = 1 (tests/test_triton_joint_density.py:255-260)
        (4, 4, 16, 64, 32),
        (3, 2, 50, 130, 32),  # nothing divides a tile
        (2, 8, 128, 512, 32),  # configs[2] per (b,h) shape
        (2, 2, 150, 96, 64),  # Nt > 128: several q tiles, tiles straddling the buffer/target border
        (1, 2, 37, 70, 128),
    ],
)
def test_teacher_forcing_matches_oracle(device, dtype, use_mfma, per_batch, B, H, Nt, Nc, D):
    ak = _ak()
    q, k, v = _ctx_inputs(B, H, 2 * Nt, Nc, D, dtype, per_batch=per_batch, scale=0.7)
    kb, vb = randn((B, H, Nt, D), 60, dtype, 0.7), randn((B, H, Nt, D), 61, dtype, 0.7)
    out, lse = ak.teacher_forcing_attention(
        q.to(device), k.to(device), v.to(device), kb.to(device), vb.to(device), Nt,
        use_triton=use_mfma, return_lse=True,
    )
    # ground truth: one masked softmax over cat(context, buffer, [never-visible targets])
    kc = to_np(k) if per_batch else np.broadcast_to(to_np(k)[None], (B, H, Nc, D))
    vc = to_np(v) if per_batch else np.broadcast_to(to_np(v)[None], (B, H, Nc, D))
    pad = np.zeros((B, H, Nt, D))
    k_full = np.concatenate([kc, to_np(kb), pad], axis=2)
    v_full = np.concatenate([vc, to_np(vb), pad], axis=2)
    mask = ao.teacher_forcing_mask(Nc, Nt)[None, None]
    ref_out, ref_lse = ao.masked_full_attention(to_np(q), k_full, v_full, mask=mask)
    tol_o = 2e-5 if dtype == torch.float32 else 2e-2
    tol_l = 2e-5 if dtype == torch.float32 else 1e-3
    assert max_abs(to_np(out), ref_out) <= tol_o
    assert max_abs(to_np(lse), ref_lse) <= tol_l
    # and the reference's own composition (context + masked buffer + merge)
    ref2 = ao.hybrid_teacher_forcing_attention(to_np(q), to_np(k), to_np(v), to_np(kb), to_np(vb), Nt)
    assert max_abs(to_np(out), ref2) <= tol_o


def test_teacher_forcing_strided_views(device):
    """q/k_buf/v_buf as views of the fresh [B,2Nt,H*Dh] projections (inference.py:869-876)."""
    ak = _ak()
    B, H, Nt, Nc, D = 3, 4, 20, 64, 32
    pq, pk, pv = (randn((B, 2 * Nt, H * D), s, torch.bfloat16, 0.7) for s in (1, 2, 3))
    k_ctx, v_ctx = randn((H, Nc, D), 4, torch.bfloat16, 0.7), randn((H, Nc, D), 5, torch.bfloat16, 0.7)

    def heads(t):
        return t.view(B, 2 * Nt, H, D).transpose(1, 2)

    qd, kd, vd = heads(pq.to(device)), heads(pk.to(device)), heads(pv.to(device))
    out = ak.hybrid_teacher_forcing_attention(
        qd, k_ctx.to(device), v_ctx.to(device), kd[:, :, :Nt], vd[:, :, :Nt], Nt
    )
    ref = ao.hybrid_teacher_forcing_attention(
        to_np(heads(pq)), to_np(k_ctx), to_np(v_ctx), to_np(heads(pk)[:, :, :Nt]), to_np(heads(pv)[:, :, :Nt]), Nt
    )
    assert max_abs(to_np(out), ref) <= 2e-2


# ----- prefill -----------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_mfma", [True, False])
@pytest.mark.parametrize("shared_cache", [True, False])
@pytest.mark.parametrize("B,H,Nc,D", [(1, 4, 64, 32), (3, 2, 100, 32), (2, 8, 512, 32), (2, 2, 300, 64), (1, 2, 130, 128)])
def test_prefill_matches_oracle_and_writes_cache(device, dtype, use_mfma, shared_cache, B, H, Nc, D):
    ak = _ak()
    # strided views of [B,Nc,H*D] projections, as the predictor produces them
    pq, pk, pv = (randn((B, Nc, H * D), s, dtype, 0.7) for s in (11, 12, 13))

    def heads(t):
        return t.view(B, Nc, H, D).transpose(1, 2)

    cap = Nc + 3
    if shared_cache:
        kc = torch.full((H, cap, D), 7.0, dtype=dtype, device=device)
    else:
        kc = torch.full((B, H, cap, D), 7.0, dtype=dtype, device=device)
    vc = kc.clone()
    out = ak.prefill_attention(
        heads(pq.to(device)), heads(pk.to(device)), heads(pv.to(device)), kc, vc, use_triton=use_mfma
    )
    ref, _ = ao.dense_self_attention(to_np(heads(pq)), to_np(heads(pk)), to_np(heads(pv)))
    assert max_abs(to_np(out), ref) <= (2e-5 if dtype == torch.float32 else 2e-2)
    k_exp = heads(pk)[0] if shared_cache else heads(pk)
    v_exp = heads(pv)[0] if shared_cache else heads(pv)
    assert torch.equal(kc[..., :Nc, :].cpu(), k_exp) and torch.equal(vc[..., :Nc, :].cpu(), v_exp)
    assert torch.all(kc[..., Nc:, :] == 7.0) and torch.all(vc[..., Nc:, :] == 7.0)


def test_prefill_permutation_invariance(device):
    """Context is bidirectional with no positions: permuting rows permutes outputs."""
    ak = _ak()
    B, H, Nc, D = 2, 4, 200, 32
    q, k, v = (randn((B, H, Nc, D), s, torch.bfloat16, 0.7).to(device) for s in (1, 2, 3))
    perm = torch.randperm(Nc, generator=torch.Generator().manual_seed(0)).to(device)
    out = ak.prefill_attention(q, k, v)
    out_p = ak.prefill_attention(q[:, :, perm], k[:, :, perm], v[:, :, perm])
    assert max_abs(to_np(out[:, :, perm]), to_np(out_p)) <= 1e-2


# ----- error behaviour through the ABI ---------------------------------------------------------------


def test_decode_errors(device):
    ak = _ak()
    q = torch.zeros(2, 2, 3, 32, device=device, dtype=torch.bfloat16)
    kc = torch.zeros(2, 8, 32, device=device, dtype=torch.bfloat16)
    cache = torch.zeros(2, 2, 4, 32, device=device, dtype=torch.bfloat16)
    with pytest.raises(ValueError):  # N not in {1,2} (inference.py:765-768)
        ak.decode_attention(q, kc, kc, cache, cache, 0)
    new = torch.zeros(2, 2, 1, 32, device=device, dtype=torch.bfloat16)
    with pytest.raises(ValueError):  # cache full (inference.py:247-250)
        ak.decode_attention(q[:, :, :2], kc, kc, cache, cache, 4, new, new)


def test_cpu_tensors_are_rejected():
    ak = _ak()
    q = torch.zeros(1, 1, 1, 32)
    k = torch.zeros(1, 4, 32)
    with pytest.raises(RuntimeError):
        ak.context_attention(q, k, k)


# ----- softmax range handling of the MFMA kernel ---------------------------------------------------


@pytest.mark.parametrize("shift", [0.0, 300.0, -300.0])
@pytest.mark.parametrize("gain", [1.0, 30.0])
def test_context_attention_extreme_scores(device, shift, gain):
    """Scores far outside the range where 2^s is representable (|s| ~ 300 nats, and
    unit-variance scores blown up 30x) must still give the exact softmax: the kernel's
    unshifted fast path has to notice and redo the rows with a running maximum."""
    ak = _ak()
    B, H, Lq, Nc, D = 40, 2, 2, 200, 32
    q, k, v = _ctx_inputs(B, H, Lq, Nc, D, torch.bfloat16, seed=5)
    q = (q.float() * gain).to(torch.bfloat16)
    if shift:
        # add a constant direction: q gets +a in dim 0, every key gets +b in dim 0 -> all
        # scores move by about shift (exactly representable factors)
        q[..., 0] = 16.0
        k[..., 0] = shift * (D ** 0.5) / 16.0
    out, lse = ak.context_attention(q.to(device), k.to(device), v.to(device))
    # At |scores| of tens to hundreds of nats the one rounding the kernel applies to
    # q * scale * log2(e) (to bf16, as the reference kernel does with q * sm_scale,
    # triton_kernels.py:120-121) moves scores by up to 2^-9 * |s|, which is visible in a
    # near-one-hot softmax.  The oracle is therefore evaluated on the q the kernel uses.
    cfac = D ** -0.5 * 1.4426950408889634
    q_eff = (q.float() * cfac).to(torch.bfloat16).double().numpy() / cfac
    ref_out, ref_lse = ao.context_attention(q_eff, to_np(k), to_np(v))
    assert np.isfinite(to_np(out)).all() and np.isfinite(to_np(lse)).all()
    assert max_abs(to_np(out), ref_out) <= 2e-2
    assert max_abs(to_np(lse), ref_lse) <= 2.5e-3


# ----- layer glue kernels -----------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,D", [(1, 4), (37, 128), (2048, 256), (5, 512), (3, 1024), (9, 36)])
@pytest.mark.parametrize("with_y,with_bias", [(True, True), (True, False), (False, False)])
def test_add_layernorm_matches_torch(device, dtype, rows, D, with_y, with_bias):
    """LayerNorm(x + y + bias) against torch.nn.LayerNorm evaluated in float64 on the same bits."""
    from ar_nanotabpfn_amd.glue import add_layer_norm

    x = randn((rows, D), 1, dtype, 2.0)
    y = randn((rows, D), 2, dtype) if with_y else None
    b = randn((D,), 3, dtype, 0.3) if with_bias else None
    norm = torch.nn.LayerNorm(D)
    with torch.no_grad():
        norm.weight.copy_(randn((D,), 4, torch.float32) * 0.2 + 1)
        norm.bias.copy_(randn((D,), 5, torch.float32) * 0.2)
    norm = norm.to(dtype)
    out = add_layer_norm(x.to(device), y.to(device) if with_y else None, b.to(device) if with_bias else None,
                         norm.to(device))
    t = x.double() + (y.double() if with_y else 0) + (b.double() if with_bias else 0)
    ref = torch.nn.functional.layer_norm(t, (D,), norm.weight.detach().cpu().double(), norm.bias.detach().cpu().double(), norm.eps)
    tol = 2e-5 if dtype == torch.float32 else 2.0 ** -8 * max(1.0, float(ref.abs().max()))  # half an output ulp
    assert out.shape == x.shape and out.dtype == dtype
    assert max_abs(to_np(out), ref.numpy()) <= tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_layernorm_strided_input(device, dtype):
    """x and y as column slices of a wider matrix (row stride != D)."""
    from ar_nanotabpfn_amd.glue import add_layer_norm

    wide = randn((64, 3 * 128), 1, dtype).to(device)
    x, y = wide[:, 128:256], wide[:, 256:]
    norm = torch.nn.LayerNorm(128).to(device=device, dtype=dtype)
    out = add_layer_norm(x, y, None, norm)
    ref = torch.nn.functional.layer_norm((x.double() + y.double()).cpu(), (128,), norm.weight.detach().cpu().double(),
                                         norm.bias.detach().cpu().double(), norm.eps)
    assert max_abs(to_np(out), ref.numpy()) <= (2e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,D", [(1, 4), (2048, 256), (7, 36)])
def test_bias_gelu_matches_torch(device, dtype, rows, D):
    from ar_nanotabpfn_amd.glue import bias_gelu

    x, b = randn((rows, D), 1, dtype, 2.0), randn((D,), 2, dtype, 0.5)
    out = bias_gelu(x.to(device), b.to(device))
    ref = torch.nn.functional.gelu(x.double() + b.double())
    # 16-bit outputs: half an output ulp (2^-8 relative for bf16) at the value's magnitude
    tol = 2e-6 if dtype == torch.float32 else 2.0 ** -8 * max(1.0, float(ref.abs().max()))
    assert max_abs(to_np(out), ref.numpy()) <= tol
    out2 = bias_gelu(x.to(device), None)
    assert max_abs(to_np(out2), torch.nn.functional.gelu(x.double()).numpy()) <= tol


# ----- whole-layer fusions ------------------------------------------------------------------------------


def _ln64(t, norm):
    return torch.nn.functional.layer_norm(t, (t.shape[-1],), norm.weight.detach().cpu().double(),
                                          norm.bias.detach().cpu().double(), norm.eps)


def _mk_norm(D, seed, dtype):
    norm = torch.nn.LayerNorm(D)
    with torch.no_grad():
        norm.weight.copy_(randn((D,), seed, torch.float32) * 0.2 + 1)
        norm.bias.copy_(randn((D,), seed + 1, torch.float32) * 0.2)
    return norm.to(dtype)


@pytest.fixture(params=[16, 32])
def tile_rows(request, tuning):
    """Both tile shapes of the layer kernels (token rows per workgroup): the library picks by row
    count, ARTAB_TILE_ROWS forces one."""
    tuning(ARTAB_TILE_ROWS=request.param)
    return request.param


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,D", [(1, 128), (33, 128), (2048, 256), (70, 512)])
def test_layer_pre_matches_float64(device, tile_rows, dtype, rows, D):
    """y = LN1(x + x Wfo^T), qkv = y Wqkv^T against float64 on the same bits; the reference
    chain rounds y to the storage dtype before the second product, as the kernel does."""
    from ar_nanotabpfn_amd.glue import layer_pre, pack_weight

    x = randn((rows, D), 1, dtype, 1.5)
    w_fo = randn((D, D), 2, dtype, D ** -0.5)
    w_qkv = randn((3 * D, D), 3, dtype, D ** -0.5)
    norm = _mk_norm(D, 4, dtype)
    y, qkv = layer_pre(x.to(device), pack_weight(w_fo.to(device)), norm.to(device), pack_weight(w_qkv.to(device)))
    y_ref = _ln64(x.double() + x.double() @ w_fo.double().t(), norm)
    qkv_ref = y_ref.to(dtype).double() @ w_qkv.double().t()
    assert y.shape == (rows, D) and qkv.shape == (rows, 3 * D) and y.dtype == dtype
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    assert max_abs(to_np(y), y_ref.numpy()) <= 1.02 * ulp * max(1.0, float(y_ref.abs().max()))
    # a flipped rounding of one y element moves a qkv entry by at most ulp*|y|*|w|; allow a few
    assert max_abs(to_np(qkv), qkv_ref.numpy()) <= 2 * ulp * max(1.0, float(qkv_ref.abs().max()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,D,F,with_bias", [(1, 128, 256, True), (33, 128, 128, False), (2048, 256, 256, True),
                                               (70, 512, 256, True), (40, 256, 512, True), (5, 512, 512, False)])
def test_layer_post_matches_float64(device, tile_rows, dtype, rows, D, F, with_bias):
    """x1 = LN2(y + attn Wo^T); out = LN3(x1 + gelu(x1 W1^T + b1) W2^T + b2) against float64
    with the kernel's two intermediate roundings."""
    from ar_nanotabpfn_amd.glue import layer_post, pack_weight

    attn = randn((rows, D), 1, dtype)
    y = randn((rows, D), 2, dtype, 1.5)
    w_o = randn((D, D), 3, dtype, D ** -0.5)
    lin1, lin2 = torch.nn.Linear(D, F, bias=with_bias), torch.nn.Linear(F, D, bias=with_bias)
    with torch.no_grad():
        lin1.weight.copy_(randn((F, D), 4, torch.float32, D ** -0.5))
        lin2.weight.copy_(randn((D, F), 5, torch.float32, F ** -0.5))
        if with_bias:
            lin1.bias.copy_(randn((F,), 6, torch.float32, 0.3))
            lin2.bias.copy_(randn((D,), 7, torch.float32, 0.3))
    lin1, lin2 = lin1.to(dtype), lin2.to(dtype)
    n2, n3 = _mk_norm(D, 8, dtype), _mk_norm(D, 10, dtype)
    lin1, lin2 = lin1.to(device), lin2.to(device)
    out = layer_post(attn.to(device), y.to(device), pack_weight(w_o.to(device)), n2.to(device),
                     pack_weight(lin1.weight), lin1.bias, pack_weight(lin2.weight), lin2.bias, n3.to(device))
    d = lambda t: t.detach().cpu().double()  # noqa: E731
    x1 = _ln64(y.double() + attn.double() @ w_o.double().t(), n2)
    x1r = x1.to(dtype).double()
    h = x1r @ d(lin1.weight).t() + (d(lin1.bias) if with_bias else 0)
    hr = torch.nn.functional.gelu(h).to(dtype).double()
    # the residual entering LN3 is the rounded copy of x1 staged for the product
    ref = _ln64(x1r + hr @ d(lin2.weight).t() + (d(lin2.bias) if with_bias else 0), n3)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    assert out.shape == (rows, D) and out.dtype == dtype
    assert max_abs(to_np(out), ref.numpy()) <= 3 * ulp * max(1.0, float(ref.abs().max()))


def test_layer_fusion_strided_inputs_and_errors(device):
    """attn given as the [B,N,H,Dh]-backed view the attention kernels return, x as a column
    slice; unsupported widths and dtypes raise."""
    from ar_nanotabpfn_amd.glue import layer_fusable, layer_pre, pack_weight

    dtype, D = torch.bfloat16, 256
    wide = randn((96, 2 * D), 1, dtype).to(device)
    x = wide[:, D:]
    w_fo = pack_weight(randn((D, D), 2, dtype, D ** -0.5).to(device))
    w_qkv = pack_weight(randn((3 * D, D), 3, dtype, D ** -0.5).to(device))
    norm = _mk_norm(D, 4, dtype).to(device)
    y, qkv = layer_pre(x, w_fo, norm, w_qkv)
    y2, qkv2 = layer_pre(x.contiguous(), w_fo, norm, w_qkv)
    assert torch.equal(y, y2) and torch.equal(qkv, qkv2)
    assert not layer_fusable(x, 96, 256) and not layer_fusable(x.float(), 256, 256) and layer_fusable(x, 256, 512)
    assert not layer_fusable(x.cpu(), 256, 256)
    with pytest.raises((ValueError, RuntimeError)):
        layer_pre(randn((4, 96), 1, dtype).to(device), randn((96, 96), 2, dtype).to(device),
                  torch.nn.LayerNorm(96).to(device=device, dtype=dtype), randn((288, 96), 3, dtype).to(device))
    with pytest.raises((ValueError, RuntimeError)):
        layer_pre(x.float(), w_fo.float(), norm.float(), w_qkv.float())
    with pytest.raises((ValueError, RuntimeError)):
        pack_weight(randn((40, 64), 1, dtype).to(device))  # N % 32 != 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,K", [(32, 16), (768, 256), (256, 512)])
def test_pack_weight_layout(device, dtype, N, K):
    """packed[blk][ks][lane][e] = W[32*blk + lane%32][16*ks + 8*(lane/32) + e], bit-exact."""
    from ar_nanotabpfn_amd.glue import pack_weight

    w = randn((N, K), 1, dtype)
    packed = pack_weight(w.to(device)).cpu()
    ref = w.view(N // 32, 32, K // 16, 2, 8).permute(0, 2, 3, 1, 4).reshape(N // 32, K // 16, 64, 8)
    assert packed.shape == ref.shape and torch.equal(packed, ref)


@pytest.mark.parametrize("D,F,H", [(128, 256, 4), (256, 256, 8), (512, 256, 16)])
def test_layer_fused_equals_unfused_composition(device, monkeypatch, D, F, H):
    """TwoStageTransformerLayer.pre_attention / finish: the two-launch path against the path
    composed from GEMMs and the row-wise kernels, same weights, bf16 tolerance."""
    from ar_nanotabpfn_amd import model as m

    torch.manual_seed(0)
    layer = m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=torch.bfloat16)
    x = randn((64, 2, D), 1, torch.bfloat16, 1.0).to(device)
    attn = randn((64, 2, H, D // H), 2, torch.bfloat16).to(device).transpose(1, 2)
    y_f, q_f, k_f, v_f = layer.pre_attention(x)
    out_f = layer.finish(y_f, attn)
    monkeypatch.setattr(m, "layer_fusable", lambda *a: False)
    y_u, q_u, k_u, v_u = layer.pre_attention(x)
    out_u = layer.finish(y_u, attn)
    for a, b in ((y_f, y_u), (q_f, q_u), (k_f, k_u), (v_f, v_u), (out_f, out_u)):
        assert a.shape == b.shape
        assert max_abs(to_np(a), to_np(b)) <= 4e-2  # two 16-bit chains with different rounding points


# ----- decode-step tail: norm + head + draw + next embedding ------------------------------------------


def _tail_model(D, F, K, bs, dtype, device, seed=0):
    from ar_nanotabpfn_amd import model as m

    torch.manual_seed(seed)
    net = m.ARTabPFN(d_model=D, n_heads=4, n_layers=1, d_ff=F, num_features=3, buffer_size=bs, num_components=K)
    with torch.no_grad():  # make every learned vector non-trivial
        for p in list(net.embedder.parameters()) + list(net.head.parameters()) + [net.ar_tokens]:
            p.add_(0.3 * torch.randn_like(p))
        net.backbone.norm.weight.add_(0.2 * torch.randn(D))
        net.backbone.norm.bias.add_(0.2 * torch.randn(D))
    return net.to(device=device, dtype=dtype)


def _tail_reference(net, x_last, x_mean, u, n, t, dtype):
    """float64 restatement of backbone.norm -> head -> inverse-CDF pick -> draw -> embeddings,
    with the kernel's rounding points (z and gelu output rounded to the storage dtype)."""
    d = lambda p: p.detach().cpu().double()  # noqa: E731
    rd = lambda v: v.to(dtype).double()  # noqa: E731
    B, Nt = x_mean.shape
    norm, head, emb = net.backbone.norm, net.head, net.embedder
    z = rd(torch.nn.functional.layer_norm(x_last.double(), (x_last.shape[-1],), d(norm.weight), d(norm.bias), norm.eps))
    h = rd(torch.nn.functional.gelu(z @ d(head.head[0].weight).t() + d(head.head[0].bias)))
    raw = (h @ d(head.head[2].weight).t() + d(head.head[2].bias)).view(B, head.num_components, 3)
    w = torch.softmax(raw[:, :, 2] + d(head.weight_bias), dim=1)
    cdf = torch.cumsum(w, dim=1)
    comp = (cdf > u[:, None]).double().argmax(dim=1)
    margin = (cdf[:, :-1] - u[:, None]).abs().min(dim=1).values
    rows = torch.arange(B)
    mean = raw[rows, comp, 0] + d(head.mean_bias)[comp]
    std = torch.nn.functional.softplus(raw[rows, comp, 1] + d(head.std_bias)[comp]).clamp(max=2.0) + head.std_min
    y = rd(mean + std * n)
    bs = net.ar_tokens.shape[0]
    wx, bx = d(emb.x_embed.weight).view(-1), d(emb.x_embed.bias)
    wy, by = d(emb.y_embed.weight).view(-1), d(emb.y_embed.bias)
    mk = d(emb.marker_embed.weight)
    buf = x_mean[:, t, None].double() * wx + bx + y[:, None] * wy + by + mk[2] + d(net.ar_tokens)[(t + 1) % bs]
    tgt = x_mean[:, min(t + 1, Nt - 1), None].double() * wx + bx + mk[0]
    return y, torch.stack([buf, tgt], dim=1), margin


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,D,F,K,t", [(70, 128, 128, 5, 3), (1024, 256, 256, 5, 1), (33, 512, 256, 10, 6),
                                       (40, 256, 512, 3, 7)])
def test_decode_sample_embed_matches_float64(device, tile_rows, dtype, B, D, F, K, t):
    from ar_nanotabpfn_amd.glue import SampleEmbedStep

    Nt, bs = 8, 5
    net = _tail_model(D, F, K, bs, dtype, device)
    g = torch.Generator().manual_seed(1)
    x_last = torch.randn(B, 2, D, generator=g).to(dtype)
    x_mean = (0.5 * torch.randn(B, Nt, generator=g)).to(dtype)
    u = torch.rand(Nt, B, generator=g)
    n = torch.randn(Nt, B, generator=g)
    step = torch.tensor([t], dtype=torch.int32, device=device)
    preds = torch.full((B, Nt), 7.0, device=device, dtype=dtype)
    emb = torch.zeros(B, 2, D, device=device, dtype=dtype)
    assert SampleEmbedStep.supported(net.embedder, net.backbone, net.head, emb)
    tail = SampleEmbedStep(net.embedder, net.backbone, net.head, net.ar_tokens, x_mean.to(device), u.to(device),
                           n.to(device), step, preds, emb)
    tail(x_last.to(device))
    y_ref, emb_ref, margin = _tail_reference(net, x_last[:, 1], x_mean, u[t].double(), n[t].double(), t, dtype)
    ok = margin > 2e-2  # rows whose uniform variate sits on a component boundary may pick the neighbour
    assert ok.float().mean() > 0.8
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    got = preds.cpu().double()
    assert torch.all(got[:, [c for c in range(Nt) if c != t]] == 7.0)  # only column t is written
    # the head runs on 16-bit z and h: allow a few output ulps on top of the final rounding
    tol_y = 6 * ulp * max(1.0, float(y_ref.abs().max()))
    assert float((got[:, t] - y_ref).abs()[ok].max()) <= tol_y
    # embeddings are compared given the kernel's own draw
    y_used = got[:, t]
    emb_fix = emb_ref.clone()
    wy = net.embedder.y_embed.weight.detach().cpu().double().view(-1)
    emb_fix[:, 0] += (y_used - y_ref)[:, None] * wy
    assert float((emb.cpu().double() - emb_fix).abs().max()) <= 1.02 * ulp * max(1.0, float(emb_fix.abs().max()))


def test_decode_sample_embed_step_out_of_range_is_noop(device):
    from ar_nanotabpfn_amd.glue import SampleEmbedStep

    dtype, B, D, Nt = torch.bfloat16, 16, 128, 4
    net = _tail_model(D, 128, 5, 3, dtype, device)
    step = torch.tensor([Nt], dtype=torch.int32, device=device)
    preds = torch.full((B, Nt), 7.0, device=device, dtype=dtype)
    emb = torch.full((B, 2, D), 3.0, device=device, dtype=dtype)
    tail = SampleEmbedStep(net.embedder, net.backbone, net.head, net.ar_tokens,
                           torch.zeros(B, Nt, device=device, dtype=dtype), torch.rand(Nt, B, device=device),
                           torch.randn(Nt, B, device=device), step, preds, emb)
    tail(torch.randn(B, 2, D, device=device).to(dtype))
    assert torch.all(preds == 7.0) and torch.all(emb == 3.0)
    step.fill_(-1)
    tail(torch.randn(B, 2, D, device=device).to(dtype))
    assert torch.all(preds == 7.0) and torch.all(emb == 3.0)


def test_decode_sample_embed_advances_loop_counters(device, tile_rows):
    """With ``advance`` the launch moves the caller's loop counters on by one, once, whatever the
    number of workgroups, writes column t of every call, and leaves its ticket word at zero; an
    out-of-range step index neither samples nor advances."""
    from ar_nanotabpfn_amd.glue import SampleEmbedStep

    dtype, B, D, Nt = torch.bfloat16, 200, 128, 6
    net = _tail_model(D, 128, 5, 3, dtype, device)
    counters = torch.tensor([1, 0, 40], dtype=torch.int32, device=device)  # (t, n_buf, anything else)
    preds = torch.full((B, Nt), 7.0, device=device, dtype=dtype)
    emb = torch.zeros((B, 2, D), device=device, dtype=dtype)
    tail = SampleEmbedStep(net.embedder, net.backbone, net.head, net.ar_tokens,
                           torch.zeros(B, Nt, device=device, dtype=dtype), torch.rand(Nt, B, device=device),
                           torch.randn(Nt, B, device=device), counters[0:1], preds, emb, advance=counters)
    x = torch.randn(B, 2, D, device=device).to(dtype)
    for n in range(1, Nt):
        tail(x)
        torch.cuda.synchronize()
        assert counters.tolist() == [1 + n, n, 40 + n]
        assert int(tail._keep["ticket"].item()) == 0
        assert torch.all(preds[:, n] != 7.0) and (n + 1 == Nt or torch.all(preds[:, n + 1 :] == 7.0))
    before = preds.clone()
    tail(x)  # t == Nt: out of range
    torch.cuda.synchronize()
    assert counters.tolist() == [Nt, Nt - 1, 40 + Nt - 1] and torch.equal(preds, before)


def test_decode_sample_embed_component_frequencies(device):
    """With many trajectories sharing one head input, the picked components follow the mixture
    weights and the draws have the mixture's mean (law of the sampler, not a bitwise check)."""
    from ar_nanotabpfn_amd.glue import SampleEmbedStep

    dtype, B, D, F, K, Nt = torch.bfloat16, 32768, 128, 128, 5, 2
    net = _tail_model(D, F, K, 3, dtype, device, seed=3)
    with torch.no_grad():
        net.head.head[2].weight.mul_(0.05)  # mild logits: no component so rare that the sample variance hinges on it
    g = torch.Generator().manual_seed(5)
    x_row = torch.randn(1, 2, D, generator=g).to(dtype).expand(B, -1, -1).contiguous()
    u, n = torch.rand(Nt, B, generator=g), torch.randn(Nt, B, generator=g)
    step = torch.tensor([1], dtype=torch.int32, device=device)
    preds = torch.zeros(B, Nt, device=device, dtype=torch.bfloat16)
    emb = torch.zeros(B, 2, D, device=device, dtype=dtype)
    tail = SampleEmbedStep(net.embedder, net.backbone, net.head, net.ar_tokens,
                           torch.zeros(B, Nt, device=device, dtype=dtype), u.to(device), n.to(device), step, preds, emb)
    tail(x_row.to(device))
    with torch.no_grad():
        mean, std, weight, _ = net.head._parameterize(net.backbone.norm(x_row[:1, 1:2].to(device)))
    mean, std, weight = (v.float().cpu().view(-1) for v in (mean, std, weight))
    assert float(weight.min()) > 0.02
    mix_mean = float((weight * mean).sum())
    mix_var = float((weight * (std ** 2 + mean ** 2)).sum()) - mix_mean ** 2
    y = preds[:, 1].float().cpu()
    assert abs(float(y.mean()) - mix_mean) <= 5 * (mix_var / B) ** 0.5 + 2e-2
    assert abs(float(y.var()) - mix_var) <= 0.1 * mix_var + 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,D,F,H", [(33, 128, 256, 4), (2048, 256, 256, 8), (70, 512, 256, 16), (40, 256, 512, 8)])
def test_layer_post_pre_equals_post_then_pre(device, tile_rows, dtype, rows, D, F, H):
    """The one-launch layer boundary must give bit for bit what the two launches give: the
    layer output between them is rounded to the storage type in both."""
    from ar_nanotabpfn_amd import model as m

    torch.manual_seed(1)
    la = m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=dtype)
    lb = m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=dtype)
    B = rows  # one row per "batch" entry keeps the shapes general
    y = randn((B, 1, D), 2, dtype, 1.0).to(device)
    attn = randn((B, 1, H, D // H), 3, dtype).to(device).transpose(1, 2)
    y2, q2, k2, v2 = la.finish_then_pre(y, attn, lb)
    y1, q1, k1, v1 = lb.pre_attention(la.finish(y, attn))
    for a, b in ((y1, y2), (q1, q2), (k1, k2), (v1, v2)):
        assert a.shape == b.shape and torch.equal(a, b)


@pytest.mark.parametrize("fetchers", [0, 3, 32])
@pytest.mark.parametrize("rows", [16 * 13 + 5, 16 * 8])
def test_layer_post_pre_with_weight_fetching_workgroups(device, tuning, fetchers, rows):
    """A layer-boundary launch may carry workgroups that only fetch weights into the L2 (per XCD,
    behind the workgroups that own rows): whatever their number, and whether or not the row tiles
    end on a multiple of the 8 XCDs, the results are those of the two separate launches."""
    from ar_nanotabpfn_amd import model as m

    D, F, H, dtype = 256, 256, 8, torch.bfloat16
    torch.manual_seed(1)
    la = m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=dtype)
    lb = m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=dtype)
    y = randn((rows, 1, D), 2, dtype, 1.0).to(device)
    attn = randn((rows, 1, H, D // H), 3, dtype).to(device).transpose(1, 2)
    ref = lb.pre_attention(la.finish(y, attn))
    tuning(ARTAB_LAYER_FETCHERS=fetchers, ARTAB_TILE_ROWS=16)
    got = la.finish_then_pre(y, attn, lb)
    for a, b in zip(ref, got):
        assert a.shape == b.shape and torch.equal(a, b)


def test_layer_post_pre_falls_back_when_not_covered(device):
    """float32 layers (or widths outside the fused kernels) compose the same result from the
    separate pieces."""
    from ar_nanotabpfn_amd import model as m

    torch.manual_seed(1)
    la = m.TwoStageTransformerLayer(64, 2, 64).to(device)
    lb = m.TwoStageTransformerLayer(64, 2, 64).to(device)
    y = randn((8, 2, 64), 2, torch.float32).to(device)
    attn = randn((8, 2, 2, 32), 3, torch.float32).to(device).transpose(1, 2)
    got = la.finish_then_pre(y, attn, lb)
    ref = lb.pre_attention(la.finish(y, attn))
    for a, b in zip(got, ref):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,Lq,Nc,n_buf,cap", [(64, 4, 2, 4096, 9, 16), (33, 8, 2, 2048, 0, 8), (40, 8, 1, 4096, 5, 8)])
def test_decode_partials_merged_in_layer_kernel(device, tuning, tile_rows, dtype, B, H, Lq, Nc, n_buf, cap):
    """decode_attention(leave_partials=True) + the layer kernels that merge the partials while
    loading, against the merged attention output fed to the same kernels: the merge is the same
    arithmetic rounded at the same point, so the results must agree bit for bit.  (Both legs on the
    general route: the one-launch kernel merges float32 partials and differs in the last bit.)"""
    from ar_nanotabpfn_amd import attention_kernels as ak
    from ar_nanotabpfn_amd import model as m

    tuning(ARTAB_SMALL=0)

    D, Dh, F = 32 * H, 32, 256
    torch.manual_seed(2)
    la = m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=dtype)
    lb = m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=dtype)
    q, k_ctx, v_ctx = (t.to(device) for t in _ctx_inputs(B, H, Lq, Nc, Dh, dtype, seed=5, scale=0.6))
    k_cache, v_cache = randn((B, H, cap, Dh), 6, dtype, 0.6).to(device), randn((B, H, cap, Dh), 7, dtype, 0.6).to(device)
    k_new = randn((B, H, 1, Dh), 8, dtype, 0.6).to(device) if Lq == 2 else None
    v_new = randn((B, H, 1, Dh), 9, dtype, 0.6).to(device) if Lq == 2 else None
    y = randn((B, Lq, D), 10, dtype, 1.0).to(device)
    side = torch.cuda.Stream(device=device)

    kc, vc = k_cache.clone(), v_cache.clone()
    merged = ak.decode_attention(q, k_ctx, v_ctx, kc, vc, n_buf, k_new, v_new, side_stream=side)
    ref_post = la.finish(y, merged)
    ref_mid = la.finish_then_pre(y, merged, lb)

    kc2, vc2 = k_cache.clone(), v_cache.clone()
    parts = ak.decode_attention(q, k_ctx, v_ctx, kc2, vc2, n_buf, k_new, v_new, side_stream=side, leave_partials=True)
    if n_buf + (Lq - 1) == 0:
        assert isinstance(parts, torch.Tensor)  # nothing to merge: the finished tensor comes back
        return
    assert isinstance(parts, ak.AttentionPartials) and parts.shape == (B, H, Lq, Dh)
    got_post = la.finish(y, parts)
    parts = ak.decode_attention(q, k_ctx, v_ctx, k_cache.clone(), v_cache.clone(), n_buf, k_new, v_new,
                                side_stream=side, leave_partials=True)
    got_mid = la.finish_then_pre(y, parts, lb)
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)
    assert torch.equal(got_post, ref_post)
    for a, b in zip(got_mid, ref_mid):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,D,F,H,Nc,n_buf,cap,partials", [
    (64, 128, 128, 4, 256, 5, 16, True),     # whole workgroups
    (200, 256, 256, 8, 4096, 9, 16, True),   # split context, the shape of configs[3]'s layers
    (37, 256, 256, 8, 300, 0, 8, True),      # ragged last workgroup (5 of 8 trajectories), the new row alone
    (1030, 128, 256, 4, 128, 3, 8, True),    # more than eight 16-row tiles: the contraction starts rotate
    (21, 512, 256, 16, 200, 2, 8, True),     # matrices deeper than the prefetch window
    (40, 128, 128, 4, 64, 0, 8, False),      # attention output given as a tensor (first target: context only)
])
def test_decode_step_boundary_equals_its_three_launches(device, tuning, dtype, B, D, F, H, Nc, n_buf, cap, partials):
    """artab_decode_step_boundary against artab_layer_post(_from_partials) on the target rows,
    artab_decode_sample_embed and artab_layer_pre launched one after the other: predictions,
    embedding, the next step's feature stage and projections, and the loop counters, bit for bit."""
    from ar_nanotabpfn_amd import attention_kernels as ak
    from ar_nanotabpfn_amd import model as m
    from ar_nanotabpfn_amd.glue import DecodeStepBoundary, SampleEmbedStep

    tuning(ARTAB_SMALL=0)
    Dh, Nt, K = D // H, 6, 5
    assert Dh == 32
    torch.manual_seed(4)
    net = m.ARTabPFN(d_model=D, n_heads=H, n_layers=2, d_ff=F, num_features=3, buffer_size=3, num_components=K)
    with torch.no_grad():
        for p in list(net.embedder.parameters()) + list(net.head.parameters()) + [net.ar_tokens]:
            p.add_(0.3 * torch.randn_like(p))
        for layer in net.backbone.layers:
            for norm in (layer.norm1, layer.norm2, layer.norm3):
                norm.weight.add_(0.2 * torch.randn(D))
                norm.bias.add_(0.2 * torch.randn(D))
    # the head's hidden width is the layers' feed-forward width in this model family
    net = net.to(device=device, dtype=dtype)
    first, last = net.backbone.layers[0], net.backbone.layers[1]
    assert net.head.head[0].out_features == F

    q, k_ctx, v_ctx = (t.to(device) for t in _ctx_inputs(B, H, 1, Nc, Dh, dtype, seed=5, scale=0.6))
    k_cache, v_cache = randn((B, H, cap, Dh), 6, dtype, 0.6).to(device), randn((B, H, cap, Dh), 7, dtype, 0.6).to(device)
    k_new, v_new = randn((B, H, 1, Dh), 8, dtype, 0.6).to(device), randn((B, H, 1, Dh), 9, dtype, 0.6).to(device)
    y_rows = randn((B, 2, D), 10, dtype, 1.0).to(device)
    y_tgt = y_rows[:, 1:2]  # the target rows: row stride 2 D
    side = torch.cuda.Stream(device=device)
    x_mean = randn((B, Nt), 11, dtype, 1.0).to(device)
    u, n = torch.rand(Nt, B, device=device), torch.randn(Nt, B, device=device)

    def attention():
        if not partials:
            return ak.context_attention(q, k_ctx, v_ctx)[0]
        out = ak.decode_attention(q, k_ctx, v_ctx, k_cache.clone(), v_cache.clone(), n_buf, k_new, v_new,
                                  side_stream=side, leave_partials=True)
        assert isinstance(out, ak.AttentionPartials)
        return out

    def make_tail():
        counters = torch.tensor([2, 1], dtype=torch.int32, device=device)
        preds = torch.full((B, Nt), 7.0, device=device, dtype=dtype)
        emb = torch.zeros((B, 2, D), device=device, dtype=dtype)
        tail = SampleEmbedStep(net.embedder, net.backbone, net.head, net.ar_tokens, x_mean, u, n, counters[0:1],
                               preds, emb, advance=counters)
        return tail, counters, preds, emb

    # three launches
    tail, counters, preds, emb = make_tail()
    x_last = last.finish(y_tgt, attention())
    tail(x_last)
    ref_state = first.pre_attention(emb)
    torch.cuda.synchronize()

    # one launch
    tail2, counters2, preds2, emb2 = make_tail()
    assert DecodeStepBoundary.supported(tail2, first, last, y_rows) == (D <= DecodeStepBoundary.MAX_WIDTH)
    boundary = DecodeStepBoundary(tail2, first, last, torch.zeros((B, 2, D), device=device, dtype=dtype),
                                  torch.zeros((B, 2, 3 * D), device=device, dtype=dtype))
    boundary(y_tgt, attention())
    torch.cuda.synchronize()
    assert counters2.tolist() == counters.tolist() == [3, 2]
    assert int(tail2._keep["ticket"].item()) == 0
    assert torch.equal(preds2, preds) and torch.all(preds2[:, 3:] == 7.0) and not torch.all(preds2[:, 2] == 7.0)
    assert torch.equal(emb2, emb)
    for got, ref in zip(boundary.state, ref_state):
        assert got.shape == ref.shape and torch.equal(got, ref)
    # the state that reset() builds from an embedding is the same again
    boundary.y_next.zero_()
    boundary.qkv_next.zero_()
    boundary.load_state(emb)
    for got, ref in zip(boundary.state, ref_state):
        assert torch.equal(got, ref)
    # an out-of-range step index: nothing is written, nothing advances
    counters2[0] = Nt
    before = (preds2.clone(), emb2.clone(), boundary.y_next.clone(), boundary.qkv_next.clone())
    boundary(y_tgt, attention())
    torch.cuda.synchronize()
    assert counters2.tolist() == [Nt, 2]
    for a, b in zip(before, (preds2, emb2, boundary.y_next, boundary.qkv_next)):
        assert torch.equal(a, b)


def test_queue_order_wait_gives_up_after_its_time_limit(device):
    """A wait whose signal never comes (forced from the host: nothing is launched on the other
    stream) ends after its time limit, counts itself in `failed`, and every later wait falls
    through at once; the streams stay usable."""
    import time

    ak = _ak()
    order = ak.QueueOrder(device)
    main = torch.cuda.current_stream(device)
    order.wait(order.SIDE, main, timeout_us=2000)      # needs counter main >= 1: never signalled
    main.synchronize()
    assert order.failed() == 1
    t0 = time.time()
    for _ in range(20):
        order.wait(order.SIDE, main, timeout_us=10_000_000)  # falls through: `failed` is set
    main.synchronize()
    assert time.time() - t0 < 5.0 and order.failed() == 21
    order.reset()
    order.wait(order.MAIN, main, timeout_us=2000)      # counter side >= counter main (0 >= 0): no wait
    order.signal(order.MAIN, main)
    order.signal(order.SIDE, main)
    order.wait(order.MAIN, main, timeout_us=2000)      # 1 >= 1
    main.synchronize()
    assert order.failed() == 0
    assert order.state[0].item() == 1 and order.state[32].item() == 1


def test_queue_order_argument_checks(device):
    ak = _ak()
    order = ak.QueueOrder(device)
    main = torch.cuda.current_stream(device)
    with pytest.raises(ValueError):
        order.signal(2, main)
    q, k_ctx, v_ctx = (t.to(device) for t in _ctx_inputs(4, 2, 2, 64, 64, torch.bfloat16, seed=1))
    kc = torch.zeros((4, 2, 8, 64), device=device, dtype=torch.bfloat16)
    kn = torch.zeros((4, 2, 1, 64), device=device, dtype=torch.bfloat16)
    side = torch.cuda.Stream(device=device)
    with pytest.raises(ValueError):  # needs a side stream and partials
        ak.decode_attention(q, k_ctx, v_ctx, kc, kc.clone(), 0, kn, kn.clone(), order=order)
    with pytest.raises(RuntimeError):  # head_dim 64 has no streaming buffer pass: refused before any launch
        ak.decode_attention(q, k_ctx, v_ctx, kc, kc.clone(), 0, kn, kn.clone(), side_stream=side,
                            leave_partials=True, order=order)
    main.synchronize()
    assert order.failed() == 0 and order.state[0].item() == 0


@pytest.mark.parametrize("absorb", [False, True])
@pytest.mark.parametrize("B,H,Nc,cap", [(64, 8, 2048, 8), (600, 8, 1024, 12)])
def test_decode_attention_ordered_by_counters_equals_event_ordered(device, tuning, B, H, Nc, cap, absorb):
    """A run of decode steps whose two streams are ordered by device-side counters (one fork
    before the first call, one join after the last) against the same steps ordered by two events
    per call: same partials (bit for bit after the merge), same cache, no wait timed out."""
    ak = _ak()
    tuning(ARTAB_SMALL=0)  # the event-ordered leg on the two-stream route as well
    dtype, D = torch.bfloat16, 32
    q0, k_ctx, v_ctx = (t.to(device) for t in _ctx_inputs(B, H, 2, Nc, D, dtype, seed=1, scale=0.6))
    k_ref, v_ref = torch.zeros((B, H, cap, D), device=device, dtype=dtype), torch.zeros((B, H, cap, D), device=device, dtype=dtype)
    k_ord, v_ord = k_ref.clone(), v_ref.clone()
    main = torch.cuda.current_stream(device)
    side, concurrent = ak.concurrent_stream(device, main)
    if not concurrent:
        pytest.skip("no second stream runs side by side with the current one here: counters cannot order them")
    order = ak.QueueOrder(device)
    order.consumer_waits = absorb  # True: the merge launch waits for the side counter itself
    steps = cap - 1
    qs = [(q0 * (1.0 + 0.1 * s)).to(dtype) for s in range(steps)]
    news = [(randn((B, H, 1, D), 10 + s, dtype, 0.6).to(device), randn((B, H, 1, D), 40 + s, dtype, 0.6).to(device))
            for s in range(steps)]
    expect = []
    for s in range(steps):
        expect.append(ak.decode_attention(qs[s], k_ctx, v_ctx, k_ref, v_ref, s, *news[s], side_stream=side))
    torch.cuda.synchronize()
    got = []
    side.wait_stream(main)
    for s in range(steps):
        parts = ak.decode_attention(qs[s], k_ctx, v_ctx, k_ord, v_ord, s, *news[s], side_stream=side,
                                    leave_partials=True, order=order)
        got.append(parts.merged())  # on the main stream, behind the wait on the side counter
    main.wait_stream(side)
    torch.cuda.synchronize()
    assert order.failed() == 0
    assert order.state[0].item() == steps and order.state[32].item() == steps
    for s in range(steps):
        assert torch.equal(got[s], expect[s]), f"step {s}"
    assert torch.equal(k_ord, k_ref) and torch.equal(v_ord, v_ref)


@pytest.mark.parametrize("gate_launch", [0, 1])
@pytest.mark.parametrize("B,H,Nc,cap", [(64, 4, 4096, 8), (200, 8, 1024, 6)])
def test_layer_kernels_wait_for_the_side_queue_themselves(device, tuning, tile_rows, gate_launch, B, H, Nc, cap):
    """Three layers of a decode step whose streams are ordered by counters, with the main
    stream's wait done by the layer kernels themselves (they wait for the buffer pass before
    they read the partials), repeated for several steps, against the event-ordered launches: bit
    for bit.  gate_launch=1 forces the wait into a launch of its own (what a grid larger than half
    the chip gets)."""
    from ar_nanotabpfn_amd import attention_kernels as ak
    from ar_nanotabpfn_amd import model as m

    tuning(ARTAB_ORDER_GATE_LAUNCH=gate_launch)
    dtype, Dh, F, n_layers = torch.bfloat16, 32, 128, 3
    D = H * Dh
    torch.manual_seed(3)
    layers = [m.TwoStageTransformerLayer(D, H, F).to(device=device, dtype=dtype) for _ in range(n_layers)]
    ctx = [tuple(x.to(device) for x in _ctx_inputs(1, H, 1, Nc, Dh, dtype, seed=20 + i, scale=0.6)[1:]) for i in range(n_layers)]
    main = torch.cuda.current_stream(device)
    side, concurrent = ak.concurrent_stream(device, main)
    if not concurrent:
        pytest.skip("no second stream runs side by side with the current one here: counters cannot order them")
    order = ak.QueueOrder(device)
    steps = cap - 1
    xs = [randn((B, 2, D), 50 + s, dtype, 1.0).to(device) for s in range(steps)]

    def run(ordered):
        caches = [(torch.zeros((B, H, cap, Dh), device=device, dtype=dtype), torch.zeros((B, H, cap, Dh), device=device, dtype=dtype))
                  for _ in range(n_layers)]
        outs = []
        if ordered:
            side.wait_stream(main)
        for s in range(steps):
            state = layers[0].pre_attention(xs[s])
            for i, layer in enumerate(layers):
                y, q, k, v = state
                attn = ak.decode_attention(q, ctx[i][0], ctx[i][1], caches[i][0], caches[i][1], s, k[:, :, 0:1], v[:, :, 0:1],
                                           side_stream=side, leave_partials=True, order=order if ordered else None)
                assert isinstance(attn, ak.AttentionPartials)
                if i + 1 == n_layers:
                    outs.append(layer.finish(y, attn))
                else:
                    state = layer.finish_then_pre(y, attn, layers[i + 1])
        if ordered:
            main.wait_stream(side)
        torch.cuda.synchronize()
        return outs, caches

    ref_out, ref_caches = run(False)
    got_out, got_caches = run(True)
    assert order.failed() == 0
    assert order.state[0].item() == steps * n_layers and order.state[32].item() == steps * n_layers
    for s in range(steps):
        assert torch.equal(got_out[s], ref_out[s]), f"step {s}"
    for (k0, v0), (k1, v1) in zip(ref_caches, got_caches):
        assert torch.equal(k0, k1) and torch.equal(v0, v1)


# ----- a buffer length read from device memory never takes an access outside the cache ---------------


@pytest.mark.parametrize("dtype,schedule", [(torch.float32, "portable"), (torch.bfloat16, "sequential"),
                                            (torch.bfloat16, "two streams")])
@pytest.mark.parametrize("cell", [8, 9, 100, -3])
def test_decode_device_length_beyond_capacity_stays_inside_the_cache(device, dtype, schedule, cell):
    """A recorded launch replayed once more than the cache has slots (or a cell that was never
    reset) hands the kernels a length the host never validated.  They clamp it to the capacity:
    rows behind the cache keep their contents, a new row that has no slot is not stored, and the
    call completes.  capacity = 8 rows; the cache is a view into a larger tensor whose remaining
    rows are the guard."""
    ak = _ak()
    B, H, D, Nc, cap, guard = 33, 8, 32, 700, 8, 4
    q = randn((B, H, 2, D), 1, dtype, 0.5).to(device)
    kc, vc = randn((H, Nc, D), 2, dtype, 0.5).to(device), randn((H, Nc, D), 3, dtype, 0.5).to(device)
    kbig = randn((B, H, cap + guard, D), 4, dtype, 0.5).to(device)
    vbig = randn((B, H, cap + guard, D), 5, dtype, 0.5).to(device)
    kb, vb = kbig[:, :, :cap], vbig[:, :, :cap]
    k0, v0 = kbig.clone(), vbig.clone()
    kn, vn = randn((B, H, 1, D), 6, dtype, 0.5).to(device), randn((B, H, 1, D), 7, dtype, 0.5).to(device)
    nbuf = torch.full((1,), cell, device=device, dtype=torch.int32)
    side = torch.cuda.Stream(device=device) if schedule == "two streams" else None
    out = ak.decode_attention(q, kc, vc, kb, vb, cap - 1, kn, vn, n_buf_device=nbuf, side_stream=side)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert torch.equal(kbig[:, :, cap:], k0[:, :, cap:]) and torch.equal(vbig[:, :, cap:], v0[:, :, cap:])
    # nothing inside the cache changed either: no slot exists for the new row at these lengths
    assert torch.equal(kbig, k0) and torch.equal(vbig, v0)
    # with the largest valid length the same call does append, in the last slot
    nbuf.fill_(cap - 1)
    out = ak.decode_attention(q, kc, vc, kb, vb, cap - 1, kn, vn, n_buf_device=nbuf, side_stream=side)
    torch.cuda.synchronize()
    assert torch.equal(kbig[:, :, cap - 1], kn[:, :, 0]) and torch.equal(kbig[:, :, cap:], k0[:, :, cap:])
    ref, _, _ = ao.decode_step_attention(to_np(q), to_np(kc), to_np(vc), to_np(k0[:, :, : cap - 1]),
                                         to_np(v0[:, :, : cap - 1]), to_np(kn), to_np(vn))
    assert max_abs(to_np(out), ref) <= out_tol(dtype)
