#!/usr/bin/env python3
"""Benchmark of the AR-TabPFN attention hot path on one MI355X.

Workload (BASELINE.json configs[3], the configuration the headline metric is quoted
on): long-context autoregressive sampling with the 12-layer d_model=256 / 8-head
(head_dim 32) bf16 model, one shared context of N_ctx=16384 rows, B=1024
trajectories.  One *step* is one decode step: every trajectory advances by one
target through all 12 layers (projections, shared-context decode attention with the
in-place buffer append and LSE merge, FFN, mixture head, sampling).  Steps are timed
from the first target on, so step t attends to t-1 buffer rows; the default K=256
is the whole configuration.  The context prefill runs before the timed region and is
reported separately.

Prints one JSON line:
  metric/value   target-steps per second over the K timed steps (inputs resident in HBM)
  roofline       the dominant kernel (MFMA context pass of the decode attention):
                 algorithmic flops 4*B*H*Lq*N_ctx*Dh per launch over its average
                 launch duration, measured with HIP events around every launch in a
                 second, instrumented run of the same K steps; peak 2.5 PFLOP/s bf16
  cpu_baseline   the numpy oracle (a port of the reference's arithmetic, float32) timed
                 on this box's host cores on a bounded sample of the same workload
  log_density    configs[2] (B=64 datasets, 512 context + 128 target rows): one
                 teacher-forced evaluation on the GPU vs the same on the host CPU

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]
       python bench.py --kernel-shapes   (instead: one decode layer-step at the shapes of
                                          configs[1], [3] and [4], timings on stderr)
       python bench.py --mix-ceiling     (instead: the instruction mix of one 32x32 score block from
                                          registers: what the SIMD's issue port allows)
       python bench.py --training-attention  (instead: forward and backward of the training row
                                          attention at the reference's training shapes)
       python bench.py --training-step   (instead: one optimiser step of the reference's training
                                          configuration; launches from autograd's worker thread —
                                          not for runs under rocprofv3 --pmc)
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16

CFG3 = dict(d_model=256, n_heads=8, n_layers=12, d_ff=256, num_features=10, buffer_size=256, num_components=5)
B3, NC3, NT3 = 1024, 16384, 256
B2, NC2, NT2 = 64, 512, 128


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_model(device, dtype):
    from ar_nanotabpfn_amd.model import ARTabPFN

    torch.manual_seed(0)
    return ARTabPFN(**CFG3).eval().to(device=device, dtype=dtype)


def gp_context(n, feats, seed, lengthscale=1.0, noise=0.05, n_rff=2048):
    """GP draw with an RBF kernel via random Fourier features (exact Cholesky at
    n=16384 would be a 2 GB float64 matrix); values do not affect throughput."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, feats, generator=g)
    w = torch.randn(feats, n_rff, generator=g) / lengthscale
    b = torch.rand(n_rff, generator=g) * 2 * math.pi
    a = torch.randn(n_rff, generator=g)
    y = math.sqrt(2.0 / n_rff) * torch.cos(x @ w + b) @ a + noise * torch.randn(n, generator=g)
    return x, y


def decode_inputs(device, dtype):
    x_ctx, y_ctx = gp_context(NC3, CFG3["num_features"], seed=3)
    g = torch.Generator().manual_seed(4)
    x_tgt = torch.randn(NT3, CFG3["num_features"], generator=g)
    x_context = x_ctx.to(device, dtype).unsqueeze(0).expand(B3, -1, -1)
    y_context = y_ctx.to(device, dtype).unsqueeze(0).expand(B3, -1)
    x_target = x_tgt.to(device, dtype).unsqueeze(0).expand(B3, -1, -1)
    return x_context, y_context, x_target


def run_decode(pred, x_context, y_context, x_target, steps, device, dtype):
    """Prefill (untimed) + `steps` decode steps; returns (prefill_ms, decode_ms)."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    pred.init_kv_cache(B3, NT3, device, dtype)
    torch.cuda.synchronize()
    ev[0].record()
    pred.prefill_context(x_context, y_context)
    ev[1].record()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[2].record()
    pred.decode_targets(x_target[:, :steps])
    ev[3].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return ev[0].elapsed_time(ev[1]), ev[2].elapsed_time(ev[3]), wall_ms


def host_info():
    """Cores, thread counts and CPU model of the host the CPU legs run on."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    blas = None
    try:
        from threadpoolctl import threadpool_info

        blas = max((int(d.get("num_threads", 0)) for d in threadpool_info()), default=None)
    except Exception:
        pass
    return {"cpu_model": model, "os_cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(),
            "blas_threads": blas}


CPU_DECODE_B = 256            # trajectories of the CPU sample (a quarter of the batch; a step is linear in B)
CPU_DECODE_NBUF = (1, 128, 255)


def cpu_decode_baseline(model, x_context, y_context, x_target, n_bufs=CPU_DECODE_NBUF, b_sample=CPU_DECODE_B):
    """The numpy oracle (float32) on the host: one full 12-layer decode step of `b_sample`
    trajectories at each buffer length in `n_bufs`, one warm-up and the median of three timed runs
    each; the context K/V are random tensors of the right shape (the prefill is not part of the
    timed GPU region either, and attention cost does not depend on values).  Returns seconds per
    step of the FULL batch (the sample's median scaled by B / b_sample) averaged over `n_bufs`."""
    from oracle import model_oracle as mo

    sd = {k: v.detach().float().cpu().numpy() for k, v in model.state_dict().items()}
    om = mo.OracleModel(sd, CFG3["n_heads"], compute=np.float32)
    op = mo.OraclePredictor(om, "shared")
    H, Dh, L = CFG3["n_heads"], CFG3["d_model"] // CFG3["n_heads"], CFG3["n_layers"]
    rng = np.random.default_rng(0)
    xt = x_target[:b_sample, :2].float().cpu().numpy()
    k_ctx = [rng.standard_normal((H, NC3, Dh), dtype=np.float32) * 0.5 for _ in range(L)]
    v_ctx = [rng.standard_normal((H, NC3, Dh), dtype=np.float32) * 0.5 for _ in range(L)]
    per_n = []
    for n in n_bufs:
        k_buf = [rng.standard_normal((b_sample, H, n - 1, Dh), dtype=np.float32) * 0.5 for _ in range(L)]
        v_buf = [rng.standard_normal((b_sample, H, n - 1, Dh), dtype=np.float32) * 0.5 for _ in range(L)]
        emb = np.concatenate(
            [om.embed_buffer(xt[:, 0:1], np.zeros((b_sample, 1), np.float32)) + om.ar_tokens[n % om.ar_tokens.shape[0]],
             om.embed_target(xt[:, 1:2])], axis=1)
        times = []
        for rep in range(4):  # the first run is the warm-up
            op.init_kv_cache(b_sample, NT3)
            op.context_len, op.k_ctx, op.v_ctx = NC3, k_ctx, v_ctx
            op.k_buf, op.v_buf, op.buffer_len = list(k_buf), list(v_buf), n - 1
            t0 = time.perf_counter()
            z = op.transformer_decode(emb, commit=1)
            om.head_parameterize(z[:, -1:])
            if rep:
                times.append(time.perf_counter() - t0)
        per_n.append(float(np.median(times)) * (B3 / b_sample))
        log(f"[cpu] decode step at n_buf={n}: median {np.median(times):.2f} s for {b_sample} trajectories "
            f"-> {per_n[-1]:.2f} s for {B3}")
    return float(np.mean(per_n)), per_n


def log_density_bench(device, dtype, model, with_cpu):
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    g = torch.Generator().manual_seed(2)
    F = CFG3["num_features"]
    x = torch.randn(B2, NC2 + NT2, F, generator=g)
    w1 = torch.randn(B2, F, 64, generator=g) / F**0.5
    w2 = torch.randn(B2, 64, 64, generator=g) / 8.0
    w3 = torch.randn(B2, 64, 1, generator=g) / 8.0
    y = (torch.tanh(torch.tanh(x @ w1) @ w2) @ w3).squeeze(-1) + 0.1 * torch.randn(B2, NC2 + NT2, generator=g)
    y = (y - y[:, :NC2].mean(1, keepdim=True)) / y[:, :NC2].std(1, keepdim=True)
    xd, yd = x.to(device, dtype), y.to(device, dtype)
    args = (xd[:, :NC2], yd[:, :NC2], xd[:, NC2:], yd[:, NC2:])
    pred = ARTabPFNPredictor.from_trained_model(model, backend="flex_attention")
    for _ in range(3):
        ll = pred.evaluate_joint_density(*args)
    torch.cuda.synchronize()
    ts = []
    for _ in range(10):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        ll = pred.evaluate_joint_density(*args)
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b))
    gpu_ms = float(np.median(ts))
    res = {"workload": "configs[2]: B=64 datasets x (512 context + 128 target rows), 12-layer d_model=256 bf16, "
                       "per-dataset contexts", "gpu_ms": round(gpu_ms, 3), "finite": bool(torch.isfinite(ll).all())}
    if with_cpu:
        from oracle import model_oracle as mo

        # host leg: the numpy oracle in float32 on a bounded sample (the first 16 of the 64
        # datasets; datasets are independent, so the evaluation is linear in their number), one
        # warm-up and the median of three timed runs, scaled to the 64 datasets
        sd = {k: v.detach().float().cpu().numpy() for k, v in model.state_dict().items()}
        om = mo.OracleModel(sd, CFG3["n_heads"], compute=np.float32)
        n_cpu = 16
        a32 = [t[:n_cpu].float().cpu().numpy() for t in args]
        times = []
        for rep in range(4):
            t0 = time.perf_counter()
            ll_cpu = mo.OraclePredictor(om, "per_dataset").evaluate_joint_density(*a32)
            if rep:
                times.append(time.perf_counter() - t0)
        cpu_s = float(np.median(times)) * (B2 / n_cpu)
        d = np.abs(ll[:n_cpu].float().cpu().numpy() - ll_cpu)
        res.update(cpu_s=round(cpu_s, 3), speedup=round(cpu_s * 1e3 / gpu_ms, 1),
                   cpu_sample=f"numpy float32 oracle on {n_cpu} of the {B2} datasets, 1 warm-up + median of 3, x{B2 // n_cpu}",
                   mean_abs_dlogp_vs_cpu_f32=float(d.mean()), max_abs_dlogp_vs_cpu_f32=float(d.max()))
        log(f"[cpu] configs[2] log-density: {cpu_s:.2f} s for {B2} datasets (from {n_cpu})  (GPU {gpu_ms:.2f} ms)")
    return res


# Measured with rocprofv3 (median over the decode launches): 10337.7 KiB x 2.0 fetched,
# 14336.0 KiB written (the partial outputs leave in 16-bit, their LSE in fp32; about 3 MB read and
# 6 MB written are the registers the kernel's prologue parks in scratch memory).
CONTEXT_PASS_HBM_BYTES = int(9339.5 * 1024 * 2.0 + 10240.0 * 1024)


def kernel_shapes(device):
    """One decode layer-step (context pass + buffer pass + merge + append) at the attention shapes
    of configs[1], configs[3] and configs[4]: HIP-event time per call over replays of a recorded graph
    of ten calls (the cross-queue dependencies of the two-stream schedule are part of it)."""
    from ar_nanotabpfn_amd import attention_kernels as ak

    dt = torch.bfloat16
    side = torch.cuda.Stream(device=device)
    out = []
    for name, B, H, Lq, Nc, Dh, cap, n_bufs, scale in (
        ("configs[1]", 256, 8, 1, 1024, 64, 64, (1, 16, 64), 0.125),
        ("configs[3]", 1024, 8, 2, 16384, 32, 256, (1, 128, 255), 0.6),
        ("configs[4]", 2048, 16, 2, 4096, 32, 256, (1, 128, 255), 0.6),
    ):
        g = torch.Generator(device=device).manual_seed(0)

        def draw(*shape):
            return (torch.randn(*shape, generator=g, device=device) * scale).to(dt)

        q, kc, vc = draw(B, H, Lq, Dh), draw(H, Nc, Dh), draw(H, Nc, Dh)
        kb, vb = draw(B, H, cap, Dh), draw(B, H, cap, Dh)
        kn, vn = (draw(B, H, 1, Dh), draw(B, H, 1, Dh)) if Lq == 2 else (None, None)
        for n in n_bufs:
            nn = min(n, cap - (1 if Lq == 2 else 0))
            for label, kw in (("sequential", {}), ("two streams", dict(side_stream=side))):
                def call():
                    return ak.decode_attention(q, kc, vc, kb, vb, nn, kn, vn, **kw)
                # ten calls recorded into one graph: the replay is free of host launch time
                warm = torch.cuda.Stream(device=device)
                warm.wait_stream(torch.cuda.current_stream(device))
                with torch.cuda.stream(warm):
                    for _ in range(3):
                        call()
                torch.cuda.current_stream(device).wait_stream(warm)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for _ in range(10):
                        call()
                graph.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                graph.replay()
                graph.replay()
                e1.record()
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) / 20 * 1e3
                flops = 4.0 * B * H * Lq * (Nc + nn + (Lq - 1)) * Dh
                byts = 2.0 * Dh * 2 * (H * Nc + B * H * (nn + (Lq - 1))) + 2.0 * 2 * B * H * Lq * Dh
                out.append(dict(config=name, n_buf=nn, schedule=label, us=round(us, 1),
                                tflops=round(flops / us / 1e6, 1), gbps=round(byts / us / 1e3, 1)))
                log(f"[shape] {name} n_buf={nn:3d} {label:11s} {us:8.1f} us  {flops / us / 1e6:7.1f} TFLOP/s  "
                    f"{byts / us / 1e3:7.1f} GB/s")
    print(json.dumps({"kernel_shapes": out}))


def mix_ceiling(device):
    """The instruction mix of one 32x32 score block of the head_dim-32 kernel, issued from registers
    with no memory traffic (``artab_bench_instruction_mix``): the rate the SIMD's issue port allows,
    for the software-pipelined pass (row sum on v_dot2c) and the lean pass (row sum on the matrix
    pipe), on constant and on random operands, with two and four wavefronts per SIMD."""
    import ctypes

    from ar_nanotabpfn_amd import _lib

    lib = _lib.load()
    iters = 20000
    names = {0: "pipelined pass: 4 mfma32 + 16 exp + 8 cvt + 8 dot2c", 1: "lean pass: 4 mfma32 + 2 mfma16 + 16 exp + 8 cvt",
             2: "matrix instructions of the lean pass alone", 3: "vector instructions of the lean pass alone"}
    rows = []
    for waves, lds in ((2, 64 * 1024), (4, 36 * 1024)):  # LDS per workgroup fixes how many share a CU
        wgs = 256 * waves
        out = torch.empty(wgs * 256, device=device, dtype=torch.float32)
        stamps = torch.zeros(wgs * 4 * 2, device=device, dtype=torch.int64)
        for rnd in (0, 1):
            for variant in (0, 1, 2, 3):
                def launch():
                    _lib.check(lib.artab_bench_instruction_mix(variant, rnd, wgs, iters, lds, ctypes.c_void_p(out.data_ptr()),
                                                               ctypes.c_void_p(stamps.data_ptr()), _lib.current_stream(device)))
                launch()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                launch()
                e1.record()
                torch.cuda.synchronize()
                ms = e0.elapsed_time(e1)
                st = stamps.view(-1, 2).double()
                ghz = float((st[:, 0] / st[:, 1]).mean()) * 0.1  # shader cycles per 10 ns tick
                ns_block = ms * 1e6 / (iters * waves)            # per SIMD and block
                tflops = 4 * 32768.0 * 1024 / ns_block / 1e3 if variant != 3 else None
                rows.append(dict(variant=names[variant], data="random" if rnd else "constant", waves_per_simd=waves,
                                 ns_per_block=round(ns_block, 1), cycles_per_block=round(ns_block * ghz, 1),
                                 clock_ghz=round(ghz, 2), tflops_equivalent=round(tflops, 1) if tflops else None,
                                 frac_of_peak=round(tflops / MFMA_BF16_PEAK_TFLOPS, 3) if tflops else None))
                log(f"[mix] {names[variant]:58s} {'random' if rnd else 'const ':6s} data, {waves} waves/SIMD: {ns_block:6.1f} ns/block "
                    f"= {ns_block * ghz:5.0f} cycles at {ghz:.2f} GHz" + (f", {tflops:6.0f} TFLOP/s-equivalent" if tflops else ""))
    print(json.dumps({"mix_ceiling": rows}))


def training_attention(device):
    """Forward (with log-sum-exp) and backward of the row attention of one training step at the
    shapes of the reference's training configuration (configs/train_tabular_online.yaml and the
    defaults of train.py:44-64: 4 heads of 32, 32 buffer rows, 512 target rows, context 64 or
    1024, batch 64 or 512), q/k/v as views of one projection output.  Algorithmic flops: 4 Dh per
    visible (query, key) pair forward, 10 Dh backward (the kernels recompute S and dP in both
    backward launches: 14 Dh executed)."""
    import ar_nanotabpfn_amd.attention_kernels as ak
    from ar_nanotabpfn_amd.attention import RowMask

    H, D, Nb, Nt = 4, 32, 32, 512
    rows = []

    def timed(fn, n=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    for B, Nc in ((64, 64), (64, 1024), (512, 64), (512, 1024)):
        R, A = Nc + Nb + Nt, Nt // (2 * Nb)
        g = torch.Generator().manual_seed(0)
        qkv = (torch.randn(B, R, 3, H, D, generator=g) * 0.7).to(device, torch.bfloat16)
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
        dout = (torch.randn(B, R, H, D, generator=g) * 0.7).to(device, torch.bfloat16).transpose(1, 2)
        pairs = int(RowMask(R, Nc, Nb, A).dense().sum()) * B * H
        out, lse = ak._row_mask_forward(q, k, v, Nc, Nb, A, True, True)
        us_f = timed(lambda: ak._row_mask_forward(q, k, v, Nc, Nb, A, True, True))
        us_b = timed(lambda: ak.row_mask_attention_backward(q, k, v, out, dout, lse, Nc, Nb, A))
        tensor_bytes = B * H * R * D * 2
        rows.append(dict(B=B, Nc=Nc, Nb=Nb, Nt=Nt, visible_pairs=pairs, forward_us=round(us_f, 1), backward_us=round(us_b, 1),
                         forward_tflops=round(4.0 * D * pairs / us_f * 1e-6, 1),
                         backward_tflops=round(10.0 * D * pairs / us_b * 1e-6, 1),
                         forward_gbs=round(4 * tensor_bytes / us_f * 1e-3, 1),
                         backward_gbs=round(8 * tensor_bytes / us_b * 1e-3, 1)))
        log(f"[training attention] B={B:3d} Nc={Nc:4d} R={R:4d}: forward {us_f:7.1f} us, backward {us_b:7.1f} us "
            f"({rows[-1]['forward_tflops']} / {rows[-1]['backward_tflops']} TFLOP/s algorithmic, "
            f"{rows[-1]['forward_gbs']} / {rows[-1]['backward_gbs']} GB/s of tensor bytes)")
    print(json.dumps({"training_attention": rows}))


def training_step(device):
    """One optimiser step of the reference's training configuration (configs/train_tabular_online.yaml:
    12 layers, d_model 128, 4 heads, d_ff 256, 20 mixture components; batch 64 of 64 context + 32
    buffer + 512 target rows; bf16 autocast, AdamW, gradient clipping at 1.0 as in train.py:289-310)
    with the row attention on the device kernels in both directions, and the same step with the row
    attention as PyTorch's scaled_dot_product_attention under the dense boolean mask."""
    import torch.nn.functional as F

    import ar_nanotabpfn_amd.attention_kernels as ak
    from ar_nanotabpfn_amd.attention import RowMask, create_dense_mask, create_row_mask
    from ar_nanotabpfn_amd.model import ARTabPFN

    cfg = dict(d_model=128, n_heads=4, n_layers=12, d_ff=256, num_features=2, buffer_size=32, num_components=20)
    B, Nc, Nb, Nt = 64, 64, 32, 512
    torch.manual_seed(0)
    model = ARTabPFN(**cfg).to(device)
    opt = torch.optim.AdamW(model.parameters(), lr=1e-3, betas=(0.9, 0.95), weight_decay=0.0)
    g = torch.Generator().manual_seed(1)
    mk = lambda *s: torch.randn(*s, generator=g).to(device)  # noqa: E731
    data = (mk(B, Nc, 2), mk(B, Nc), mk(B, Nb, 2), mk(B, Nb), mk(B, Nt, 2))
    y_t = mk(B, Nt)
    masks = (create_dense_mask(1, device=device), create_row_mask(Nc + Nb + Nt, Nc, Nb, device=device))

    def sdpa_row_attention(q, k, v, context_len, buffer_len, attending_chunks, use_triton=True):
        mask = RowMask(q.shape[2], context_len, buffer_len, attending_chunks).dense(q.device)
        return F.scaled_dot_product_attention(q, k, v, attn_mask=mask)

    def one_step():
        opt.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = model(*data, *masks, y_target=y_t)
        loss.backward()
        torch.nn.utils.clip_grad_norm_(model.parameters(), 1.0)
        opt.step()
        return loss

    def timed(n=10):
        for _ in range(3):
            one_step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            loss = one_step()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n, loss.item()

    ms_dev, loss_dev = timed()
    device_attention = ak.row_mask_attention
    ak.row_mask_attention = sdpa_row_attention
    try:
        ms_ref, loss_ref = timed()
    finally:
        ak.row_mask_attention = device_attention
    log(f"[training step] 12 layers, B={B}, rows {Nc}+{Nb}+{Nt}, bf16 autocast + AdamW: {ms_dev:.2f} ms per step with the "
        f"device row attention, {ms_ref:.2f} ms with scaled_dot_product_attention under the dense mask")
    print(json.dumps({"training_step": dict(
        config="train_tabular_online.yaml", B=B, Nc=Nc, Nb=Nb, Nt=Nt, ms_per_step=round(ms_dev, 3),
        ms_per_step_sdpa_dense_mask=round(ms_ref, 3), loss_after=round(loss_dev, 4), loss_after_sdpa=round(loss_ref, 4))}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=NT3)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline legs")
    ap.add_argument("--full-last-layer", action="store_true",
                    help="let the last layer of a decode step finish the buffer row too (its output is read by nobody)")
    ap.add_argument("--event-ordering", action="store_true",
                    help="order the two streams of the recorded step with events instead of device-side counters")
    ap.add_argument("--separate-step-boundary", action="store_true",
                    help="last layer's tail, step tail and first layer's head as three launches instead of one")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only copy a 256 MiB buffer five times (reference kernel for scaling HBM counters)")
    ap.add_argument("--mix-ceiling", action="store_true",
                    help="only run the instruction mix of one score block from registers (issue-port ceiling of the kernel)")
    ap.add_argument("--training-attention", action="store_true",
                    help="only time forward and backward of the training row attention at the reference's training shapes")
    ap.add_argument("--training-step", action="store_true",
                    help="only time one optimiser step of the reference's training configuration")
    ap.add_argument("--kernel-shapes", action="store_true",
                    help="only time one decode layer-step at the attention shapes of configs[1], [3], [4]")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: trajectories are independent given the context, so more GPUs "
                 "shard B with no per-step exchange; run with --gpus 1.")
    if not 1 <= args.steps <= NT3:
        sys.exit(f"--steps must be in [1, {NT3}] (one step per target of the configuration)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")

    if args.copy_calibration:
        a = torch.empty(128 * 1024 * 1024, dtype=torch.bfloat16, device="cuda:0").normal_()
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": a.numel() * 2, "copy_bytes_written": a.numel() * 2, "launches": 5}))
        return

    from ar_nanotabpfn_amd import _lib
    from ar_nanotabpfn_amd.inference import ARTabPFNPredictor

    lib = _lib.load()  # fails loudly when the extension is not built
    if args.kernel_shapes:
        kernel_shapes(torch.device("cuda:0"))
        return
    if args.mix_ceiling:
        mix_ceiling(torch.device("cuda:0"))
        return
    if args.training_attention:
        training_attention(torch.device("cuda:0"))
        return
    if args.training_step:
        training_step(torch.device("cuda:0"))
        return
    device, dtype = torch.device("cuda:0"), torch.bfloat16
    model = build_model(device, dtype)
    x_context, y_context, x_target = decode_inputs(device, dtype)
    pred = ARTabPFNPredictor.from_trained_model(model, backend="triton_shared_context")
    if args.event_ordering:
        pred.counter_ordering = False
    if args.full_last_layer:
        pred.target_only_last_layer = False
    if args.separate_step_boundary:
        pred.fuse_step_boundary = False

    torch.manual_seed(0)
    # Untimed warm-up: W decode steps (at least the three a recorded step needs).  The recorded
    # graph depends on the cache capacity, not on the number of steps, so the timed call below
    # only replays it; that is asserted.
    run_decode(pred, x_context, y_context, x_target, min(max(args.warmup, 3), NT3), device, dtype)
    recorded = pred.graph_recordings
    prefill_ms, decode_ms, wall_ms = run_decode(pred, x_context, y_context, x_target, args.steps, device, dtype)
    if args.steps >= 3 and pred.graph_recordings != recorded:
        sys.exit("bench.py: a HIP graph was recorded inside the timed region")
    ms_per_step = decode_ms / args.steps
    value = 1e3 / ms_per_step
    log(f"[gpu] prefill {prefill_ms:.2f} ms; {args.steps} decode steps in {decode_ms:.2f} ms "
        f"({ms_per_step:.3f} ms/step, host wall {wall_ms:.1f} ms)")

    # instrumented re-run of the same steps: HIP events around every context-pass launch
    import ctypes

    # (launched kernel by kernel from Python: events cannot be recorded into a replayed graph)
    pred.use_hip_graph = False
    lib.artab_profile_begin(CFG3["n_layers"] * (args.steps + 1) + 64)
    run_decode(pred, x_context, y_context, x_target, args.steps, device, dtype)
    tot, cnt = ctypes.c_double(0.0), ctypes.c_int(0)
    lib.artab_profile_end(ctypes.byref(tot), ctypes.byref(cnt))
    # the same launches with the buffer pass after the context pass instead of beside it: the
    # context-pass kernel with the chip to itself
    pred.overlap_buffer_pass = False
    lib.artab_profile_begin(CFG3["n_layers"] * (args.steps + 1) + 64)
    run_decode(pred, x_context, y_context, x_target, args.steps, device, dtype)
    tot_alone, cnt_alone = ctypes.c_double(0.0), ctypes.c_int(0)
    lib.artab_profile_end(ctypes.byref(tot_alone), ctypes.byref(cnt_alone))
    pred.overlap_buffer_pass = True
    pred.use_hip_graph = True
    # the first L launches are the prefill's dense passes, the first decode step has Lq=1
    H, Dh, L = CFG3["n_heads"], CFG3["d_model"] // CFG3["n_heads"], CFG3["n_layers"]
    n_dec = cnt.value - L
    # per-launch algorithmic flops: 4*B*H*Lq*Nc*Dh with Lq=1 for step 0 and 2 afterwards
    flops_total = 4.0 * B3 * H * NC3 * Dh * L * (1 + 2 * (args.steps - 1))
    # time of the decode launches = total - prefill launches; measure prefill launches separately
    lib.artab_profile_begin(L + 8)
    pred.init_kv_cache(B3, NT3, device, dtype)
    pred.prefill_context(x_context, y_context)
    ptot, pcnt = ctypes.c_double(0.0), ctypes.c_int(0)
    lib.artab_profile_end(ctypes.byref(ptot), ctypes.byref(pcnt))
    dec_kernel_ms = tot.value - ptot.value
    alone_ms = tot_alone.value - ptot.value
    avg_launch_us = dec_kernel_ms * 1e3 / max(n_dec, 1)
    achieved = flops_total / (dec_kernel_ms * 1e-3) / 1e12 if dec_kernel_ms > 0 else 0.0
    prefill_flops = 4.0 * H * NC3 * NC3 * Dh * L
    roofline = {
        "kernel": "flash_kernel<bf16,32> context pass of artab_decode_attention",
        "bound": "mfma",
        "achieved": round(achieved, 2),
        "peak": MFMA_BF16_PEAK_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
        # HBM bytes of one decode-shaped launch: FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 from two
        # rocprofv3 --pmc runs of this script, the factors from the same counters on a 256 MiB copy
        # (--copy-calibration); algorithmic: K/V 16.8 MB + Q 1.0 MB read, 8.9 MB of partials written.
        "traffic": CONTEXT_PASS_HBM_BYTES,
        "launches": n_dec,
        "avg_launch_us": round(avg_launch_us, 2),
        # In the timed schedule the buffer pass of the same layer runs beside this kernel and takes
        # issue slots from it; these two are the kernel without that neighbour.
        "avg_launch_us_alone": round(alone_ms * 1e3 / max(n_dec, 1), 2),
        "frac_alone": round(flops_total / (alone_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4) if alone_ms > 0 else None,
        "flops_per_launch_lq2": 4.0 * B3 * H * 2 * NC3 * Dh,
        "prefill_tflops": round(prefill_flops / (ptot.value * 1e-3) / 1e12, 2) if ptot.value > 0 else None,
    }
    log(f"[gpu] context-pass kernel: {n_dec} launches, avg {avg_launch_us:.1f} us, {achieved:.1f} TFLOP/s")

    out = {
        "metric": "ar_decode_target_steps_per_sec",
        "value": round(value, 2),
        "unit": "target-steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "configs[3] long-context AR sampling: shared context N_ctx=16384 (x in R^10, GP prior via "
                        "random Fourier features), B=1024 trajectories, 12-layer d_model=256 8-head bf16 model, "
                        "decode steps 0..K-1 with the in-place buffer K/V (N_buf = step-1) and LSE merge",
            "B": B3, "N_ctx": NC3, "N_targets": NT3, "layers": L, "heads": H, "head_dim": Dh,
        },
        "trajectory_steps_per_sec": round(value * B3, 1),
        # the last layer of a recorded step finishes the target row only (the buffer row's output of
        # that layer is read by nobody; --full-last-layer computes it as the reference does: -0.7 %)
        "target_only_last_layer": bool(pred.target_only_last_layer),
        # last layer's tail + head/draw/embedding + first layer's head of the next step as one launch
        "step_boundary_fused": bool(pred._graph_state is not None
                                    and getattr(pred._graph_state.chains[0], "boundary", None) is not None),
        "stream_ordering": ("counters" if getattr(pred._graph_state.chains[0], "order", None) is not None else "events")
        if pred._graph_state is not None else None,
        "prefill_ms": round(prefill_ms, 3),
        "roofline": roofline,
    }

    if not args.no_cpu:
        cpu_s, per_n = cpu_decode_baseline(model, x_context, y_context, x_target)
        host = host_info()
        out["cpu_baseline"] = {
            "value": round(1.0 / cpu_s, 4),
            "unit": "target-steps/s",
            "cores": host["blas_threads"] or host["torch_threads"],
            "kind": "port",
            "dtype": "f32",
            "sample": f"numpy float32 oracle (a port of the reference's arithmetic), one full 12-layer decode step "
                      f"(N_ctx=16384) of {CPU_DECODE_B} of the {B3} trajectories at each of N_buf={list(CPU_DECODE_NBUF)}: "
                      f"1 warm-up + median of 3, scaled x{B3 // CPU_DECODE_B} to the batch, mean over N_buf; "
                      f"context K/V random (the prefill is outside the timed GPU region as well)",
            "seconds_per_step_by_n_buf": [round(t, 3) for t in per_n],
            "host": host,
        }
    else:
        out["cpu_baseline"] = None
    out["log_density"] = log_density_bench(device, dtype, model, with_cpu=not args.no_cpu)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
