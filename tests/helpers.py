"""Shared test helpers: seeded inputs that are bit-identical on every box, and
conversions between torch tensors and the numpy oracle."""

import numpy as np
import torch

# Tolerances of the build's target: max-abs on 16-bit outputs, float32 LSE.
TOL_OUT_16 = 2e-2
TOL_LSE = 1e-3
# The reference's own float32 kernel-vs-PyTorch tolerance (tests/test_triton_kernel.py:51-66).
TOL_F32 = 1e-5


def randn(shape, seed, dtype=torch.bfloat16, scale=1.0):
    """CPU-generated normal tensor (fixed generator) cast to ``dtype``."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def to_np(t):
    """Exact float64 copy of a tensor's values."""
    return t.detach().to("cpu", torch.float32).numpy().astype(np.float64)


def max_abs(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    both_inf = np.isinf(a) & np.isinf(b) & (np.sign(a) == np.sign(b))
    d = np.abs(np.where(both_inf, 0.0, a - b))
    return float(np.max(d)) if d.size else 0.0


def out_tol(dtype):
    return TOL_F32 if dtype == torch.float32 else TOL_OUT_16


def lse_tol(dtype):
    return TOL_F32 if dtype == torch.float32 else TOL_LSE
