"""The entry point that allocates nothing (``artab_decode_attention_static``) against the entry
point it is a variant of (``artab_decode_attention`` with a caller-owned workspace): same kernels,
so the outputs and the appended cache rows must agree bit for bit.  Two calls in a row on one
device, the second with a smaller problem (the built-in scratch still holds the first call's
partials), then the oracle as the arbiter of the smaller one.  Both entry points are reached
through the C ABI (ctypes), as a foreign caller would."""

import ctypes

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from tests.helpers import TOL_OUT_16, max_abs, randn, to_np

pytestmark = pytest.mark.gpu


def _call(lib, L, name, q, kc, vc, kb, vb, kn, vn, n_buf, workspace=None):
    B, H, Lq, Dh = q.shape
    Nc = kc.shape[1]
    out = torch.empty((B, Lq, H, Dh), device=q.device, dtype=q.dtype).transpose(1, 2)
    views = [L.view4(q), L.view4(kc, shared_batch=True), L.view4(vc, shared_batch=True), L.view4(kb), L.view4(vb),
             L.view4(kn), L.view4(vn), L.view4(out)]
    head = [L.ref(v) for v in views] + [B, H, Lq, Nc, n_buf, None, kb.shape[2], Dh, 0.0, L.dtype_code(q.dtype)]
    stream = L.current_stream(q.device)
    if name == "artab_decode_attention_static":
        rc = lib.artab_decode_attention_static(*head, L.IMPL_MFMA, stream)
    else:
        rc = lib.artab_decode_attention(*head, ctypes.c_void_p(workspace.data_ptr()), workspace.numel() * 4,
                                        L.IMPL_MFMA, stream)
    L.check(rc)
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_static_scratch_decode_equals_workspace_decode_twice(device, dtype):
    from ar_nanotabpfn_amd import _lib as L

    lib = L.load()
    H, Dh, cap = 8, 32, 16
    # The second call is the smaller problem; both are outside the one-launch route for small decode
    # calls (a context above 2048*64 elements per head), so both cut the context into slices and
    # the second finds the first call's partials in the built-in scratch.
    for call, (B, Nc, n_buf) in enumerate(((96, 4200, 5), (40, 4200, 2))):
        q = randn((B, H, 2, Dh), 10 + call, dtype, 0.5).to(device)
        kc, vc = randn((H, Nc, Dh), 20 + call, dtype, 0.5).to(device), randn((H, Nc, Dh), 30 + call, dtype, 0.5).to(device)
        kb, vb = randn((B, H, cap, Dh), 40 + call, dtype, 0.5).to(device), randn((B, H, cap, Dh), 50 + call, dtype, 0.5).to(device)
        kn, vn = randn((B, H, 1, Dh), 60 + call, dtype, 0.5).to(device), randn((B, H, 1, Dh), 70 + call, dtype, 0.5).to(device)
        need = lib.artab_workspace_bytes(B, H, 2, Nc, Dh, L.dtype_code(dtype))
        assert 0 < need <= L.STATIC_SCRATCH_BYTES  # a split context: the scratch is really used
        ws = torch.empty((need + 3) // 4, device=device, dtype=torch.float32)
        kb_a, vb_a, kb_b, vb_b = kb.clone(), vb.clone(), kb.clone(), vb.clone()
        out_ws = _call(lib, L, "artab_decode_attention", q, kc, vc, kb_a, vb_a, kn, vn, n_buf, ws)
        out_st = _call(lib, L, "artab_decode_attention_static", q, kc, vc, kb_b, vb_b, kn, vn, n_buf)
        torch.cuda.synchronize()
        assert torch.equal(out_st, out_ws), f"call {call}: outputs differ"
        assert torch.equal(kb_a, kb_b) and torch.equal(vb_a, vb_b)
        assert torch.equal(kb_b[:, :, n_buf], kn[:, :, 0]) and torch.equal(vb_b[:, :, n_buf], vn[:, :, 0])
        ref, _, _ = ao.decode_step_attention(to_np(q), to_np(kc), to_np(vc), to_np(kb[:, :, :n_buf]),
                                             to_np(vb[:, :, :n_buf]), to_np(kn), to_np(vn))
        assert max_abs(to_np(out_st), ref) <= TOL_OUT_16


def test_static_scratch_decode_rejects_what_does_not_fit(device):
    from ar_nanotabpfn_amd import _lib as L

    lib = L.load()
    B, H, Nc, Dh = 8192, 16, 65536, 32
    assert lib.artab_workspace_bytes(B, H, 2, Nc, Dh, L.ARTAB_BF16) > L.STATIC_SCRATCH_BYTES
    v = L.ArtabView(0, 0, 0, 0)
    rc = lib.artab_decode_attention_static(*([ctypes.byref(v)] * 8), B, H, 2, Nc, 0, None, 4, Dh, 0.0, L.ARTAB_BF16,
                                           L.IMPL_AUTO, None)
    assert rc == L.ARTAB_ERR_WORKSPACE and b"built-in" in lib.artab_last_error()
