"""float32 PyTorch restatement of the attention entry points (TEST INFRASTRUCTURE ONLY — never
imported by the shipped package).

Same call signatures as ``ar_nanotabpfn_amd.attention_kernels``; every function
up-casts to float32, evaluates one masked softmax over the concatenated key set
(triton_kernels.py:204-240 is the reference's own statement of that equivalence) and
returns the input dtype.  It lets an end-to-end test, and the log-density leg of
bench.py, run the same PyTorch-ROCm model twice on the same device, changing nothing
but the attention implementation: what is left between the two runs is the attention
kernels' own error, and what both miss the float64 oracle by is the model's 16-bit
rounding.  It is itself checked against the numpy oracle in tests/test_predictor_gpu.py.
"""

import torch


def _sdpa(q, k, v, mask=None):
    qf, kf, vf = q.float(), k.float(), v.float()
    s = torch.matmul(qf, kf.transpose(-1, -2)) * q.shape[-1] ** -0.5
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf"))
    return torch.matmul(torch.softmax(s, dim=-1), vf).to(q.dtype)


def _ctx(k, B):
    return k.unsqueeze(0).expand(B, -1, -1, -1) if k.dim() == 3 else k


def prefill_attention(q, k, v, k_cache=None, v_cache=None, use_triton=True):
    if k_cache is not None:
        Nc = k.shape[2]
        if k_cache.dim() == 3:
            k_cache[:, :Nc] = k[0]
            v_cache[:, :Nc] = v[0]
        else:
            k_cache[:, :, :Nc] = k
            v_cache[:, :, :Nc] = v
    return _sdpa(q, k, v)


def decode_attention(q, k_ctx, v_ctx, k_buf_cache, v_buf_cache, n_buf, k_new=None, v_new=None, use_triton=True):
    B = q.shape[0]
    ks, vs = [_ctx(k_ctx, B)], [_ctx(v_ctx, B)]
    if n_buf:
        ks.append(k_buf_cache[:, :, :n_buf])
        vs.append(v_buf_cache[:, :, :n_buf])
    if k_new is not None:
        ks.append(k_new)
        vs.append(v_new)
        k_buf_cache[:, :, n_buf : n_buf + 1] = k_new
        v_buf_cache[:, :, n_buf : n_buf + 1] = v_new
    return _sdpa(q, torch.cat(ks, dim=2), torch.cat(vs, dim=2))


def teacher_forcing_attention(q, k_ctx, v_ctx, k_buf, v_buf, num_targets, use_triton=True, return_lse=False):
    B, Nt = q.shape[0], num_targets
    kc, vc = _ctx(k_ctx, B), _ctx(v_ctx, B)
    Nc = kc.shape[2]
    qi = torch.arange(2 * Nt, device=q.device)[:, None]
    kj = torch.arange(Nt, device=q.device)[None, :]
    buf = torch.where(qi < Nt, kj <= qi, kj < qi - Nt)
    mask = torch.cat([torch.ones(2 * Nt, Nc, dtype=torch.bool, device=q.device), buf], dim=1)[None, None]
    return _sdpa(q, torch.cat([kc, k_buf], dim=2), torch.cat([vc, v_buf], dim=2), mask)


def hybrid_teacher_forcing_attention(q, k_ctx, v_ctx, k_buf, v_buf, num_targets, use_triton=True):
    return teacher_forcing_attention(q, k_ctx, v_ctx, k_buf, v_buf, num_targets)
