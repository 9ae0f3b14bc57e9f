"""Pure-PyTorch gather oracle for the CLUSTEN ops.  TEST INFRASTRUCTURE ONLY (see __init__.py).

The three `*_gather` functions restate, line for line in meaning, the "pytorch equivalent"
expressions that the reference's own kernel test scripts compare its CUDA kernels against:

    QK  clusten/test_qk_kernel.py:39-40
    AV  clusten/test_av_kernel.py:39-40
    WF  clusten/test_wf_kernel.py:40-41

They are built from library routines only (`gather`, broadcast multiply, `sum`, `matmul`), run on
any device and dtype, and are differentiable, so the backward oracle is PyTorch autograd through
them (`*_gather_backward`).  The `*_loops` functions are an independent second statement of the same
sums as explicit nested loops in float64 numpy, for tiny shapes; `clusten_ref.c` is a third, in C.

Parity status: every function here is pinned by tests/test_oracle.py — against the nested-loop and
C restatements, against dense `matmul` (lists that enumerate all tokens), against plain `gather`
(one-hot weights, integer-valued data, bit exact), by permutation/linearity/duplicate invariants,
and (backward) by `torch.autograd.gradcheck` in float64, an `index_add_` formulation and a
conservation law.  The reference holds no golden vectors for these ops (its scripts print norms of
random data), so there are none to check against.
"""
from __future__ import annotations

import numpy as np
import torch


# --------------------------------------------------------------------------------------------
# forward: the reference's gather expressions
# --------------------------------------------------------------------------------------------

def qk_gather(query: torch.Tensor, key: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """attn[b,h,i,j] = sum_c query[b,h,i,c] * key[b,h,nbhd_idx[b,i,j],c]   (test_qk_kernel.py:39-40)

    query, key: (b,h,n,c); nbhd_idx: (b,n,m) int64; returns (b,h,n,m).
    """
    b, h, n, c = query.shape
    m = nbhd_idx.shape[-1]
    key_gather = key.gather(index=nbhd_idx.reshape(b, 1, -1, 1).expand(-1, h, -1, c), dim=2).reshape(b, h, n, m, c)
    return (query.unsqueeze(3) * key_gather).sum(-1)


def av_gather(attn: torch.Tensor, v: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """feat[b,h,i,c] = sum_j attn[b,h,i,j] * v[b,h,nbhd_idx[b,i,j],c]   (test_av_kernel.py:39-40)

    attn: (b,h,n,m); v: (b,h,n,c); nbhd_idx: (b,n,m) int64; returns (b,h,n,c).
    """
    b, h, n, m = attn.shape
    c = v.shape[-1]
    v_gather = v.gather(index=nbhd_idx.reshape(b, 1, -1, 1).expand(-1, h, -1, c), dim=2).reshape(b, h, n, m, c)
    return (attn.unsqueeze(4) * v_gather).sum(3)


def wf_gather(weights: torch.Tensor, feat: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """feat_new[b,i,ic,c] = sum_j weights[b,i,j,ic] * feat[b,nbhd_idx[b,i,j],c]   (test_wf_kernel.py:40-41)

    weights: (b,n_,m,ic); feat: (b,n,c); nbhd_idx: (b,n_,m) int64; returns (b,n_,ic,c).
    """
    b, n_, m, _ = weights.shape
    c = feat.shape[-1]
    feat_gather = feat.gather(index=nbhd_idx.reshape(b, -1, 1).expand(-1, -1, c), dim=1).reshape(b, n_, m, c)
    return weights.transpose(-1, -2) @ feat_gather


def _chunked(fn, batch_chunk, *tensors):
    """Apply `fn` to slices of the batch axis so the (b,h,n,m,c) intermediate stays small."""
    b = tensors[0].shape[0]
    if not batch_chunk or batch_chunk >= b:
        return fn(*tensors)
    outs = [fn(*(t[s:s + batch_chunk] for t in tensors)) for s in range(0, b, batch_chunk)]
    return torch.cat(outs, dim=0)


def qk_gather_chunked(query, key, nbhd_idx, batch_chunk=4):
    return _chunked(qk_gather, batch_chunk, query, key, nbhd_idx)


def av_gather_chunked(attn, v, nbhd_idx, batch_chunk=4):
    return _chunked(av_gather, batch_chunk, attn, v, nbhd_idx)


def wf_gather_chunked(weights, feat, nbhd_idx, batch_chunk=4):
    return _chunked(wf_gather, batch_chunk, weights, feat, nbhd_idx)


# --------------------------------------------------------------------------------------------
# backward: autograd through the gather expressions, with an explicit upstream gradient
# (the reference scripts use `.mean().backward()`, whose constant upstream gradient cannot see a
#  mis-indexed gradient; the tests use random ones)
# --------------------------------------------------------------------------------------------

def _backward(fn, grad_out, a, b, nbhd_idx):
    a = a.detach().clone().requires_grad_(True)
    b = b.detach().clone().requires_grad_(True)
    out = fn(a, b, nbhd_idx)
    ga, gb = torch.autograd.grad(out, (a, b), grad_out)
    return ga, gb


def qk_gather_backward(d_attn, query, key, nbhd_idx):
    """(d_query, d_key) of clusten/clusten.py:35-40."""
    return _backward(qk_gather, d_attn, query, key, nbhd_idx)


def av_gather_backward(d_feat, attn, v, nbhd_idx):
    """(d_attn, d_v) of clusten/clusten.py:61-66."""
    return _backward(av_gather, d_feat, attn, v, nbhd_idx)


def wf_gather_backward(d_feat_new, weights, feat, nbhd_idx):
    """(d_weights, d_feat) of clusten/clusten.py:87-92."""
    return _backward(wf_gather, d_feat_new, weights, feat, nbhd_idx)


# --------------------------------------------------------------------------------------------
# second statement: nested loops in float64 numpy (tiny shapes only)
# follows the index expressions of the reference kernels:
#   clustenqk_cuda_kernel.cu:36-45,112-129  clustenav_cuda_kernel.cu:36-46,110-123,146-156
#   clustenwf_cuda_kernel.cu:36-50,116-131,156-165
# --------------------------------------------------------------------------------------------

def _np64(t):
    return t.detach().cpu().to(torch.float64).numpy()


def qk_loops(query, key, nbhd_idx):
    q, k, idx = _np64(query), _np64(key), nbhd_idx.cpu().numpy()
    b, h, n, c = q.shape
    m = idx.shape[-1]
    out = np.zeros((b, h, n, m))
    for bi in range(b):
        for hi in range(h):
            for i in range(n):
                for j in range(m):
                    nb = idx[bi, i, j]
                    s = 0.0
                    for ci in range(c):
                        s += q[bi, hi, i, ci] * k[bi, hi, nb, ci]
                    out[bi, hi, i, j] = s
    return out


def av_loops(attn, v, nbhd_idx):
    a, vv, idx = _np64(attn), _np64(v), nbhd_idx.cpu().numpy()
    b, h, n, m = a.shape
    c = vv.shape[-1]
    out = np.zeros((b, h, n, c))
    for bi in range(b):
        for hi in range(h):
            for i in range(n):
                for ci in range(c):
                    s = 0.0
                    for j in range(m):
                        s += a[bi, hi, i, j] * vv[bi, hi, idx[bi, i, j], ci]
                    out[bi, hi, i, ci] = s
    return out


def wf_loops(weights, feat, nbhd_idx):
    w, f, idx = _np64(weights), _np64(feat), nbhd_idx.cpu().numpy()
    b, n_, m, ic = w.shape
    c = f.shape[-1]
    out = np.zeros((b, n_, ic, c))
    for bi in range(b):
        for i in range(n_):
            for ici in range(ic):
                for ci in range(c):
                    s = 0.0
                    for j in range(m):
                        s += w[bi, i, j, ici] * f[bi, idx[bi, i, j], ci]
                    out[bi, i, ici, ci] = s
    return out


def qk_backward_loops(d_attn, query, key, nbhd_idx):
    g, q, k, idx = _np64(d_attn), _np64(query), _np64(key), nbhd_idx.cpu().numpy()
    b, h, n, c = q.shape
    m = idx.shape[-1]
    dq, dk = np.zeros_like(q), np.zeros_like(k)
    for bi in range(b):
        for hi in range(h):
            for i in range(n):
                for j in range(m):
                    nb = idx[bi, i, j]
                    for ci in range(c):
                        dq[bi, hi, i, ci] += k[bi, hi, nb, ci] * g[bi, hi, i, j]
                        dk[bi, hi, nb, ci] += q[bi, hi, i, ci] * g[bi, hi, i, j]
    return dq, dk


def av_backward_loops(d_feat, attn, v, nbhd_idx):
    g, a, vv, idx = _np64(d_feat), _np64(attn), _np64(v), nbhd_idx.cpu().numpy()
    b, h, n, m = a.shape
    c = vv.shape[-1]
    da, dv = np.zeros_like(a), np.zeros_like(vv)
    for bi in range(b):
        for hi in range(h):
            for i in range(n):
                for j in range(m):
                    nb = idx[bi, i, j]
                    for ci in range(c):
                        da[bi, hi, i, j] += vv[bi, hi, nb, ci] * g[bi, hi, i, ci]
                        dv[bi, hi, nb, ci] += a[bi, hi, i, j] * g[bi, hi, i, ci]
    return da, dv


def wf_backward_loops(d_feat_new, weights, feat, nbhd_idx):
    g, w, f, idx = _np64(d_feat_new), _np64(weights), _np64(feat), nbhd_idx.cpu().numpy()
    b, n_, m, ic = w.shape
    c = f.shape[-1]
    dw, df = np.zeros_like(w), np.zeros_like(f)
    for bi in range(b):
        for i in range(n_):
            for j in range(m):
                nb = idx[bi, i, j]
                for ici in range(ic):
                    for ci in range(c):
                        dw[bi, i, j, ici] += f[bi, nb, ci] * g[bi, i, ici, ci]
                        df[bi, nb, ci] += g[bi, i, ici, ci] * w[bi, i, j, ici]
    return dw, df


# --------------------------------------------------------------------------------------------
# comparison metric used by every parity test
# --------------------------------------------------------------------------------------------

def rel_err(x: torch.Tensor, ref: torch.Tensor) -> float:
    """max|x - ref| / max|ref| in float64 (0 when both are all-zero)."""
    x64 = x.detach().to(torch.float64).cpu()
    r64 = ref.detach().to(torch.float64).cpu()
    denom = r64.abs().max().item()
    num = (x64 - r64).abs().max().item()
    if denom == 0.0:
        return num
    return num / denom
