"""Randomised GPU parity of the three operators, forward and backward through the autograd Functions, against the
CPU gather oracle: a few hundred seeded cases drawn over batch size, head count, sequence length, head dim, list
length, storage type and the kinds of neighbour list the kernels tell apart (cluster-shared, the model's own,
arbitrary, runs of eight with their irregularities).  Tolerances as in the other GPU tests: forward 1e-5 (fp32),
1e-2 (fp16 / bf16), 1e-12 (fp64); gradients 1e-4 (fp32, atomics in any order), 2e-2 (16-bit), 1e-11 (fp64).
"""
import random

import pytest
import torch

import workloads as wl
from clusten import CLUSTENAVFunction, CLUSTENQKFunction, CLUSTENWFFunction
from conftest import TOL, TOL_SCATTER_F32
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu

GRAD_TOL = {torch.float32: TOL_SCATTER_F32, torch.float16: 2e-2, torch.bfloat16: 2e-2, torch.float64: 1e-11}
DTYPES = [torch.float32, torch.float32, torch.float16, torch.bfloat16, torch.float64]
LISTS = ["windowed", "model", "random", "runs:clusters", "runs:unaligned", "runs:padded", "runs:scattered",
         "runs:repeated"]


def _ref(t):
    return t.double() if t.dtype == torch.float64 else t.float()


def _close(what, case, x, ref, tol):
    err = oracle.rel_err(x, ref)
    assert err <= tol, "%s of %s: rel err %.3g > %.3g" % (what, case, err, tol)


def _attn_case(rng, n, device):
    dtype = rng.choice(DTYPES)
    B, H = rng.choice([1, 2, 3, 5]), rng.choice([1, 2, 3, 4, 5, 8, 16])
    C = rng.choice([16, 32, 32, 64, 8, 24])
    kind = rng.choice(LISTS)
    if kind == "model":
        M, N = 48, rng.choice([64, 144, 256, 400, 784])
    else:
        M, N = rng.choice([48, 48, 16, 32, 64, 8, 24, 40]), rng.choice([49, 56, 64, 100, 196, 197, 333, 784])
        if kind.startswith("runs:"):
            M = M if M % 8 == 0 else 48
            N = max(N, M)
        if kind == "windowed":
            M = min(M, N - 1)
    name = "attn case %d %s B%d H%d N%d C%d M%d %s" % (n, dtype, B, H, N, C, M, kind)
    case = wl.attn_case("random", 5000 + n, B, H, N, C, M=M, dtype=dtype, lists=kind)
    q, k, v, idx = case.query, case.key, case.value, case.nbhd_idx
    qd, kd, vd = (t.to(device).requires_grad_(True) for t in (q, k, v))
    attn = CLUSTENQKFunction.apply(qd, kd, idx.to(device))
    attn_ref = oracle.qk_gather_chunked(_ref(q), _ref(k), idx)
    _close("QK", name, attn.detach(), attn_ref, TOL[dtype])
    g = torch.randn(attn_ref.shape, generator=wl.generator(n)).to(dtype)
    dq, dk = torch.autograd.grad(attn, (qd, kd), g.to(device))
    rq, rk = oracle.qk_gather_backward(_ref(g), _ref(q), _ref(k), idx)
    _close("d_query", name, dq, rq, GRAD_TOL[dtype])
    _close("d_key", name, dk, rk, GRAD_TOL[dtype])
    p = torch.softmax(attn_ref, -1).to(dtype)
    pd = p.to(device).requires_grad_(True)
    feat = CLUSTENAVFunction.apply(pd, vd, idx.to(device))
    feat_ref = oracle.av_gather_chunked(_ref(p), _ref(v), idx)
    _close("AV", name, feat.detach(), feat_ref, TOL[dtype])
    g = torch.randn(feat_ref.shape, generator=wl.generator(n + 1)).to(dtype)
    dp, dv = torch.autograd.grad(feat, (pd, vd), g.to(device))
    rp, rv = oracle.av_gather_backward(_ref(g), _ref(p), _ref(v), idx)
    _close("d_attn", name, dp, rp, GRAD_TOL[dtype])
    _close("d_value", name, dv, rv, GRAD_TOL[dtype])


def _wf_case(rng, n, device):
    dtype = rng.choice(DTYPES)
    B, C, IC = rng.choice([1, 2, 4]), rng.choice([32, 64, 96, 128, 256, 512, 48]), rng.choice([4, 4, 1, 2, 3])
    M = rng.choice([48, 48, 16, 20, 64, 144])
    N = max(rng.choice([196, 200, 784, 1000]), M + 1)
    Nout = rng.choice([N // 4, N // 4 + 1, 7, 1])
    name = "wf case %d %s B%d N%d->%d C%d IC%d M%d" % (n, dtype, B, N, Nout, C, IC, M)
    case = wl.wf_case("random", 7000 + n, B, N, C, IC=IC, M=M, dtype=dtype, Nout=Nout)
    w, f, idx = case.weights, case.feat, case.nbhd_idx
    wd, fd = (t.to(device).requires_grad_(True) for t in (w, f))
    out = CLUSTENWFFunction.apply(wd, fd, idx.to(device))
    out_ref = oracle.wf_gather_chunked(_ref(w), _ref(f), idx)
    _close("WF", name, out.detach(), out_ref, TOL[dtype])
    g = torch.randn(out_ref.shape, generator=wl.generator(n + 2)).to(dtype)
    dw, df = torch.autograd.grad(out, (wd, fd), g.to(device))
    rw, rf = oracle.wf_gather_backward(_ref(g), _ref(w), _ref(f), idx)
    _close("d_weights", name, dw, rw, GRAD_TOL[dtype])
    _close("d_feat", name, df, rf, GRAD_TOL[dtype])


@pytest.mark.parametrize("seed", [11, 12])
def test_random_attention_cases(device, seed):
    rng = random.Random(seed)
    for n in range(120):
        _attn_case(rng, 1000 * seed + n, device)


@pytest.mark.parametrize("seed", [21])
def test_random_wf_cases(device, seed):
    rng = random.Random(seed)
    for n in range(80):
        _wf_case(rng, 1000 * seed + n, device)
