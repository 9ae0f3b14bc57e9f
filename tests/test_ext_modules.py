"""The stand-ins for the reference's three compiled extension modules (`clusten_ext`): called the way the reference's
wrapper calls them — forward with the transposed key copy of clusten/clusten.py:30, backward with the saved
un-transposed tensors of clusten/clusten.py:32,37-38 — and compared with the gather oracle."""
import pytest
import torch

import workloads as wl
from clusten_ext import clustenav_cuda, clustenqk_cuda, clustenwf_cuda
from conftest import TOL, TOL_SCATTER_F32
from oracle import clusten_oracle as oracle


def test_cpu_tensors_are_refused_like_check_cuda():
    q = torch.zeros(1, 1, 8, 16)
    idx = torch.zeros(1, 8, 4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        clustenqk_cuda.forward(q, q.permute(0, 1, 3, 2).contiguous(), idx)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        clustenav_cuda.forward(torch.zeros(1, 1, 8, 4), q, idx)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        clustenwf_cuda.forward(torch.zeros(1, 2, 4, 4), torch.zeros(1, 8, 16), torch.zeros(1, 2, 4, dtype=torch.int64))


def _ref(t):
    return t.float()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("lists", ["windowed", "model", "random"])
def test_qk_and_av_modules(device, dtype, lists):
    case = wl.attn_case("ext", 321, 2, 3, 256, 32, dtype=dtype, lists=lists)
    q, k, v, idx = case.query, case.key, case.value, case.nbhd_idx
    qd, kd, vd, idxd = q.to(device), k.to(device), v.to(device), idx.to(device)
    grad_tol = TOL_SCATTER_F32 if dtype == torch.float32 else 2e-2

    attn = clustenqk_cuda.forward(qd, kd.permute(0, 1, 3, 2).contiguous(), idxd)
    attn_ref = oracle.qk_gather_chunked(_ref(q), _ref(k), idx)
    assert attn.dtype == dtype and oracle.rel_err(attn, attn_ref) <= TOL[dtype]
    g = torch.randn(attn_ref.shape, generator=wl.generator(5)).to(dtype)
    d_q, d_k = clustenqk_cuda.backward(g.to(device), qd, kd, idxd)
    r_q, r_k = oracle.qk_gather_backward(_ref(g), _ref(q), _ref(k), idx)
    assert oracle.rel_err(d_q, r_q) <= grad_tol and oracle.rel_err(d_k, r_k) <= grad_tol

    p = torch.softmax(attn_ref, -1).to(dtype)
    feat = clustenav_cuda.forward(p.to(device), vd, idxd)
    feat_ref = oracle.av_gather_chunked(_ref(p), _ref(v), idx)
    assert feat.dtype == dtype and oracle.rel_err(feat, feat_ref) <= TOL[dtype]
    g = torch.randn(feat_ref.shape, generator=wl.generator(6)).to(dtype)
    d_p, d_v = clustenav_cuda.backward(g.to(device), p.to(device), vd, idxd)
    r_p, r_v = oracle.av_gather_backward(_ref(g), _ref(p), _ref(v), idx)
    assert oracle.rel_err(d_p, r_p) <= grad_tol and oracle.rel_err(d_v, r_v) <= grad_tol


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_wf_module(device, dtype):
    case = wl.wf_case("ext", 322, 2, 196, 32, IC=4, dtype=dtype, Nout=64)   # the reference script's shape, b = 2
    w, f, idx = case.weights, case.feat, case.nbhd_idx
    wd, fd, idxd = w.to(device), f.to(device), idx.to(device)
    grad_tol = TOL_SCATTER_F32 if dtype == torch.float32 else 2e-2
    out = clustenwf_cuda.forward(wd, fd, idxd)
    out_ref = oracle.wf_gather_chunked(_ref(w), _ref(f), idx)
    assert out.shape == out_ref.shape and oracle.rel_err(out, out_ref) <= TOL[dtype]
    g = torch.randn(out_ref.shape, generator=wl.generator(7)).to(dtype)
    d_w, d_f = clustenwf_cuda.backward(g.to(device), wd, fd, idxd)
    r_w, r_f = oracle.wf_gather_backward(_ref(g), _ref(w), _ref(f), idx)
    assert oracle.rel_err(d_w, r_w) <= grad_tol and oracle.rel_err(d_f, r_f) <= grad_tol


def test_modules_import_as_top_level_names():
    """clusten/clusten.py:9-11 says `import clustenqk_cuda` etc.: with the directory itself on sys.path that works."""
    import importlib
    import os
    import sys

    import clusten_ext
    sys.path.insert(0, os.path.dirname(clusten_ext.__file__))
    try:
        for name in ("clustenqk_cuda", "clustenav_cuda", "clustenwf_cuda"):
            mod = importlib.import_module(name)
            assert callable(mod.forward) and callable(mod.backward)
    finally:
        sys.path.pop(0)
        for name in ("clustenqk_cuda", "clustenav_cuda", "clustenwf_cuda", "clusten_hip_abi"):
            sys.modules.pop(name, None)
