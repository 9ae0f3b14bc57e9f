"""Builds the C restatement of the CLUSTEN sums (clusten_ref.c) into oracle/_build/libclusten_ref.so
and exposes it through ctypes.  TEST INFRASTRUCTURE ONLY.

`/root/reference` holds no CPU-buildable implementation of this path (its kernels are CUDA sources
that need nvcc and ATen headers), so there is no `oracle/_ref` build: this file compiles the
build's own C statement of the sums only.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "clusten_ref.c")
_OUT_DIR = os.path.join(_HERE, "_build")
_LIB = os.path.join(_OUT_DIR, "libclusten_ref.so")


def build(force: bool = False) -> str:
    """Compile clusten_ref.c with gcc; returns the path of the shared object."""
    os.makedirs(_OUT_DIR, exist_ok=True)
    stale = not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(_SRC)
    if force or stale:
        subprocess.run(["gcc", "-O2", "-fPIC", "-shared", "-std=c99", "-o", _LIB, _SRC], check=True)
    return _LIB


_lib = None


def load() -> ctypes.CDLL:
    """Load the prebuilt library (building it when a compiler is at hand and it is missing)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = ctypes.CDLL(_LIB)
    return _lib


def _f32(t):
    t = t.detach().to(torch.float32).cpu().contiguous()
    return t, ctypes.c_void_p(t.data_ptr())


def _i64(t):
    t = t.detach().to(torch.int64).cpu().contiguous()
    return t, ctypes.c_void_p(t.data_ptr())


def qk_forward(query, key, nbhd_idx):
    lib = load()
    b, h, n, c = query.shape
    m = nbhd_idx.shape[-1]
    q, qp = _f32(query)
    k, kp = _f32(key)
    i, ip = _i64(nbhd_idx)
    out = torch.empty(b, h, n, m, dtype=torch.float32)
    lib.ref_qk_forward(qp, kp, ip, ctypes.c_void_p(out.data_ptr()), b, h, n, c, m)
    return out


def av_forward(attn, v, nbhd_idx):
    lib = load()
    b, h, n, m = attn.shape
    c = v.shape[-1]
    a, ap = _f32(attn)
    vv, vp = _f32(v)
    i, ip = _i64(nbhd_idx)
    out = torch.empty(b, h, n, c, dtype=torch.float32)
    lib.ref_av_forward(ap, vp, ip, ctypes.c_void_p(out.data_ptr()), b, h, n, c, m)
    return out


def wf_forward(weights, feat, nbhd_idx):
    lib = load()
    b, n_out, m, ic = weights.shape
    n, c = feat.shape[1], feat.shape[2]
    w, wp = _f32(weights)
    f, fp = _f32(feat)
    i, ip = _i64(nbhd_idx)
    out = torch.empty(b, n_out, ic, c, dtype=torch.float32)
    lib.ref_wf_forward(wp, fp, ip, ctypes.c_void_p(out.data_ptr()), b, n, n_out, c, m, ic)
    return out


def qk_backward(d_attn, query, key, nbhd_idx):
    lib = load()
    b, h, n, c = query.shape
    m = nbhd_idx.shape[-1]
    g, gp = _f32(d_attn)
    q, qp = _f32(query)
    k, kp = _f32(key)
    i, ip = _i64(nbhd_idx)
    dq = torch.empty(b, h, n, c, dtype=torch.float32)
    dk = torch.empty(b, h, n, c, dtype=torch.float32)
    lib.ref_qk_backward(gp, qp, kp, ip, ctypes.c_void_p(dq.data_ptr()), ctypes.c_void_p(dk.data_ptr()), b, h, n, c, m)
    return dq, dk


def av_backward(d_feat, attn, v, nbhd_idx):
    lib = load()
    b, h, n, m = attn.shape
    c = v.shape[-1]
    g, gp = _f32(d_feat)
    a, ap = _f32(attn)
    vv, vp = _f32(v)
    i, ip = _i64(nbhd_idx)
    da = torch.empty(b, h, n, m, dtype=torch.float32)
    dv = torch.empty(b, h, n, c, dtype=torch.float32)
    lib.ref_av_backward(gp, ap, vp, ip, ctypes.c_void_p(da.data_ptr()), ctypes.c_void_p(dv.data_ptr()), b, h, n, c, m)
    return da, dv


def wf_backward(d_feat_new, weights, feat, nbhd_idx):
    lib = load()
    b, n_out, m, ic = weights.shape
    n, c = feat.shape[1], feat.shape[2]
    g, gp = _f32(d_feat_new)
    w, wp = _f32(weights)
    f, fp = _f32(feat)
    i, ip = _i64(nbhd_idx)
    dw = torch.empty(b, n_out, m, ic, dtype=torch.float32)
    df = torch.empty(b, n, c, dtype=torch.float32)
    lib.ref_wf_backward(gp, wp, fp, ip, ctypes.c_void_p(dw.data_ptr()), ctypes.c_void_p(df.data_ptr()), b, n, n_out, c,
                        m, ic)
    return dw, df


if __name__ == "__main__":
    print(build(force=True))
