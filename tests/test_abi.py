"""The C-ABI shared libraries load, export every symbol that include/clusten_hip.h (the operators) and
include/clusten_probe.h (the measurement kernels) declare, and reject bad arguments with the documented status codes.  No kernel is launched: every call below
returns from the argument checks, so the file runs without a GPU."""
import ctypes
import os
import re

import pytest

from conftest import ROOT
from clusten import _native
import probe

HEADER = os.path.join(ROOT, "include", "clusten_hip.h")
PROBE_HEADER = os.path.join(ROOT, "include", "clusten_probe.h")


def _declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(clusten_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_binds():
    assert _declared_functions() == sorted(_native.EXPORTS)
    assert _declared_functions(PROBE_HEADER) == sorted(probe.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_native.library_path())
    for name in _declared_functions():
        assert hasattr(lib, name), name
    plib = ctypes.CDLL(probe.library_path())
    for name in _declared_functions(PROBE_HEADER):
        assert hasattr(plib, name), name


def test_measurement_kernels_are_not_in_the_operator_library():
    lib = ctypes.CDLL(_native.library_path())
    for name in _declared_functions(PROBE_HEADER):
        assert not hasattr(lib, name), name
    assert probe.load().clusten_probe_abi_version() == probe.ABI_VERSION


def test_abi_version_and_status_strings():
    lib = _native.load()
    assert lib.clusten_abi_version() == _native.ABI_VERSION
    seen = set()
    for code in range(0, 9):
        s = lib.clusten_status_string(code).decode()
        assert s and s not in seen
        seen.add(s)
    assert lib.clusten_status_string(99).decode() == "unknown status"


def _shape(**kw):
    d = dict(B=1, H=1, N=8, C=16, M=4)
    d.update(kw)
    return _native.AttnShape(**d)


def _wshape(**kw):
    d = dict(B=1, N=8, Nout=2, C=64, M=4, IC=4)
    d.update(kw)
    return _native.WfShape(**d)


P = ctypes.c_void_p
FAKE = P(0x1000)  # never dereferenced: the calls below fail their argument checks first
ROWS = _native.Strides(8 * 16, 8 * 16, 16)


def test_null_pointers_are_rejected():
    lib = _native.load()
    assert lib.clusten_qk_forward(P(0), ROWS, FAKE, ROWS, FAKE, FAKE, _shape(), 0, P(0)) == 1
    assert lib.clusten_av_forward(FAKE, FAKE, ROWS, P(0), FAKE, ROWS, _shape(), 0, P(0)) == 1
    assert lib.clusten_wf_forward(FAKE, FAKE, FAKE, P(0), _wshape(), 0, P(0)) == 1
    assert lib.clusten_qk_backward(FAKE, FAKE, ROWS, FAKE, ROWS, FAKE, P(0), FAKE, P(0), 0, _shape(), 0, P(0)) == 1
    assert lib.clusten_av_backward(FAKE, ROWS, FAKE, FAKE, ROWS, FAKE, FAKE, P(0), P(0), 0, _shape(), 0, P(0)) == 1
    assert lib.clusten_wf_backward(FAKE, FAKE, FAKE, FAKE, FAKE, P(0), P(0), 0, _wshape(), 0, P(0)) == 1
    assert probe.load().clusten_copy_probe(P(0), FAKE, 16, P(0)) == 1


@pytest.mark.parametrize("dtype", [-1, 4, 17])
def test_bad_dtype_is_rejected(dtype):
    lib = _native.load()
    assert lib.clusten_qk_forward(FAKE, ROWS, FAKE, ROWS, FAKE, FAKE, _shape(), dtype, P(0)) == 2
    assert lib.clusten_av_forward(FAKE, FAKE, ROWS, FAKE, FAKE, ROWS, _shape(), dtype, P(0)) == 2
    assert lib.clusten_wf_forward(FAKE, FAKE, FAKE, FAKE, _wshape(), dtype, P(0)) == 2
    assert lib.clusten_qk_backward_workspace_bytes(_shape(), dtype) == 0


def test_bad_dims_are_rejected():
    lib = _native.load()
    for bad in (dict(B=0), dict(H=-1), dict(N=0), dict(C=0), dict(M=0), dict(H=64, N=1 << 20, M=64)):
        assert lib.clusten_qk_forward(FAKE, ROWS, FAKE, ROWS, FAKE, FAKE, _shape(**bad), 0, P(0)) == 3, bad
    for bad in (dict(B=0), dict(Nout=0), dict(IC=0), dict(N=1 << 24, C=512)):
        assert lib.clusten_wf_forward(FAKE, FAKE, FAKE, FAKE, _wshape(**bad), 0, P(0)) == 3, bad
    assert probe.load().clusten_copy_probe(FAKE, FAKE, 24, P(0)) == 3
    assert probe.load().clusten_copy_probe(FAKE, P(0x1008), 32, P(0)) == 7


def test_bad_strides_are_rejected():
    lib = _native.load()
    overlapping = _native.Strides(128, 128, 8)   # token stride smaller than the head dim
    negative = _native.Strides(-128, 128, 16)
    for s in (overlapping, negative):
        assert lib.clusten_qk_forward(FAKE, s, FAKE, ROWS, FAKE, FAKE, _shape(), 0, P(0)) == 4
        assert lib.clusten_av_forward(FAKE, FAKE, s, FAKE, FAKE, ROWS, _shape(), 0, P(0)) == 4


def test_workspace_contract():
    lib = _native.load()
    s = _shape(B=2, H=2, N=16, C=32, M=8)
    assert lib.clusten_qk_backward_workspace_bytes(s, 3) == 0          # fp64: atomics straight into d_key
    pairs = lib.clusten_cluster_pairs_bytes(2, 16, 8, 16)              # the pair lists of (B,N,M) lists over N rows
    assert pairs > 0 and pairs % 256 == 0
    tiles = 256                                                        # one byte per tile of 8 tokens, to 256 bytes
    assert lib.clusten_qk_backward_workspace_bytes(s, 0) == pairs + tiles   # fp32 accumulates in place
    need = lib.clusten_qk_backward_workspace_bytes(s, 1)
    assert need == pairs + tiles + 2 * 2 * 16 * 32 * 4                  # ... plus one fp32 per d_key element
    assert lib.clusten_av_backward_workspace_bytes(s, 2) == need
    odd = _shape(B=2, H=2, N=16, C=32, M=5)                            # no runs of 8: no pair lists
    assert lib.clusten_qk_backward_workspace_bytes(odd, 0) == 0
    assert lib.clusten_qk_backward_workspace_bytes(odd, 1) == 2 * 2 * 16 * 32 * 4
    assert lib.clusten_cluster_pairs_bytes(2, 16, 5, 16) == 0 and lib.clusten_cluster_pairs_bytes(2, 16, 8, 4) == 0
    rows = _native.Strides(2 * 16 * 32, 16 * 32, 32)
    assert lib.clusten_qk_backward(FAKE, FAKE, rows, FAKE, rows, FAKE, FAKE, FAKE, P(0), 0, s, 1, P(0)) == 5
    assert lib.clusten_qk_backward(FAKE, FAKE, rows, FAKE, rows, FAKE, FAKE, FAKE, FAKE, need - 1, s, 1, P(0)) == 5
    w = _wshape(B=2, N=16, Nout=4, C=64, M=8, IC=4)
    wpairs = lib.clusten_cluster_pairs_bytes(2, 4, 8, 16)
    wf32 = lib.clusten_wf_backward_workspace_bytes(w, 0)
    assert wf32 >= wpairs + 2 * 4 * 8 * 4 + 2 * 2 * 16 * 4              # pair lists, then the entries by destination row
    assert lib.clusten_wf_backward_workspace_bytes(w, 2) == wf32 + 2 * 16 * 64 * 4
    assert lib.clusten_wf_backward_workspace_bytes(w, 3) == 0          # fp64: atomics straight into d_feat
    assert lib.clusten_wf_backward(FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, P(0), 0, w, 2, P(0)) == 5


def test_python_surface_fails_loudly_without_a_gpu_tensor():
    import torch
    from clusten import CLUSTENQKFunction, CLUSTENAVFunction, CLUSTENWFFunction
    q = torch.randn(1, 1, 8, 16)
    idx = torch.zeros(1, 8, 4, dtype=torch.long)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        CLUSTENQKFunction.apply(q, q, idx)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        CLUSTENAVFunction.apply(torch.randn(1, 1, 8, 4), q, idx)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        CLUSTENWFFunction.apply(torch.randn(1, 2, 4, 4), torch.randn(1, 8, 64), torch.zeros(1, 2, 4, dtype=torch.long))


def test_debug_index_check_raises_on_stray_entries(monkeypatch):
    """The optional range check of the shim (the reference checks no index either: clustenqk_cuda.cpp:21-23)."""
    import torch
    idx = torch.tensor([[[0, 3, 7], [1, 2, 6]]])
    _native.check_index_range(idx, 8)                       # all inside [0, 8)
    with pytest.raises(RuntimeError, match=r"outside \[0, 7\): min 0, max 7"):
        _native.check_index_range(idx, 7)
    with pytest.raises(RuntimeError, match="min -1"):
        _native.check_index_range(idx - 1, 8)
    _native.check_index_range(idx[:, :0], 8)                # nothing to check
    monkeypatch.delenv("CLUSTEN_DEBUG_INDICES", raising=False)
    assert not _native.debug_indices()
    monkeypatch.setenv("CLUSTEN_DEBUG_INDICES", "0")
    assert not _native.debug_indices()
    monkeypatch.setenv("CLUSTEN_DEBUG_INDICES", "1")
    assert _native.debug_indices()
