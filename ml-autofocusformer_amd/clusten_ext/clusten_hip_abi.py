"""ctypes view of libclusten_hip.so shared by the three modules of this directory.

The modules carry the names and the `forward` / `backward` signatures of the reference's pybind11 extension modules
(clusten/src/clustenqk_cuda.cpp:48-51, clustenav_cuda.cpp:48-51, clustenwf_cuda.cpp:48-51), so that the reference's
own clusten/clusten.py:9-11 can import them unchanged: put this directory on sys.path ahead of the compiled modules.
The library is looked up in $CLUSTEN_HIP_LIB, else next to this package (../lib/libclusten_hip.so).
"""
import ctypes
import os

import torch

_DEFAULT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "lib", "libclusten_hip.so")
_path = os.environ.get("CLUSTEN_HIP_LIB", _DEFAULT)
if not os.path.exists(_path):
    raise RuntimeError("libclusten_hip.so not found at %s: build it with make -C csrc" % _path)
lib = ctypes.CDLL(_path)

P = ctypes.c_void_p


class Strides(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int64) for k in ("b", "h", "n")]


class AttnShape(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int32) for k in ("B", "H", "N", "C", "M")]


class WfShape(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int32) for k in ("B", "N", "Nout", "C", "M", "IC")]


CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3}

lib.clusten_status_string.restype = ctypes.c_char_p
lib.clusten_status_string.argtypes = [ctypes.c_int]
for _name, _shape in (("qk", AttnShape), ("av", AttnShape), ("wf", WfShape)):
    _fn = getattr(lib, "clusten_%s_backward_workspace_bytes" % _name)
    _fn.restype = ctypes.c_size_t
    _fn.argtypes = [_shape, ctypes.c_int]
lib.clusten_qk_forward.argtypes = [P, Strides, P, Strides, P, P, AttnShape, ctypes.c_int, P]
lib.clusten_qk_backward.argtypes = [P, P, Strides, P, Strides, P, P, P, P, ctypes.c_size_t, AttnShape, ctypes.c_int, P]
lib.clusten_av_forward.argtypes = [P, P, Strides, P, P, Strides, AttnShape, ctypes.c_int, P]
lib.clusten_av_backward.argtypes = [P, Strides, P, P, Strides, P, P, P, P, ctypes.c_size_t, AttnShape, ctypes.c_int, P]
lib.clusten_wf_forward.argtypes = [P, P, P, P, WfShape, ctypes.c_int, P]
lib.clusten_wf_backward.argtypes = [P, P, P, P, P, P, P, ctypes.c_size_t, WfShape, ctypes.c_int, P]


def strides(t):
    return Strides(t.stride(0), t.stride(1), t.stride(2))


def stream(t):
    return P(torch.cuda.current_stream(t.device).cuda_stream)


def ptr(t):
    return P(t.data_ptr())


def check_cuda(*tensors):
    """The reference's CHECK_CUDA / CHECK_CONTIGUOUS (clustenqk_cuda.cpp:21-23) for the operands of a call."""
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("tensor must be a CUDA tensor")


def rows_unit_stride(t):
    """A (b,h,n,c) operand as the library reads it: any batch / head / token strides, channel stride 1."""
    return t if t.stride(3) == 1 else t.contiguous()


def workspace(kind, shape, code, like):
    n = getattr(lib, "clusten_%s_backward_workspace_bytes" % kind)(shape, code)
    buf = torch.empty(max(n, 1), dtype=torch.uint8, device=like.device)
    return (ptr(buf) if n else None), n, buf


def done(what, status):
    if status:
        raise RuntimeError("%s: %s" % (what, lib.clusten_status_string(status).decode()))
