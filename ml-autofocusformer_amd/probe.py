"""ctypes binding of libclusten_probe.so (C ABI in include/clusten_probe.h): measurement kernels for benchmarks.

Not part of the operators: a streaming copy of known traffic, the stream / gather probe, and the three forward kernels
compiled without their arithmetic.  Only a benchmark or a profiler run loads this library.
"""
from __future__ import annotations

import ctypes
import os

import torch

from clusten import _native
from clusten._native import AttnShape, Strides, WfShape, _check, _ptr, _require_cuda, _stream

_LIB_PATH = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libclusten_probe.so"))

ABI_VERSION = 1

_P = ctypes.c_void_p
_PROTOTYPES = {
    # name: (restype, argtypes)  — one entry per declaration in include/clusten_probe.h
    "clusten_probe_abi_version": (ctypes.c_int, []),
    "clusten_copy_probe": (ctypes.c_int, [_P, _P, ctypes.c_size_t, _P]),
    "clusten_stream_gather_probe": (ctypes.c_int, [_P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                   ctypes.c_int, _P]),
    "clusten_qk_forward_replay": (ctypes.c_int, [_P, Strides, _P, Strides, _P, _P, AttnShape, ctypes.c_int, _P]),
    "clusten_av_forward_replay": (ctypes.c_int, [_P, _P, Strides, _P, _P, Strides, AttnShape, ctypes.c_int, _P]),
    "clusten_wf_forward_replay": (ctypes.c_int, [_P, _P, _P, _P, WfShape, ctypes.c_int, _P]),
}

EXPORTS = tuple(_PROTOTYPES)

_lib = None


def library_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load libclusten_probe.so once.  Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError("Could not load the CLUSTEN probe library (%s). Build it with "
                               "`make -C ml-autofocusformer_amd/csrc` (hipcc, gfx950)." % _LIB_PATH)
        try:
            lib = ctypes.CDLL(_LIB_PATH)
        except OSError as e:
            raise RuntimeError("Could not load the CLUSTEN probe library (%s): %s" % (_LIB_PATH, e)) from e
        for name, (restype, argtypes) in _PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.clusten_probe_abi_version() != ABI_VERSION:
            raise RuntimeError("libclusten_probe.so has ABI version %d, this binding expects %d" %
                               (lib.clusten_probe_abi_version(), ABI_VERSION))
        _lib = lib
    return _lib


def qk_forward_replay(query: torch.Tensor, key: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """The QK forward kernels without their arithmetic (fp32): same loads, LDS traffic and stores; the result holds no
    meaningful values."""
    return _native.qk_forward(query, key, nbhd_idx, _entry=load().clusten_qk_forward_replay)


def av_forward_replay(attn: torch.Tensor, v: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """The AV forward kernels without their arithmetic (fp32)."""
    return _native.av_forward(attn, v, nbhd_idx, _entry=load().clusten_av_forward_replay)


def wf_forward_replay(weights: torch.Tensor, feat: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """The WF forward kernels without their arithmetic (fp32)."""
    return _native.wf_forward(weights, feat, nbhd_idx, _entry=load().clusten_wf_forward_replay)


def copy_probe(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst <- src with the probe library's streaming copy kernel."""
    lib = load()
    _require_cuda("src", src)
    _require_cuda("dst", dst, src.device)
    nbytes = src.numel() * src.element_size()
    if not (src.is_contiguous() and dst.is_contiguous()) or dst.numel() * dst.element_size() != nbytes:
        raise RuntimeError("copy_probe needs contiguous tensors of equal byte size")
    with torch.cuda.device(src.device):
        _check(lib.clusten_copy_probe(_ptr(src), _ptr(dst), nbytes, _stream(src.device)), "clusten_copy_probe")


def stream_gather_probe(stream_in: torch.Tensor, stream_out: torch.Tensor, rows: torch.Tensor, tiles: int, gathers: int,
                        window_rows: int, tiles_per_window: int, mode: int) -> None:
    """`clusten_stream_gather_probe`: per tile, mode bit 0 = read 5 KiB of `stream_in` and write 3 KiB of `stream_out`,
    bit 1 = gather `gathers` x 1 KiB of random 256-byte rows inside the tile's window of `rows`."""
    lib = load()
    _require_cuda("stream_in", stream_in)
    device = stream_in.device
    _require_cuda("stream_out", stream_out, device)
    _require_cuda("rows", rows, device)
    nbytes = lambda t: t.numel() * t.element_size()
    windows = (tiles + tiles_per_window - 1) // tiles_per_window
    if (nbytes(stream_in) < tiles * 5120 or nbytes(stream_out) < tiles * 3072
            or nbytes(rows) < windows * window_rows * 256):
        raise RuntimeError("stream_gather_probe: a buffer is too small for %d tiles" % tiles)
    with torch.cuda.device(device):
        _check(lib.clusten_stream_gather_probe(_ptr(stream_in), _ptr(stream_out), _ptr(rows), tiles, gathers, window_rows,
                                               tiles_per_window, mode, _stream(device)), "clusten_stream_gather_probe")
