"""ctypes binding of libclusten_hip.so (C ABI in include/clusten_hip.h) for PyTorch-ROCm tensors.

PyTorch is used for device memory and streams only: outputs and workspaces are allocated with
`torch.empty` (stream-ordered caching allocator), kernels are enqueued on the tensor device's
current stream, nothing synchronises and nothing is remembered between calls.  There is no CPU path and no fallback: a missing library,
a CPU tensor or a non-zero status raises RuntimeError.
"""
from __future__ import annotations

import ctypes
import os

import torch

_LIB_PATH = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "lib", "libclusten_hip.so"))

ABI_VERSION = 4

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3}


class AttnShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("B", "H", "N", "C", "M")]


class Strides(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("b", "h", "n")]


class WfShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("B", "N", "Nout", "C", "M", "IC")]


_P = ctypes.c_void_p
_PROTOTYPES = {
    # name: (restype, argtypes)  — one entry per declaration in include/clusten_hip.h
    "clusten_abi_version": (ctypes.c_int, []),
    "clusten_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "clusten_qk_forward": (ctypes.c_int, [_P, Strides, _P, Strides, _P, _P, AttnShape, ctypes.c_int, _P]),
    "clusten_qk_backward_workspace_bytes": (ctypes.c_size_t, [AttnShape, ctypes.c_int]),
    "clusten_qk_backward": (ctypes.c_int, [_P, _P, Strides, _P, Strides, _P, _P, _P, _P, ctypes.c_size_t, AttnShape,
                                           ctypes.c_int, _P]),
    "clusten_qk_backward_static": (ctypes.c_int, [_P, _P, Strides, _P, Strides, _P, _P, _P, AttnShape, ctypes.c_int, _P]),
    "clusten_av_forward": (ctypes.c_int, [_P, _P, Strides, _P, _P, Strides, AttnShape, ctypes.c_int, _P]),
    "clusten_av_forward_mixed": (ctypes.c_int, [_P, _P, Strides, ctypes.c_int, _P, _P, Strides, AttnShape, _P]),
    "clusten_av_backward_workspace_bytes": (ctypes.c_size_t, [AttnShape, ctypes.c_int]),
    "clusten_av_backward": (ctypes.c_int, [_P, Strides, _P, _P, Strides, _P, _P, _P, _P, ctypes.c_size_t, AttnShape,
                                           ctypes.c_int, _P]),
    "clusten_wf_forward": (ctypes.c_int, [_P, _P, _P, _P, WfShape, ctypes.c_int, _P]),
    "clusten_wf_forward_mixed": (ctypes.c_int, [_P, _P, ctypes.c_int, _P, _P, WfShape, _P]),
    "clusten_wf_backward_workspace_bytes": (ctypes.c_size_t, [WfShape, ctypes.c_int]),
    "clusten_wf_backward": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, ctypes.c_size_t, WfShape, ctypes.c_int, _P]),
    "clusten_cluster_size_for": (ctypes.c_int, [ctypes.c_int]),
    "clusten_cluster_pairs_from_numbers": (ctypes.c_int, [_P, _P, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                          ctypes.c_int, _P]),
    "clusten_qk_forward_clusters": (ctypes.c_int, [_P, Strides, _P, Strides, _P, _P, AttnShape, ctypes.c_int, _P]),
    "clusten_av_forward_clusters": (ctypes.c_int, [_P, _P, Strides, _P, _P, Strides, AttnShape, ctypes.c_int, _P]),
    "clusten_attn_softmax_forward": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, Strides, _P, _P, _P, AttnShape, ctypes.c_int,
                                                   _P]),
    "clusten_cluster_attention_forward": (ctypes.c_int, [_P, Strides, _P, Strides, _P, Strides, _P, _P, _P, _P,
                                                        ctypes.c_int, _P, _P, _P, Strides, ctypes.c_float, AttnShape,
                                                        ctypes.c_int, _P]),
    "clusten_cluster_attention_plan_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "clusten_cluster_attention_plan": (ctypes.c_int, [_P, _P, _P, _P, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                                     ctypes.c_int, _P]),
    "clusten_cluster_attention_forward_planned": (ctypes.c_int, [_P, Strides, _P, Strides, _P, Strides, _P, _P,
                                                                ctypes.c_int, _P, _P, _P, Strides, ctypes.c_float,
                                                                AttnShape, ctypes.c_int, _P]),
    "clusten_cluster_attention_forward_train": (ctypes.c_int, [_P, Strides, _P, Strides, _P, Strides, _P, _P, ctypes.c_int,
                                                               _P, _P, _P, Strides, _P, ctypes.c_float, AttnShape,
                                                               ctypes.c_int, _P]),
    "clusten_cluster_attention_backward": (ctypes.c_int, [_P, Strides, _P, Strides, _P, Strides, _P, Strides, _P, Strides,
                                                          _P, _P, _P, ctypes.c_int, _P, _P, _P, Strides, _P, _P, _P, _P,
                                                          ctypes.c_float, AttnShape, ctypes.c_int, _P]),
    "clusten_cluster_pairs_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "clusten_cluster_pairs": (ctypes.c_int, [_P, _P, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                             ctypes.c_int, _P]),
    "clusten_wf_backward_by_cluster": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, WfShape, ctypes.c_int, _P]),
    "clusten_scatter_rows_by_cluster": (ctypes.c_int, [_P, _P, Strides, _P, _P, AttnShape, ctypes.c_int, _P]),
    "clusten_scatter_rows_workspace_bytes": (ctypes.c_size_t, [AttnShape, ctypes.c_int]),
    "clusten_scatter_rows": (ctypes.c_int, [_P, _P, Strides, _P, _P, _P, _P, ctypes.c_size_t, AttnShape, ctypes.c_int,
                                            _P]),
    "clusten_dense_attention_forward": (ctypes.c_int, [_P, Strides, _P, Strides, _P, Strides, _P, _P, _P, _P, _P, Strides,
                                                      ctypes.c_float, AttnShape, ctypes.c_int, _P]),
    "clusten_linear_supported": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "clusten_linear_forward": (ctypes.c_int, [_P, ctypes.c_int64, _P, _P, _P, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                             ctypes.c_int, ctypes.c_int, _P]),
    "clusten_layer_norm_forward": (ctypes.c_int, [_P, ctypes.c_int, _P, _P, _P, ctypes.c_int64, ctypes.c_int,
                                                 ctypes.c_float, ctypes.c_int, _P]),
    "clusten_layer_norm_rows_forward": (ctypes.c_int, [_P, ctypes.c_int, _P, ctypes.c_int, _P, _P, _P, _P, ctypes.c_int64,
                                                      ctypes.c_int, ctypes.c_float, ctypes.c_int, _P]),
    "clusten_channel_affine_gelu_forward": (ctypes.c_int, [_P, _P, _P, _P, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                                          ctypes.c_int, _P]),
    "clusten_add_row_score_forward": (ctypes.c_int, [_P, ctypes.c_int, _P, _P, _P, _P, _P, ctypes.c_int64, ctypes.c_int,
                                                    ctypes.c_int, _P]),
    "clusten_add_layer_norm_forward": (ctypes.c_int, [_P, ctypes.c_int, _P, ctypes.c_int, _P, _P, _P, _P, ctypes.c_int64,
                                                     ctypes.c_int, ctypes.c_float, _P]),
    "clusten_neighbour_lists": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
    "clusten_attn_softmax_backward": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                                    _P]),
    "clusten_bias_table_grad": (ctypes.c_int, [_P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_int, ctypes.c_int, _P]),
    "clusten_merge_weights_forward": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                    ctypes.c_int, ctypes.c_int, _P]),
    "clusten_scanline_rank_max_tokens": (ctypes.c_int, []),
    "clusten_cluster_centres": (ctypes.c_int, [_P, _P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
    "clusten_gather_rows": (ctypes.c_int, [_P, _P, _P, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
    "clusten_merge_centres_max_tokens": (ctypes.c_int, []),
    "clusten_merge_centres": (ctypes.c_int, [_P, _P, _P, ctypes.c_int, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_int, _P]),
    "clusten_merge_rows": (ctypes.c_int, [_P, _P, _P, ctypes.c_int, _P, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _P]),
    "clusten_scanline_rank_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int]),
    "clusten_scanline_rank": (ctypes.c_int, [_P, _P, _P, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_float, ctypes.c_float, _P]),
    "clusten_knn2d": (ctypes.c_int, [_P, _P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
}

EXPORTS = tuple(_PROTOTYPES)

_lib = None


def library_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load libclusten_hip.so once.  Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                "Could not load the CLUSTEN HIP library (%s). Build it with `make -C ml-autofocusformer_amd/csrc` "
                "(hipcc, gfx950); there is no CPU or PyTorch fallback." % _LIB_PATH)
        try:
            lib = ctypes.CDLL(_LIB_PATH)
        except OSError as e:  # e.g. the HIP runtime is missing
            raise RuntimeError("Could not load the CLUSTEN HIP library (%s): %s" % (_LIB_PATH, e)) from e
        for name, (restype, argtypes) in _PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.clusten_abi_version() != ABI_VERSION:
            raise RuntimeError("libclusten_hip.so has ABI version %d, this binding expects %d" %
                               (lib.clusten_abi_version(), ABI_VERSION))
        _lib = lib
    return _lib


def _check(status: int, what: str) -> None:
    if status != 0:
        raise RuntimeError("%s failed: %s (status %d)" % (what, load().clusten_status_string(status).decode(), status))


def _dtype_code(t: torch.Tensor, name: str) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise RuntimeError("%s has unsupported dtype %s (float32, float16, bfloat16, float64)" % (name, t.dtype))


def _require_cuda(name: str, t: torch.Tensor, device=None) -> None:
    # same message as the reference's CHECK_CUDA (clusten/src/clustenqk_cuda.cpp:21)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if device is not None and t.device != device:
        raise RuntimeError("%s is on %s, expected %s" % (name, t.device, device))


def _rows(t: torch.Tensor) -> torch.Tensor:
    """A (B,H,N,C) tensor the kernels can address: channel stride 1, rows that do not overlap.
    Anything else (e.g. a transposed channel axis) is copied, as the reference always does
    (clusten/clusten.py:23-24)."""
    sb, sh, sn, sc = t.stride()
    C = t.shape[3]
    if (sc == 1 or C == 1) and sn >= C and sb >= 0 and sh >= 0:
        return t
    return t.contiguous()


def _strides(t: torch.Tensor) -> Strides:
    return Strides(t.stride(0), t.stride(1), t.stride(2))


def _ptr(t) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def debug_indices() -> bool:
    """True when the environment asks for the index-range check (CLUSTEN_DEBUG_INDICES set to anything but 0 / empty)."""
    return os.environ.get("CLUSTEN_DEBUG_INDICES", "0") not in ("", "0")


def check_index_range(nbhd_idx: torch.Tensor, n_rows: int, name: str = "nbhd_idx") -> None:
    """Raise RuntimeError unless every entry of `nbhd_idx` lies in [0, n_rows).  The kernels, like the reference's
    (clusten/src/clustenqk_cuda.cpp:21-23 checks devices and contiguity only), read rows at whatever index they are
    given; a stray index is an out-of-bounds access on the device.  This check reads the extrema back to the host and
    therefore synchronises: it runs only under CLUSTEN_DEBUG_INDICES=1."""
    if nbhd_idx.numel() == 0:
        return
    lo, hi = int(nbhd_idx.min()), int(nbhd_idx.max())
    if lo < 0 or hi >= n_rows:
        raise RuntimeError("%s holds entries outside [0, %d): min %d, max %d" % (name, n_rows, lo, hi))


def _idx(nbhd_idx: torch.Tensor, shape, device, n_rows=None) -> torch.Tensor:
    """The list tensor as the kernels take it; `n_rows` = length of the sequence its entries point into (the second
    entry of `shape` unless given), used by the optional range check."""
    _require_cuda("nbhd_idx", nbhd_idx, device)
    if nbhd_idx.dtype != torch.int64:
        raise RuntimeError("nbhd_idx must be int64, got %s" % nbhd_idx.dtype)
    if tuple(nbhd_idx.shape[:2]) != tuple(shape):
        raise RuntimeError("nbhd_idx has shape %s, expected (%d, %d, m)" % (tuple(nbhd_idx.shape), shape[0], shape[1]))
    if debug_indices():
        check_index_range(nbhd_idx, shape[1] if n_rows is None else n_rows)
    return nbhd_idx.contiguous()


def _attn_problem(a: torch.Tensor, rows: torch.Tensor, nbhd_idx: torch.Tensor, names):
    """Common checks of (query,key) / (d_feat,value) pairs: returns device, dtype code, idx, shape."""
    _require_cuda(names[0], a)
    device = a.device
    _require_cuda(names[1], rows, device)
    if a.dim() != 4 or rows.dim() != 4 or nbhd_idx.dim() != 3:
        raise RuntimeError("%s and %s must be (b,h,n,c) and nbhd_idx (b,n,m)" % names)
    if a.shape != rows.shape:
        raise RuntimeError("%s %s and %s %s must have the same shape" % (names[0], tuple(a.shape), names[1],
                                                                         tuple(rows.shape)))
    if a.dtype != rows.dtype:
        raise RuntimeError("%s and %s must have the same dtype" % names)
    B, H, N, C = a.shape
    idx = _idx(nbhd_idx, (B, N), device)
    return device, _dtype_code(a, names[0]), idx, AttnShape(B, H, N, C, idx.shape[2])


def qk_forward(query: torch.Tensor, key: torch.Tensor, nbhd_idx: torch.Tensor, _entry=None) -> torch.Tensor:
    """attn (b,h,n,m) = query · key[nbhd_idx]; query/key (b,h,n,c) may be strided views.  (`_entry`: another library's
    function of the same signature, for the measurement bindings of probe.py.)"""
    lib = load()
    device, code, idx, shape = _attn_problem(query, key, nbhd_idx, ("query", "key"))
    query, key = _rows(query), _rows(key)
    attn = torch.empty((shape.B, shape.H, shape.N, shape.M), dtype=query.dtype, device=device)
    if attn.numel() == 0:
        return attn
    with torch.cuda.device(device):
        fn = _entry or lib.clusten_qk_forward
        _check(fn(_ptr(query), _strides(query), _ptr(key), _strides(key), _ptr(idx), _ptr(attn), shape, code,
                  _stream(device)), "clusten_qk_forward")
    return attn


def cluster_pairs(nbhd_idx: torch.Tensor, n_rows=None):
    """The pair lists of `nbhd_idx` (b,rows,m) int64, whose entries point into sequences of `n_rows` rows (rows by
    default): an opaque uint8 block for `scatter_rows_by_cluster` / `wf_backward_by_cluster`, built on the device by
    `clusten_cluster_pairs` (keys, then a stable counting sort per image); the host reads nothing back.  Its first
    int32 (`pairs_not_whole`) is 1 when the lists are not made of whole clusters — the consumers then leave their
    outputs untouched.  None when the shape is not supported (m not a multiple of 8 or above 64, n_rows < 8)."""
    lib = load()
    _require_cuda("nbhd_idx", nbhd_idx)
    if nbhd_idx.dim() != 3 or nbhd_idx.dtype != torch.int64:
        raise RuntimeError("nbhd_idx must be an int64 (b,rows,m) tensor")
    B, rows, M = nbhd_idx.shape
    D = rows if n_rows is None else int(n_rows)
    nbytes = lib.clusten_cluster_pairs_bytes(B, rows, M, D) if B and rows and M else 0
    if nbytes == 0:
        return None
    idx = nbhd_idx.contiguous()
    device = idx.device
    block = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        _check(lib.clusten_cluster_pairs(_ptr(idx), _ptr(block), nbytes, B, rows, M, D, _stream(device)),
               "clusten_cluster_pairs")
    return block


def cluster_pairs_from_numbers(cluster_idx: torch.Tensor, n_rows=None):
    """The block `cluster_pairs` builds for the expanded lists, from the (b,rows,nnc) int32 numbers of clusters of 8 rows
    themselves (`clusten_cluster_pairs_from_numbers`).  A number outside [0, ceil(n_rows / 8)) sets the block's flag.
    None when the shape is not supported."""
    lib = load()
    _require_cuda("cluster_idx", cluster_idx)
    if cluster_idx.dim() != 3 or cluster_idx.dtype != torch.int32:
        raise RuntimeError("cluster_idx must be an int32 (b,rows,clusters per token) tensor")
    B, rows, nnc = cluster_idx.shape
    D = rows if n_rows is None else int(n_rows)
    nbytes = lib.clusten_cluster_pairs_bytes(B, rows, 8 * nnc, D) if B and rows and nnc else 0
    if nbytes == 0:
        return None
    cidx = cluster_idx.contiguous()
    device = cidx.device
    block = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        _check(lib.clusten_cluster_pairs_from_numbers(_ptr(cidx), _ptr(block), nbytes, B, rows, nnc, D, _stream(device)),
               "clusten_cluster_pairs_from_numbers")
    return block


def qk_backward_clusters(d_attn: torch.Tensor, query: torch.Tensor, key: torch.Tensor, cluster_idx: torch.Tensor,
                         pairs=None):
    """(d_query, d_key) of `qk_forward_clusters` (clusters of 8 rows, numbers inside the sequence): a gather on the
    numbers and the by-cluster scatter over `pairs` = `cluster_pairs_from_numbers(cluster_idx)` (built here when not
    given; a caller keeps it for all layers of a stage)."""
    if pairs is None:
        pairs = cluster_pairs_from_numbers(cluster_idx)
    if pairs is None:
        raise RuntimeError("qk_backward_clusters: lists of this shape have no pair lists")
    return av_forward_clusters(d_attn, key, cluster_idx), scatter_rows_by_cluster(d_attn, query, pairs)


def av_backward_clusters(d_feat: torch.Tensor, attn: torch.Tensor, v: torch.Tensor, cluster_idx: torch.Tensor, pairs=None):
    """(d_attn, d_v) of `av_forward_clusters`: see `qk_backward_clusters`."""
    if pairs is None:
        pairs = cluster_pairs_from_numbers(cluster_idx)
    if pairs is None:
        raise RuntimeError("av_backward_clusters: lists of this shape have no pair lists")
    return qk_forward_clusters(d_feat, v, cluster_idx), scatter_rows_by_cluster(attn, d_feat, pairs)


def pairs_not_whole(pair_lists: torch.Tensor) -> torch.Tensor:
    """The flag of a `cluster_pairs` block as a one-element int32 device tensor (reading it on the host synchronises)."""
    return pair_lists[:4].view(torch.int32)


def scatter_rows_by_cluster(p: torch.Tensor, x: torch.Tensor, pair_lists: torch.Tensor, out=None) -> torch.Tensor:
    """y (b,h,n,c) with y[b,h,8g+t] = sum over the pairs (i,r) of cluster (b,g) of p[b,h,i,8r+t] * x[b,h,i]: the d_key /
    d_value of the attention backward passes for lists made of whole clusters, `pair_lists` from `cluster_pairs`.
    When the block's flag says the lists are not whole clusters `out` (new memory unless given) is left untouched."""
    lib = load()
    _require_cuda("p", p)
    device = p.device
    _require_cuda("x", x, device)
    if p.dim() != 4 or x.dim() != 4 or p.shape[:3] != x.shape[:3] or p.dtype != x.dtype:
        raise RuntimeError("p must be (b,h,n,m) and x (b,h,n,c) of one dtype")
    B, H, N, C = x.shape
    M = p.shape[3]
    if pair_lists is None or pair_lists.numel() != lib.clusten_cluster_pairs_bytes(B, N, M, N):
        raise RuntimeError("scatter_rows_by_cluster: pair lists of these lists (cluster_pairs)")
    code = _dtype_code(p, "p")
    p, x = p.contiguous(), _rows(x)
    y = torch.empty((B, H, N, C), dtype=p.dtype, device=device) if out is None else out
    if y.numel() == 0:
        return y
    shape = AttnShape(B, H, N, C, M)
    with torch.cuda.device(device):
        _check(lib.clusten_scatter_rows_by_cluster(_ptr(p), _ptr(x), _strides(x), _ptr(pair_lists), _ptr(y), shape,
                                                   code, _stream(device)),
               "clusten_scatter_rows_by_cluster")
    return y


def _workspace(nbytes: int, device):
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


def scatter_rows(p: torch.Tensor, x: torch.Tensor, nbhd_idx: torch.Tensor, pair_lists=None) -> torch.Tensor:
    """y (b,h,n,c) with y[b,h,nbhd_idx[b,i,j]] += p[b,h,i,j] * x[b,h,i]: the d_key (p = d_attn, x = query) and d_value
    (p = attn, x = d_feat) of the attention backward passes, for any lists.  Lists made of whole clusters take the
    gather over pair lists, anything else the atomic kernels; the device chooses.  `pair_lists`: the block
    `cluster_pairs(nbhd_idx)` made of these lists, kept by the caller across calls (it is otherwise rebuilt here)."""
    lib = load()
    device, code, idx, shape = _attn_problem(x, x, nbhd_idx, ("x", "x"))
    _require_cuda("p", p, device)
    if tuple(p.shape) != (shape.B, shape.H, shape.N, shape.M) or p.dtype != x.dtype:
        raise RuntimeError("p must be (b,h,n,m) with the dtype of x")
    p, x = p.contiguous(), _rows(x)
    y = torch.empty((shape.B, shape.H, shape.N, shape.C), dtype=x.dtype, device=device)
    if y.numel() == 0 or shape.M == 0:
        return y.zero_()
    if pair_lists is not None:
        _require_cuda("pair_lists", pair_lists, device)
        if pair_lists.numel() != lib.clusten_cluster_pairs_bytes(shape.B, shape.N, shape.M, shape.N):
            raise RuntimeError("scatter_rows: pair_lists does not belong to lists of this shape (cluster_pairs)")
    ws_bytes = lib.clusten_scatter_rows_workspace_bytes(shape, code)
    ws = _workspace(ws_bytes, device)
    with torch.cuda.device(device):
        _check(lib.clusten_scatter_rows(_ptr(p), _ptr(x), _strides(x), _ptr(idx), _ptr(pair_lists), _ptr(y), _ptr(ws),
                                        ws_bytes, shape, code, _stream(device)), "clusten_scatter_rows")
    return y


def qk_backward(d_attn: torch.Tensor, query: torch.Tensor, key: torch.Tensor, nbhd_idx: torch.Tensor, pairs=None):
    """(d_query, d_key), both contiguous (b,h,n,c).  `pairs`: the block `cluster_pairs(nbhd_idx)` of a caller that keeps
    it across the layers of a stage; the call then runs as its two halves (same kernels, same results) and skips the
    rebuild of the pair lists."""
    if pairs is not None:
        if tuple(d_attn.shape) != tuple(query.shape[:3]) + (nbhd_idx.shape[2],) or d_attn.dtype != query.dtype:
            raise RuntimeError("d_attn must be (b,h,n,m) with the dtype of query")
        return av_forward(d_attn, key, nbhd_idx), scatter_rows(d_attn, query, nbhd_idx, pairs)
    lib = load()
    device, code, idx, shape = _attn_problem(query, key, nbhd_idx, ("query", "key"))
    _require_cuda("d_attn", d_attn, device)
    if tuple(d_attn.shape) != (shape.B, shape.H, shape.N, shape.M) or d_attn.dtype != query.dtype:
        raise RuntimeError("d_attn must be (b,h,n,m) with the dtype of query")
    d_attn = d_attn.contiguous()
    query, key = _rows(query), _rows(key)
    d_query = torch.empty((shape.B, shape.H, shape.N, shape.C), dtype=query.dtype, device=device)
    d_key = torch.empty_like(d_query)
    if d_query.numel() == 0 or shape.M == 0:
        return d_query.zero_(), d_key.zero_()
    ws_bytes = lib.clusten_qk_backward_workspace_bytes(shape, code)
    ws = _workspace(ws_bytes, device)
    with torch.cuda.device(device):
        _check(lib.clusten_qk_backward(_ptr(d_attn), _ptr(query), _strides(query), _ptr(key), _strides(key), _ptr(idx),
                                       _ptr(d_query), _ptr(d_key), _ptr(ws), ws_bytes, shape, code, _stream(device)),
               "clusten_qk_backward")
    return d_query, d_key


STATIC_SCRATCH_BYTES = 32 << 20   # CLUSTEN_STATIC_SCRATCH_BYTES of include/clusten_hip.h


def qk_backward_static(d_attn: torch.Tensor, query: torch.Tensor, key: torch.Tensor, nbhd_idx: torch.Tensor,
                       d_query: torch.Tensor, d_key: torch.Tensor) -> None:
    """`clusten_qk_backward_static`: the QK backward into the caller's contiguous (b,h,n,c) tensors d_query and d_key,
    through the entry point that allocates nothing (the fp32 sums of 16-bit data live in a fixed device array of
    the library: at most STATIC_SCRATCH_BYTES / 4 elements of d_key, else RuntimeError).  Nothing is allocated here
    either; calls that overlap in time on one GPU race on that array."""
    lib = load()
    device, code, idx, shape = _attn_problem(query, key, nbhd_idx, ("query", "key"))
    for name, t in (("d_attn", d_attn), ("d_query", d_query), ("d_key", d_key)):
        _require_cuda(name, t, device)
    if tuple(d_attn.shape) != (shape.B, shape.H, shape.N, shape.M) or d_attn.dtype != query.dtype:
        raise RuntimeError("d_attn must be (b,h,n,m) with the dtype of query")
    for name, t in (("d_query", d_query), ("d_key", d_key)):
        if t.shape != query.shape or t.dtype != query.dtype or not t.is_contiguous():
            raise RuntimeError("%s must be a contiguous (b,h,n,c) tensor with the dtype of query" % name)
    if not d_attn.is_contiguous() or _rows(query) is not query or _rows(key) is not key or idx is not nbhd_idx:
        raise RuntimeError("qk_backward_static copies nothing: d_attn and nbhd_idx contiguous, rows with channel stride 1")
    if d_query.numel() == 0 or shape.M == 0:
        raise RuntimeError("qk_backward_static: empty problem")
    with torch.cuda.device(device):
        _check(lib.clusten_qk_backward_static(_ptr(d_attn), _ptr(query), _strides(query), _ptr(key), _strides(key),
                                              _ptr(idx), _ptr(d_query), _ptr(d_key), shape, code, _stream(device)),
               "clusten_qk_backward_static")


def av_forward(attn: torch.Tensor, v: torch.Tensor, nbhd_idx: torch.Tensor, token_major: bool = False,
               _entry=None) -> torch.Tensor:
    """feat (b,h,n,c) = attn · v[nbhd_idx].  With token_major=True the result is a (b,h,n,c) view of
    (b,n,h,c) storage, so that `.permute(0,2,1,3).reshape(b,n,h*c)` needs no copy.  `_entry`: see qk_forward."""
    lib = load()
    _require_cuda("attn", attn)
    device = attn.device
    _require_cuda("v", v, device)
    if attn.dim() != 4 or v.dim() != 4 or nbhd_idx.dim() != 3:
        raise RuntimeError("attn must be (b,h,n,m), v (b,h,n,c) and nbhd_idx (b,n,m)")
    if attn.shape[:3] != v.shape[:3] or attn.dtype != v.dtype:
        raise RuntimeError("attn %s and v %s must agree in (b,h,n) and dtype" % (tuple(attn.shape), tuple(v.shape)))
    B, H, N, C = v.shape
    idx = _idx(nbhd_idx, (B, N), device)
    if idx.shape[2] != attn.shape[3]:
        raise RuntimeError("attn has %d slots per token, nbhd_idx %d" % (attn.shape[3], idx.shape[2]))
    shape = AttnShape(B, H, N, C, idx.shape[2])
    code = _dtype_code(attn, "attn")
    attn, v = attn.contiguous(), _rows(v)
    if token_major:
        feat = torch.empty((B, N, H, C), dtype=attn.dtype, device=device).permute(0, 2, 1, 3)
    else:
        feat = torch.empty((B, H, N, C), dtype=attn.dtype, device=device)
    if feat.numel() == 0:
        return feat
    if shape.M == 0:
        return feat.zero_()
    with torch.cuda.device(device):
        fn = _entry or lib.clusten_av_forward
        _check(fn(_ptr(attn), _ptr(v), _strides(v), _ptr(idx), _ptr(feat), _strides(feat), shape, code, _stream(device)),
               "clusten_av_forward")
    return feat


def mixed_supported(first: torch.Tensor, second: torch.Tensor, attention: bool = False) -> bool:
    """True for the operand pair mixed precision hands AV and WF: an fp32 first operand (attention weights, merge
    weights) and an fp16 / bf16 second one (values, features), both on the GPU.  For attention (`attention=True`) lists
    of more than 64 slots are left to the cast-first path: they have kernels of their own (long runs), and only the
    same kernel gives the same bits."""
    return (first.is_cuda and second.is_cuda and first.dtype == torch.float32
            and second.dtype in (torch.float16, torch.bfloat16) and (not attention or first.shape[-1] <= 64))


def av_forward_mixed(attn: torch.Tensor, v: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """feat (b,h,n,c) fp32 = attn (fp32) · v[nbhd_idx] with v fp16 / bf16 read in place: bit-identical to
    `av_forward(attn, v.float(), nbhd_idx)` (the cast clusten/clusten.py:52-53 makes) without the copy."""
    lib = load()
    if not mixed_supported(attn, v, attention=True):
        raise RuntimeError("av_forward_mixed takes fp32 attn of at most 64 slots and fp16 / bf16 v on the GPU")
    device = attn.device
    _require_cuda("v", v, device)
    if attn.dim() != 4 or v.dim() != 4 or nbhd_idx.dim() != 3 or attn.shape[:3] != v.shape[:3]:
        raise RuntimeError("attn must be (b,h,n,m), v (b,h,n,c) and nbhd_idx (b,n,m)")
    B, H, N, C = v.shape
    idx = _idx(nbhd_idx, (B, N), device)
    if idx.shape[2] != attn.shape[3]:
        raise RuntimeError("attn has %d slots per token, nbhd_idx %d" % (attn.shape[3], idx.shape[2]))
    shape = AttnShape(B, H, N, C, idx.shape[2])
    attn, v = attn.contiguous(), _rows(v)
    feat = torch.empty((B, H, N, C), dtype=torch.float32, device=device)
    if feat.numel() == 0:
        return feat
    if shape.M == 0:
        return feat.zero_()
    with torch.cuda.device(device):
        _check(lib.clusten_av_forward_mixed(_ptr(attn), _ptr(v), _strides(v), _DTYPE_CODE[v.dtype], _ptr(idx), _ptr(feat),
                                            _strides(feat), shape, _stream(device)), "clusten_av_forward_mixed")
    return feat


def av_backward(d_feat: torch.Tensor, attn: torch.Tensor, v: torch.Tensor, nbhd_idx: torch.Tensor, pairs=None):
    """(d_attn (b,h,n,m), d_v (b,h,n,c)), both contiguous.  `pairs`: see qk_backward."""
    if pairs is not None:
        if tuple(attn.shape) != tuple(v.shape[:3]) + (nbhd_idx.shape[2],) or attn.dtype != v.dtype:
            raise RuntimeError("attn must be (b,h,n,m) with the dtype of v")
        return qk_forward(d_feat, v, nbhd_idx), scatter_rows(attn, d_feat, nbhd_idx, pairs)
    lib = load()
    device, code, idx, shape = _attn_problem(d_feat, v, nbhd_idx, ("d_feat", "v"))
    _require_cuda("attn", attn, device)
    if tuple(attn.shape) != (shape.B, shape.H, shape.N, shape.M) or attn.dtype != v.dtype:
        raise RuntimeError("attn must be (b,h,n,m) with the dtype of v")
    attn = attn.contiguous()
    d_feat, v = _rows(d_feat), _rows(v)
    d_attn = torch.empty((shape.B, shape.H, shape.N, shape.M), dtype=attn.dtype, device=device)
    d_v = torch.empty((shape.B, shape.H, shape.N, shape.C), dtype=attn.dtype, device=device)
    if d_v.numel() == 0 or shape.M == 0:
        return d_attn.zero_(), d_v.zero_()
    ws_bytes = lib.clusten_av_backward_workspace_bytes(shape, code)
    ws = _workspace(ws_bytes, device)
    with torch.cuda.device(device):
        _check(lib.clusten_av_backward(_ptr(d_feat), _strides(d_feat), _ptr(attn), _ptr(v), _strides(v), _ptr(idx),
                                       _ptr(d_attn), _ptr(d_v), _ptr(ws), ws_bytes, shape, code, _stream(device)),
               "clusten_av_backward")
    return d_attn, d_v


def _wf_problem(weights: torch.Tensor, feat: torch.Tensor, nbhd_idx: torch.Tensor):
    _require_cuda("weights", weights)
    device = weights.device
    _require_cuda("feat", feat, device)
    if weights.dim() != 4 or feat.dim() != 3 or nbhd_idx.dim() != 3:
        raise RuntimeError("weights must be (b,n_,m,ic), feat (b,n,c) and nbhd_idx (b,n_,m)")
    if weights.shape[0] != feat.shape[0] or weights.dtype != feat.dtype:
        raise RuntimeError("weights and feat must agree in batch size and dtype")
    B, Nout, M, IC = weights.shape
    N, C = feat.shape[1], feat.shape[2]
    idx = _idx(nbhd_idx, (B, Nout), device, n_rows=N)
    if idx.shape[2] != M:
        raise RuntimeError("weights has %d slots per token, nbhd_idx %d" % (M, idx.shape[2]))
    return device, _dtype_code(weights, "weights"), idx, WfShape(B, N, Nout, C, M, IC)


def wf_forward(weights: torch.Tensor, feat: torch.Tensor, nbhd_idx: torch.Tensor, _entry=None) -> torch.Tensor:
    """feat_new (b,n_,ic,c) = weightsᵀ · feat[nbhd_idx].  `_entry`: see qk_forward."""
    lib = load()
    device, code, idx, shape = _wf_problem(weights, feat, nbhd_idx)
    weights, feat = weights.contiguous(), feat.contiguous()
    out = torch.empty((shape.B, shape.Nout, shape.IC, shape.C), dtype=weights.dtype, device=device)
    if out.numel() == 0:
        return out
    if shape.M == 0 or shape.N == 0:
        return out.zero_()
    with torch.cuda.device(device):
        fn = _entry or lib.clusten_wf_forward
        _check(fn(_ptr(weights), _ptr(feat), _ptr(idx), _ptr(out), shape, code, _stream(device)), "clusten_wf_forward")
    return out


def wf_forward_mixed(weights: torch.Tensor, feat: torch.Tensor, nbhd_idx: torch.Tensor) -> torch.Tensor:
    """feat_new (b,n_,ic,c) fp32 = weights (fp32)ᵀ · feat[nbhd_idx] with feat fp16 / bf16 read in place: bit-identical to
    `wf_forward(weights, feat.float(), nbhd_idx)` (the cast clusten/clusten.py:78-79 makes) without the copy."""
    lib = load()
    if not mixed_supported(weights, feat):
        raise RuntimeError("wf_forward_mixed takes fp32 weights and fp16 / bf16 feat on the GPU")
    device = weights.device
    _require_cuda("feat", feat, device)
    if weights.dim() != 4 or feat.dim() != 3 or nbhd_idx.dim() != 3 or weights.shape[0] != feat.shape[0]:
        raise RuntimeError("weights must be (b,n_,m,ic), feat (b,n,c) and nbhd_idx (b,n_,m)")
    B, Nout, M, IC = weights.shape
    N, C = feat.shape[1], feat.shape[2]
    idx = _idx(nbhd_idx, (B, Nout), device, n_rows=N)
    if idx.shape[2] != M:
        raise RuntimeError("weights has %d slots per token, nbhd_idx %d" % (M, idx.shape[2]))
    shape = WfShape(B, N, Nout, C, M, IC)
    weights, feat = weights.contiguous(), feat.contiguous()
    out = torch.empty((B, Nout, IC, C), dtype=torch.float32, device=device)
    if out.numel() == 0:
        return out
    if M == 0 or N == 0:
        return out.zero_()
    with torch.cuda.device(device):
        _check(lib.clusten_wf_forward_mixed(_ptr(weights), _ptr(feat), _DTYPE_CODE[feat.dtype], _ptr(idx), _ptr(out), shape,
                                            _stream(device)), "clusten_wf_forward_mixed")
    return out


def wf_backward(d_feat_new: torch.Tensor, weights: torch.Tensor, feat: torch.Tensor, nbhd_idx: torch.Tensor):
    """(d_weights (b,n_,m,ic), d_feat (b,n,c)), both contiguous."""
    lib = load()
    device, code, idx, shape = _wf_problem(weights, feat, nbhd_idx)
    _require_cuda("d_feat_new", d_feat_new, device)
    if tuple(d_feat_new.shape) != (shape.B, shape.Nout, shape.IC, shape.C) or d_feat_new.dtype != weights.dtype:
        raise RuntimeError("d_feat_new must be (b,n_,ic,c) with the dtype of weights")
    d_feat_new, weights, feat = d_feat_new.contiguous(), weights.contiguous(), feat.contiguous()
    d_weights = torch.empty_like(weights)
    d_feat = torch.empty_like(feat)
    if d_weights.numel() == 0 or d_feat.numel() == 0:
        return d_weights.zero_(), d_feat.zero_()
    ws_bytes = lib.clusten_wf_backward_workspace_bytes(shape, code)
    ws = _workspace(ws_bytes, device)
    with torch.cuda.device(device):
        _check(lib.clusten_wf_backward(_ptr(d_feat_new), _ptr(weights), _ptr(feat), _ptr(idx), _ptr(d_weights),
                                       _ptr(d_feat), _ptr(ws), ws_bytes, shape, code, _stream(device)),
               "clusten_wf_backward")
    return d_weights, d_feat


def wf_backward_by_cluster(d_feat_new: torch.Tensor, weights: torch.Tensor, feat: torch.Tensor, nbhd_idx: torch.Tensor,
                           pair_lists: torch.Tensor, d_feat=None):
    """(d_weights, d_feat) of the WF operator through `clusten_wf_backward_by_cluster`: the feature gradient as a gather
    over `pair_lists` = `cluster_pairs(nbhd_idx, n)`.  When the block's flag says the lists are not whole clusters
    `d_feat` (new memory unless given) is left untouched."""
    lib = load()
    device, code, idx, shape = _wf_problem(weights, feat, nbhd_idx)
    _require_cuda("d_feat_new", d_feat_new, device)
    if tuple(d_feat_new.shape) != (shape.B, shape.Nout, shape.IC, shape.C) or d_feat_new.dtype != weights.dtype:
        raise RuntimeError("d_feat_new must be (b,n_,ic,c) with the dtype of weights")
    if pair_lists is None or pair_lists.numel() != lib.clusten_cluster_pairs_bytes(shape.B, shape.Nout, shape.M, shape.N):
        raise RuntimeError("wf_backward_by_cluster: pair lists of these lists (cluster_pairs(nbhd_idx, n))")
    d_feat_new, weights, feat = d_feat_new.contiguous(), weights.contiguous(), feat.contiguous()
    d_weights = torch.empty_like(weights)
    d_feat = torch.empty_like(feat) if d_feat is None else d_feat
    with torch.cuda.device(device):
        _check(lib.clusten_wf_backward_by_cluster(_ptr(d_feat_new), _ptr(weights), _ptr(feat), _ptr(idx), _ptr(pair_lists),
                                                  _ptr(d_weights), _ptr(d_feat), shape, code, _stream(device)),
               "clusten_wf_backward_by_cluster")
    return d_weights, d_feat


def clusters_supported(a: torch.Tensor, nnc: int, cluster_size: int = 8) -> bool:
    """True when the cluster-number entry points take this case: head dim 16/32/64, at most 8 clusters per token, of 8
    rows or of the size `cluster_size_for` gives their slot count (24 for 144 slots; rows of at least 64 bytes there)."""
    if not (a.is_cuda and a.dtype in (torch.float32, torch.float16, torch.bfloat16) and a.shape[3] in (16, 32, 64)
            and 1 <= nnc <= 8):
        return False
    if cluster_size == 8:
        return True
    return cluster_size_for(cluster_size * nnc) == cluster_size and a.shape[3] * a.element_size() >= 64


def _cluster_idx(cluster_idx: torch.Tensor, shape, device) -> torch.Tensor:
    _require_cuda("cluster_idx", cluster_idx, device)
    if cluster_idx.dtype != torch.int32 or cluster_idx.dim() != 3 or tuple(cluster_idx.shape[:2]) != tuple(shape):
        raise RuntimeError("cluster_idx must be int32 of shape (B,N,clusters per token)")
    return cluster_idx.contiguous()


def cluster_size_for(m: int) -> int:
    """The cluster size the cluster-number forms read a list of m slots in (0: no such form)."""
    return int(load().clusten_cluster_size_for(int(m)))


def _clusters_slots(cidx: torch.Tensor, cluster_size: int) -> int:
    m = cluster_size * cidx.shape[2]
    if cluster_size_for(m) != cluster_size:
        raise RuntimeError("lists of %d clusters of %d rows are not taken by the cluster-number forms" %
                           (cidx.shape[2], cluster_size))
    return m


def qk_forward_clusters(query: torch.Tensor, key: torch.Tensor, cluster_idx: torch.Tensor,
                        cluster_size: int = 8) -> torch.Tensor:
    """qk_forward on nbhd_idx[b,i,L*r+t] = L*cluster_idx[b,i,r]+t (0 where that is >= N), without building it;
    L = `cluster_size` (8, or the cluster size `cluster_size_for(L * clusters per token)` names: 24 for 144 slots)."""
    lib = load()
    _require_cuda("query", query)
    device = query.device
    _require_cuda("key", key, device)
    if query.shape != key.shape or query.dim() != 4 or query.dtype != key.dtype:
        raise RuntimeError("query and key must be (B,H,N,C) tensors of one dtype")
    B, H, N, C = query.shape
    cidx = _cluster_idx(cluster_idx, (B, N), device)
    shape = AttnShape(B, H, N, C, _clusters_slots(cidx, cluster_size))
    query, key = _rows(query), _rows(key)
    attn = torch.empty((B, H, N, shape.M), dtype=query.dtype, device=device)
    if attn.numel() == 0:
        return attn
    with torch.cuda.device(device):
        _check(lib.clusten_qk_forward_clusters(_ptr(query), _strides(query), _ptr(key), _strides(key), _ptr(cidx),
                                               _ptr(attn), shape, _dtype_code(query, "query"), _stream(device)),
               "clusten_qk_forward_clusters")
    return attn


def av_forward_clusters(attn: torch.Tensor, v: torch.Tensor, cluster_idx: torch.Tensor,
                        cluster_size: int = 8) -> torch.Tensor:
    """av_forward on the lists qk_forward_clusters describes; v is cast to attn's dtype like the AV Function does."""
    lib = load()
    _require_cuda("attn", attn)
    device = attn.device
    _require_cuda("v", v, device)
    B, H, N, C = v.shape
    cidx = _cluster_idx(cluster_idx, (B, N), device)
    m = _clusters_slots(cidx, cluster_size)
    if tuple(attn.shape) != (B, H, N, m):
        raise RuntimeError("attn must be (B,H,N,cluster size * clusters per token)")
    shape = AttnShape(B, H, N, C, m)
    attn, v = attn.contiguous(), _rows(v.to(attn.dtype))
    feat = torch.empty((B, H, N, C), dtype=attn.dtype, device=device)
    if feat.numel() == 0:
        return feat
    with torch.cuda.device(device):
        _check(lib.clusten_av_forward_clusters(_ptr(attn), _ptr(v), _strides(v), _ptr(cidx), _ptr(feat), _strides(feat),
                                               shape, _dtype_code(attn, "attn"), _stream(device)),
               "clusten_av_forward_clusters")
    return feat


def attn_softmax_supported(attn: torch.Tensor, m: int) -> bool:
    """True when `attn_softmax` takes this case: a CUDA tensor of a 16/32-bit float type, M <= 256, M % 4 == 0."""
    return attn.is_cuda and attn.dtype in (torch.float32, torch.float16, torch.bfloat16) and m <= 256 and m % 4 == 0


def attn_softmax(attn: torch.Tensor, bias_table: torch.Tensor, pe_idx: torch.Tensor, mask, blank_logit=None,
                 query=None, blank_key=None):
    """softmax over M neighbours and one blank token of attn + bias_table[pe_idx] - 100 * (1 - mask) | blank logit.

    attn (B,H,N,M); bias_table (rows,H), cast to attn's dtype; pe_idx (B,N,M) int64; mask (B,N,M) int64 or None.
    The blank token's logit is either given, blank_logit (B,H,N) or (B,H,N,1), or computed in the same pass as
    (query * blank_key).sum(-1) from query (B,H,N,C) (any strides, channel stride 1, attn's dtype) and blank_key (H,C).
    Returns (probs (B,H,N,M) fp32, blank_prob (B,H,N,1) fp32).
    No autograd: for inference.  The fused form of models/aff_transformer.py:122-147.
    """
    lib = load()
    _require_cuda("attn", attn)
    device = attn.device
    for name, t in (("bias_table", bias_table), ("pe_idx", pe_idx)):
        _require_cuda(name, t, device)
    b, h, n, m = attn.shape
    if blank_logit is None and (query is None or blank_key is None):
        raise RuntimeError("attn_softmax needs blank_logit, or query and blank_key")
    if pe_idx.shape != (b, n, m) or pe_idx.dtype != torch.int64:
        raise RuntimeError("pe_idx must be int64 of shape (B,N,M)")
    if bias_table.dim() != 2 or bias_table.shape[1] != h:
        raise RuntimeError("bias_table must have shape (rows, H)")
    code = _dtype_code(attn, "attn")
    attn = attn.contiguous()
    bias_table = bias_table.to(attn.dtype).contiguous()
    pe_idx = pe_idx.contiguous()
    if mask is not None:
        _require_cuda("mask", mask, device)
        if mask.shape != (b, n, m):
            raise RuntimeError("mask must have shape (B,N,M)")
        mask = mask.to(torch.int64).contiguous()
    qs, c = Strides(0, 0, 0), 1
    if blank_logit is not None:
        _require_cuda("blank_logit", blank_logit, device)
        blank_logit = blank_logit.reshape(b, h, n).float().contiguous()
        query = blank_key = None
    else:
        _require_cuda("query", query, device)
        _require_cuda("blank_key", blank_key, device)
        c = query.shape[3]
        if query.shape[:3] != (b, h, n) or blank_key.numel() != h * c:
            raise RuntimeError("query must be (B,H,N,C) and blank_key (H,C)")
        query = _rows(query.to(attn.dtype))
        qs = _strides(query)
        blank_key = blank_key.detach().reshape(h, c).float().contiguous()
    probs = torch.empty(b, h, n, m, dtype=torch.float32, device=device)
    blank_prob = torch.empty(b, h, n, 1, dtype=torch.float32, device=device)
    if probs.numel() == 0:
        return probs, blank_prob
    shape = AttnShape(b, h, n, c, m)
    with torch.cuda.device(device):
        _check(lib.clusten_attn_softmax_forward(_ptr(attn), _ptr(bias_table), _ptr(pe_idx), _ptr(mask),
                                                _ptr(blank_logit), _ptr(query), qs, _ptr(blank_key), _ptr(probs),
                                                _ptr(blank_prob), shape, code, _stream(device)),
               "clusten_attn_softmax_forward")
    return probs, blank_prob


def attn_softmax_backward(probs: torch.Tensor, blank_prob: torch.Tensor, d_probs: torch.Tensor,
                          d_blank_prob: torch.Tensor, logit_dtype):
    """(d_logit (B,H,N,M) of logit_dtype, d_blank_logit (B,H,N,1) fp32): the backward of `attn_softmax` with respect
    to the attention logits (= the gradient of the gathered bias too) and to the blank token's logit."""
    lib = load()
    _require_cuda("probs", probs)
    device = probs.device
    if probs.dim() != 4 or probs.dtype != torch.float32 or logit_dtype not in _DTYPE_CODES:
        raise RuntimeError("probs must be fp32 (B,H,N,M); logits fp32, fp16 or bf16")
    b, h, n, m = probs.shape
    if m > 256 or m % 4:
        raise RuntimeError("attn_softmax_backward: M <= 256, M % 4 == 0")
    probs = probs.contiguous()
    d_probs = d_probs.to(torch.float32).expand_as(probs).contiguous()
    blank_prob = blank_prob.reshape(b, h, n).float().contiguous()
    d_blank_prob = d_blank_prob.to(torch.float32).expand(b, h, n, 1).reshape(b, h, n).contiguous()
    d_logit = torch.empty(b, h, n, m, dtype=logit_dtype, device=device)
    d_blank_logit = torch.empty(b, h, n, 1, dtype=torch.float32, device=device)
    if d_logit.numel() == 0:
        return d_logit, d_blank_logit
    with torch.cuda.device(device):
        _check(lib.clusten_attn_softmax_backward(_ptr(probs), _ptr(blank_prob), _ptr(d_probs), _ptr(d_blank_prob),
                                                 _ptr(d_logit), _ptr(d_blank_logit), b * h * n, m,
                                                 _DTYPE_CODES[logit_dtype], _stream(device)),
               "clusten_attn_softmax_backward")
    return d_logit, d_blank_logit


def cluster_attention_supported(query: torch.Tensor, nnc: int, cluster_size: int = 8) -> bool:
    """True when `cluster_attention` takes this case: CUDA queries of head dim 32, six clusters per token; clusters of 8
    tokens (fp16 / bf16 / fp32) or of 24 tokens (fp16 / bf16)."""
    types = {8: (torch.float16, torch.bfloat16, torch.float32), 24: (torch.float16, torch.bfloat16)}.get(cluster_size, ())
    return query.is_cuda and query.dtype in types and query.dim() == 4 and query.shape[3] == 32 and nnc == 6


def cluster_attention_plan(cluster_idx: torch.Tensor, pe_idx: torch.Tensor, mask) -> torch.Tensor:
    """What `cluster_attention` works out from its three index tensors before its first head, for every tile of 8
    tokens: a uint8 tensor to hand to every call that uses these lists (`plan=`), e.g. all layers of a stage.
    cluster_idx (B,N,6) int32, pe_idx (B,N,M) int64, mask (B,N,M) of 0/1 or None — B = 1 for lists shared by every
    image; M = 48 (clusters of 8 tokens) or 144 (clusters of 24)."""
    lib = load()
    _require_cuda("cluster_idx", cluster_idx)
    device = cluster_idx.device
    _require_cuda("pe_idx", pe_idx, device)
    if cluster_idx.dim() != 3 or cluster_idx.shape[2] != 6:
        raise RuntimeError("cluster_idx must be (B,N,6)")
    lb, n = cluster_idx.shape[:2]
    cidx = _cluster_idx(cluster_idx, (lb, n), device)
    m = pe_idx.shape[2] if pe_idx.dim() == 3 else 0
    if pe_idx.shape != (lb, n, m) or m not in (48, 144) or pe_idx.dtype != torch.int64:
        raise RuntimeError("pe_idx must be int64 of shape (B,N,48) or (B,N,144), B and N like cluster_idx")
    pe_idx = pe_idx.contiguous()
    if mask is not None:
        _require_cuda("mask", mask, device)
        if mask.shape != (lb, n, m):
            raise RuntimeError("mask must have the shape of pe_idx")
        mask = mask.to(torch.int64).contiguous()
    nbytes = lib.clusten_cluster_attention_plan_bytes(lb, n, m)
    plan = torch.empty(nbytes, dtype=torch.uint8, device=device)
    if nbytes:
        with torch.cuda.device(device):
            _check(lib.clusten_cluster_attention_plan(_ptr(cidx), _ptr(pe_idx), _ptr(mask), _ptr(plan), nbytes, lb, n, m,
                                                      _stream(device)), "clusten_cluster_attention_plan")
    return plan


def cluster_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, cluster_idx: torch.Tensor,
                      bias_table: torch.Tensor, pe_idx: torch.Tensor, mask, blank_key: torch.Tensor,
                      blank_value: torch.Tensor, scale: float = 1.0, plan=None, return_lse: bool = False):
    """Local attention over the members of each token's clusters plus one blank token, in one kernel.

    query, key, value (B,H,N,32) fp16 / bf16 / fp32 (any strides, channel stride 1); cluster_idx (B,N,6) int32;
    bias_table (rows,H); pe_idx (B,N,M) int64; mask (B,N,M) of 0/1 or None; blank_key, blank_value (H*32,).
    M = 48: clusters of 8 tokens (row(i,j) = 8 * cluster + j % 8); M = 144, fp16 / bf16 only: clusters of 24.
    cluster_idx, pe_idx and mask may all have a leading 1 instead of B: one set of lists for every image.
    Returns softmax(scale * q.k + bias - 100 * (1 - mask) | scale * q.blank_key) applied to the gathered values and
    the blank value, as a (B,N,H*32) tensor of query's dtype (heads side by side, the layout the output
    projection takes).  No autograd: for inference.  The fused form of models/aff_transformer.py:120-155.
    `plan`: what `cluster_attention_plan` made of the same three index tensors; they are then not read (and may be
    None), the result is the same.  `return_lse` (needs a plan): also return the fp32 (B,H,N) logarithms of the
    softmax denominators, what `cluster_attention_backward` recomputes the probabilities from.
    """
    lib = load()
    _require_cuda("query", query)
    device = query.device
    for name, t in (("key", key), ("value", value), ("bias_table", bias_table), ("pe_idx", pe_idx),
                    ("blank_key", blank_key), ("blank_value", blank_value)):
        if not (plan is not None and t is None):
            _require_cuda(name, t, device)
    if query.dim() != 4 or key.shape != query.shape or value.shape != query.shape:
        raise RuntimeError("query, key and value must be (B,H,N,C) tensors of one shape")
    b, h, n, c = query.shape
    if plan is not None:
        _require_cuda("plan", plan, device)
        # the plan's size tells the batch elements of its lists (b, or 1 for shared lists) and their length
        fits = [(lb_, m_) for m_ in (48, 144) for lb_ in (b, 1)
                if plan.numel() == lib.clusten_cluster_attention_plan_bytes(lb_, n, m_)]
        if plan.dtype != torch.uint8 or not fits:
            raise RuntimeError("plan does not belong to lists of this shape")
        lb, m = fits[0]
        shared = b != 1 and lb == 1
        cidx = pe_idx = mask = None
    else:
        shared = b != 1 and cluster_idx.dim() == 3 and cluster_idx.shape[0] == 1
        lb = 1 if shared else b
        cidx = _cluster_idx(cluster_idx, (lb, n), device)
        m = pe_idx.shape[2] if pe_idx.dim() == 3 else 0
        if cidx.shape[2] != 6 or m not in (48, 144):
            raise RuntimeError("cluster_idx must be (B,N,6) and pe_idx (B,N,48) or (B,N,144)")
        if pe_idx.shape != (lb, n, m) or pe_idx.dtype != torch.int64:
            raise RuntimeError("pe_idx must be int64 of shape (B,N,M), or (1,N,M) like cluster_idx")
        pe_idx = pe_idx.contiguous()
    if bias_table.dim() != 2 or bias_table.shape[1] != h:
        raise RuntimeError("bias_table must have shape (rows, H)")
    if blank_key.numel() != h * c or blank_value.numel() != h * c:
        raise RuntimeError("blank_key and blank_value must have H*C elements")
    code = _dtype_code(query, "query")
    dtype = query.dtype
    query, key, value = _rows(query), _rows(key.to(dtype)), _rows(value.to(dtype))
    bias_table = bias_table.detach().to(dtype).contiguous()
    if mask is not None:
        _require_cuda("mask", mask, device)
        if mask.shape != (lb, n, m):
            raise RuntimeError("mask must have shape (B,N,M), or (1,N,M) like cluster_idx")
        mask = mask.to(torch.int64).contiguous()
    blank_key = blank_key.detach().reshape(h, c).float().contiguous()
    blank_value = blank_value.detach().reshape(h, c).float().contiguous()
    out = torch.empty(b, n, h, c, dtype=dtype, device=device)
    if out.numel() == 0:
        flat = out.reshape(b, n, h * c)
        return (flat, torch.empty(b, h, n, dtype=torch.float32, device=device)) if return_lse else flat
    out_view = out.permute(0, 2, 1, 3)                                   # (B,H,N,C) view of the (B,N,H,C) memory
    shape = AttnShape(b, h, n, c, m)
    if return_lse:
        if plan is None:
            raise RuntimeError("return_lse needs a plan")
        lse = torch.empty(b, h, n, dtype=torch.float32, device=device)
        with torch.cuda.device(device):
            _check(lib.clusten_cluster_attention_forward_train(_ptr(query), _strides(query), _ptr(key), _strides(key),
                                                               _ptr(value), _strides(value), _ptr(plan), _ptr(bias_table),
                                                               int(shared), _ptr(blank_key), _ptr(blank_value), _ptr(out),
                                                               _strides(out_view), _ptr(lse), ctypes.c_float(scale), shape,
                                                               code, _stream(device)),
                   "clusten_cluster_attention_forward_train")
        return out.reshape(b, n, h * c), lse
    if plan is not None:
        with torch.cuda.device(device):
            _check(lib.clusten_cluster_attention_forward_planned(_ptr(query), _strides(query), _ptr(key), _strides(key),
                                                                 _ptr(value), _strides(value), _ptr(plan), _ptr(bias_table),
                                                                 int(shared), _ptr(blank_key), _ptr(blank_value), _ptr(out),
                                                                 _strides(out_view), ctypes.c_float(scale), shape, code,
                                                                 _stream(device)),
                   "clusten_cluster_attention_forward_planned")
        return out.reshape(b, n, h * c)
    with torch.cuda.device(device):
        _check(lib.clusten_cluster_attention_forward(_ptr(query), _strides(query), _ptr(key), _strides(key),
                                                     _ptr(value), _strides(value), _ptr(cidx), _ptr(bias_table),
                                                     _ptr(pe_idx), _ptr(mask), int(shared), _ptr(blank_key),
                                                     _ptr(blank_value),
                                                     _ptr(out), _strides(out_view), ctypes.c_float(scale), shape, code,
                                                     _stream(device)),
               "clusten_cluster_attention_forward")
    return out.reshape(b, n, h * c)


def cluster_attention_backward_supported(query: torch.Tensor, nnc: int) -> bool:
    """True when `cluster_attention_backward` takes this case: CUDA fp32 / fp16 / bf16 queries of head dim 32, six
    clusters per token."""
    return (query.is_cuda and query.dtype in (torch.float32, torch.float16, torch.bfloat16) and query.dim() == 4
            and query.shape[3] == 32 and nnc == 6)


def cluster_attention_backward(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, d_out: torch.Tensor,
                               out: torch.Tensor, lse: torch.Tensor, plan: torch.Tensor, bias_table: torch.Tensor,
                               blank_key: torch.Tensor, blank_value: torch.Tensor, scale: float = 1.0):
    """The query-side half of the backward of `cluster_attention(..., plan=plan, return_lse=True)` in one kernel.

    query, key, value (B,H,N,32) fp32 / fp16 / bf16 as in the forward; out (B,N,H*32) its result, d_out the gradient of it,
    lse (B,H,N) fp32 from the forward.  Returns (d_query, probs, d_logit, blank_prob, d_blank_logit): d_query a
    (B,H,N,32) view of (B,N,H,32) memory, probs and d_logit (B,H,N,48) of query's dtype, blank_prob and d_blank_logit
    fp32 (B,H,N).  The other gradients are sums of these: d_value = scatter_rows_by_cluster(probs, d_out),
    d_key = scale * scatter_rows_by_cluster(d_logit, query), d_bias_table = bias_table_grad(d_logit, ...),
    d_blank_key = scale * sum d_blank_logit * query, d_blank_value = sum blank_prob * d_out."""
    lib = load()
    _require_cuda("query", query)
    device = query.device
    for name, t in (("key", key), ("value", value), ("d_out", d_out), ("out", out), ("lse", lse), ("plan", plan),
                    ("bias_table", bias_table), ("blank_key", blank_key), ("blank_value", blank_value)):
        _require_cuda(name, t, device)
    if query.dim() != 4 or key.shape != query.shape or value.shape != query.shape:
        raise RuntimeError("query, key and value must be (B,H,N,C) tensors of one shape")
    b, h, n, c = query.shape
    m = 48
    if tuple(out.shape) != (b, n, h * c) or tuple(d_out.shape) != (b, n, h * c):
        raise RuntimeError("out and d_out must be (B,N,H*C)")
    if tuple(lse.shape) != (b, h, n) or lse.dtype != torch.float32:
        raise RuntimeError("lse must be fp32 (B,H,N)")
    lb = b if plan.numel() == lib.clusten_cluster_attention_plan_bytes(b, n, 48) else 1
    if plan.dtype != torch.uint8 or plan.numel() != lib.clusten_cluster_attention_plan_bytes(lb, n, 48):
        raise RuntimeError("plan does not belong to lists of this shape")
    shared = b != 1 and lb == 1
    code = _dtype_code(query, "query")
    dtype = query.dtype
    query, key, value = _rows(query), _rows(key.to(dtype)), _rows(value.to(dtype))
    out_view = out.to(dtype).contiguous().view(b, n, h, c).permute(0, 2, 1, 3)
    g_view = d_out.to(dtype).contiguous().view(b, n, h, c).permute(0, 2, 1, 3)
    bias_table = bias_table.detach().to(dtype).contiguous()
    blank_key = blank_key.detach().reshape(h, c).float().contiguous()
    blank_value = blank_value.detach().reshape(h, c).float().contiguous()
    d_query = torch.empty(b, n, h, c, dtype=dtype, device=device).permute(0, 2, 1, 3)
    probs = torch.empty(b, h, n, m, dtype=dtype, device=device)
    d_logit = torch.empty(b, h, n, m, dtype=dtype, device=device)
    blank_prob = torch.empty(b, h, n, dtype=torch.float32, device=device)
    d_blank = torch.empty(b, h, n, dtype=torch.float32, device=device)
    if probs.numel() == 0:
        return d_query, probs, d_logit, blank_prob, d_blank
    with torch.cuda.device(device):
        _check(lib.clusten_cluster_attention_backward(_ptr(query), _strides(query), _ptr(key), _strides(key), _ptr(value),
                                                      _strides(value), _ptr(g_view), _strides(g_view), _ptr(out_view),
                                                      _strides(out_view), _ptr(lse.contiguous()), _ptr(plan),
                                                      _ptr(bias_table), int(shared), _ptr(blank_key), _ptr(blank_value),
                                                      _ptr(d_query), _strides(d_query), _ptr(probs), _ptr(d_logit),
                                                      _ptr(blank_prob), _ptr(d_blank), ctypes.c_float(scale),
                                                      AttnShape(b, h, n, c, m), code, _stream(device)),
               "clusten_cluster_attention_backward")
    return d_query, probs, d_logit, blank_prob, d_blank


def dense_attention_supported(query: torch.Tensor) -> bool:
    """True when `dense_attention` takes this case: CUDA fp16 / bf16 queries of head dim 32, at most 64 tokens."""
    return (query.is_cuda and query.dtype in (torch.float16, torch.bfloat16) and query.dim() == 4
            and query.shape[3] == 32 and query.shape[2] <= 64)


def dense_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, bias_table: torch.Tensor,
                    pe_idx: torch.Tensor, blank_key: torch.Tensor, blank_value: torch.Tensor,
                    scale: float = 1.0) -> torch.Tensor:
    """Attention of every token over every token of a short sequence plus one blank token, in one kernel.

    query, key, value (B,H,N,32) fp16 / bf16 (any strides, channel stride 1), N <= 64; bias_table (rows,H);
    pe_idx (B,N,N) int64; blank_key, blank_value (H*32,).  Returns softmax(scale * q.k^T + bias | scale * q.blank_key)
    applied to the values and the blank value, as a (B,N,H*32) tensor of query's dtype (heads side by side, the
    layout the output projection takes).  No autograd: for inference.  The fused form of the global branch of
    models/aff_transformer.py:108-155.
    """
    lib = load()
    _require_cuda("query", query)
    device = query.device
    for name, t in (("key", key), ("value", value), ("bias_table", bias_table), ("pe_idx", pe_idx),
                    ("blank_key", blank_key), ("blank_value", blank_value)):
        _require_cuda(name, t, device)
    if query.dim() != 4 or key.shape != query.shape or value.shape != query.shape:
        raise RuntimeError("query, key and value must be (B,H,N,C) tensors of one shape")
    b, h, n, c = query.shape
    if pe_idx.shape != (b, n, n) or pe_idx.dtype != torch.int64:
        raise RuntimeError("pe_idx must be int64 of shape (B,N,N)")
    if bias_table.dim() != 2 or bias_table.shape[1] != h:
        raise RuntimeError("bias_table must have shape (rows, H)")
    if blank_key.numel() != h * c or blank_value.numel() != h * c:
        raise RuntimeError("blank_key and blank_value must have H*C elements")
    code = _dtype_code(query, "query")
    dtype = query.dtype
    query, key, value = _rows(query), _rows(key.to(dtype)), _rows(value.to(dtype))
    bias_table = bias_table.detach().to(dtype).contiguous()
    pe_idx = pe_idx.contiguous()
    blank_key = blank_key.detach().reshape(h, c).float().contiguous()
    blank_value = blank_value.detach().reshape(h, c).float().contiguous()
    out = torch.empty(b, n, h, c, dtype=dtype, device=device)
    if out.numel() == 0:
        return out.reshape(b, n, h * c)
    out_view = out.permute(0, 2, 1, 3)                                   # (B,H,N,C) view of the (B,N,H,C) memory
    shape = AttnShape(b, h, n, c, n)
    with torch.cuda.device(device):
        _check(lib.clusten_dense_attention_forward(_ptr(query), _strides(query), _ptr(key), _strides(key), _ptr(value),
                                                   _strides(value), _ptr(bias_table), _ptr(pe_idx), _ptr(blank_key),
                                                   _ptr(blank_value), _ptr(out), _strides(out_view),
                                                   ctypes.c_float(scale), shape, code, _stream(device)),
               "clusten_dense_attention_forward")
    return out.reshape(b, n, h * c)


_LINEAR_SHAPES = {(64, 64, 0), (64, 128, 0), (64, 192, 0), (128, 64, 0), (192, 64, 0),
                  (64, 64, 1), (64, 128, 1), (64, 192, 1)}                   # (K, Nout, gelu)
_LINEAR_MIN_ROWS = 65536


def linear_supported(x: torch.Tensor, weight: torch.Tensor, gelu: bool = False) -> bool:
    """True when `linear` takes this case: a CUDA fp16 / bf16 activation of many rows (the kernel is built for
    layers that move memory: at least 65536 rows) whose last axis is contiguous and a weight of one of the small
    shapes it is compiled for."""
    if not (x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and weight.dim() == 2 and x.dim() >= 2):
        return False
    nout, k = weight.shape
    if x.shape[-1] != k or (k, nout, int(gelu)) not in _LINEAR_SHAPES:
        return False
    return x.numel() // k >= _LINEAR_MIN_ROWS and x.is_contiguous()


def linear(x: torch.Tensor, weight: torch.Tensor, bias, gelu: bool = False) -> torch.Tensor:
    """`gelu(x @ weight.T + bias)` (or without the GELU) for x (..., K) and weight (Nout, K) of one 16-bit dtype,
    bias (Nout,) of that dtype or None: `nn.Linear` (+ `nn.GELU`) of models/aff_transformer.py:60-68, 181-196 for
    the small layers of the first stage.  No autograd: for inference."""
    lib = load()
    _require_cuda("x", x)
    device = x.device
    _require_cuda("weight", weight, device)
    if weight.dim() != 2 or x.dim() < 2 or x.shape[-1] != weight.shape[1]:
        raise RuntimeError("x must be (..., K) and weight (Nout, K)")
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise RuntimeError("x, weight and bias must have one dtype")
    nout, k = weight.shape
    code = _dtype_code(x, "x")
    if x.dim() == 2 and x.stride(1) == 1 and x.stride(0) >= k and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0:
        x2 = x                                       # rows of a wider matrix: read in place
    else:
        x2 = x.contiguous().view(-1, k)
    weight = weight.detach().contiguous()
    if bias is not None:
        _require_cuda("bias", bias, device)
        bias = bias.detach().contiguous()
        if bias.numel() != nout:
            raise RuntimeError("bias must have Nout elements")
    out = torch.empty(x.shape[:-1] + (nout,), dtype=x.dtype, device=device)
    if out.numel() == 0:
        return out
    with torch.cuda.device(device):
        _check(lib.clusten_linear_forward(_ptr(x2), x2.stride(0), _ptr(weight), _ptr(bias), _ptr(out), x2.shape[0], k,
                                          nout, int(bool(gelu)), code, _stream(device)),
               "clusten_linear_forward")
    return out


_LAYER_NORM_WIDTHS = (64, 128, 256, 384, 512, 768, 1024)
_DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def layer_norm_supported(x: torch.Tensor, out_dtype=None) -> bool:
    """True when `layer_norm` takes this case: a CUDA fp32 / fp16 / bf16 tensor whose last axis has one of the built
    widths."""
    return (x.is_cuda and x.dtype in _DTYPE_CODES and x.dim() >= 1 and x.shape[-1] in _LAYER_NORM_WIDTHS
            and (out_dtype is None or out_dtype in _DTYPE_CODES))


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5, out_dtype=None,
               order=None, pre_bias=None):
    """F.layer_norm(x.float(), (C,), weight, bias, eps), returned as `out_dtype` (fp32 unless given): the widening
    of a 16-bit input, the normalisation in fp32 and the rounding a following mixed-precision Linear applies, in
    one pass.  With `order` ((N,) int64, a permutation) x is (B,N,C) and row i of every image is the norm of its row
    order[i]; with `pre_bias` ((C,), x's dtype) the rows are x + pre_bias, rounded to x's dtype.  No autograd."""
    lib = load()
    _require_cuda("x", x)
    device = x.device
    _require_cuda("weight", weight, device)
    _require_cuda("bias", bias, device)
    out_dtype = torch.float32 if out_dtype is None else out_dtype
    if x.dtype not in _DTYPE_CODES or out_dtype not in _DTYPE_CODES:
        raise RuntimeError("layer_norm reads and writes fp32, fp16 or bf16")
    c = x.shape[-1]
    if weight.numel() != c or bias.numel() != c:
        raise RuntimeError("weight and bias must have as many elements as the last axis of x")
    x = x.detach().contiguous()
    weight = weight.detach().float().contiguous()
    bias = bias.detach().float().contiguous()
    out = torch.empty(x.shape, dtype=out_dtype, device=device)
    if out.numel() == 0:
        return out
    if order is None and pre_bias is None:
        with torch.cuda.device(device):
            _check(lib.clusten_layer_norm_forward(_ptr(x), _DTYPE_CODES[x.dtype], _ptr(weight), _ptr(bias), _ptr(out),
                                                  x.numel() // c, c,
                                                  ctypes.c_float(eps), _DTYPE_CODES[out_dtype], _stream(device)),
                   "clusten_layer_norm_forward")
        return out
    group = 1
    if order is not None:
        _require_cuda("order", order, device)
        if x.dim() != 3 or order.shape != (x.shape[1],) or order.dtype != torch.int64:
            raise RuntimeError("order must be an int64 tensor of N entries for x of shape (B,N,C)")
        order = order.contiguous()
        group = x.shape[1]
    if pre_bias is not None:
        _require_cuda("pre_bias", pre_bias, device)
        if pre_bias.numel() != c:
            raise RuntimeError("pre_bias must have as many elements as the last axis of x")
        pre_bias = pre_bias.detach().to(x.dtype).contiguous()
    with torch.cuda.device(device):
        _check(lib.clusten_layer_norm_rows_forward(_ptr(x), _DTYPE_CODES[x.dtype], _ptr(order), group, _ptr(pre_bias),
                                                   _ptr(weight), _ptr(bias), _ptr(out), x.numel() // c, c,
                                                   ctypes.c_float(eps), _DTYPE_CODES[out_dtype], _stream(device)),
               "clusten_layer_norm_rows_forward")
    return out


def channel_affine_gelu_supported(x: torch.Tensor) -> bool:
    """True when `channel_affine_gelu` takes this case: a contiguous CUDA fp16 / bf16 (B,C,H,W) tensor, H*W % 8 == 0."""
    return (x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and x.dim() == 4 and x.is_contiguous()
            and (x.shape[2] * x.shape[3]) % 8 == 0 and x.shape[0] * x.shape[1] < 65536)


def channel_affine_gelu(x: torch.Tensor, scale: torch.Tensor, shift: torch.Tensor) -> torch.Tensor:
    """F.gelu(x * scale[None,:,None,None] + shift[None,:,None,None]) in fp32, rounded once to x's 16-bit dtype: bias,
    inference BatchNorm and GELU after the first convolution of the patch embedding
    (models/aff_transformer.py:542) in one pass.  No autograd."""
    lib = load()
    _require_cuda("x", x)
    device = x.device
    _require_cuda("scale", scale, device)
    _require_cuda("shift", shift, device)
    if not channel_affine_gelu_supported(x):
        raise RuntimeError("channel_affine_gelu takes a contiguous fp16 / bf16 (B,C,H,W) tensor with H*W % 8 == 0")
    b, c, h, w = x.shape
    if scale.numel() != c or shift.numel() != c:
        raise RuntimeError("scale and shift must have C elements")
    scale = scale.detach().float().contiguous()
    shift = shift.detach().float().contiguous()
    out = torch.empty_like(x)
    if out.numel() == 0:
        return out
    with torch.cuda.device(device):
        _check(lib.clusten_channel_affine_gelu_forward(_ptr(x), _ptr(scale), _ptr(shift), _ptr(out), b, c, h * w,
                                                       _DTYPE_CODES[x.dtype], _stream(device)),
               "clusten_channel_affine_gelu_forward")
    return out


def add_layer_norm_supported(x: torch.Tensor, branch: torch.Tensor) -> bool:
    """True when `add_layer_norm` takes this case: CUDA tensors of one shape, the branch fp16 / bf16, x fp32 or of
    the branch's type, the last axis of one of the built widths."""
    return (x.is_cuda and branch.is_cuda and branch.dtype in (torch.float16, torch.bfloat16)
            and x.dtype in (torch.float32, branch.dtype) and x.shape == branch.shape and x.dim() >= 1
            and x.shape[-1] in _LAYER_NORM_WIDTHS)


def add_layer_norm(x: torch.Tensor, branch: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5):
    """(x + branch, F.layer_norm((x + branch).float(), (C,), weight, bias, eps).to(branch.dtype)) in one pass: the
    residual addition ahead of a norm and the norm (models/aff_transformer.py:230-232, :219).  The sum has x's dtype
    (fp32, or the branch's 16-bit type) and is rounded before it is normalised, like the separate addition's.
    No autograd: for inference."""
    lib = load()
    _require_cuda("x", x)
    device = x.device
    for name, t in (("branch", branch), ("weight", weight), ("bias", bias)):
        _require_cuda(name, t, device)
    if not add_layer_norm_supported(x, branch):
        raise RuntimeError("add_layer_norm: x fp32 or of the branch's type, branch fp16 / bf16, equal shapes, a built width")
    c = x.shape[-1]
    if weight.numel() != c or bias.numel() != c:
        raise RuntimeError("weight and bias must have as many elements as the last axis of x")
    x = x.detach().contiguous()
    branch = branch.detach().contiguous()
    weight = weight.detach().float().contiguous()
    bias = bias.detach().float().contiguous()
    total = torch.empty_like(x)
    out = torch.empty(x.shape, dtype=branch.dtype, device=device)
    if out.numel() == 0:
        return total, out
    with torch.cuda.device(device):
        _check(lib.clusten_add_layer_norm_forward(_ptr(x), _DTYPE_CODES[x.dtype], _ptr(branch), _DTYPE_CODES[branch.dtype],
                                                  _ptr(total), _ptr(weight), _ptr(bias), _ptr(out), x.numel() // c, c,
                                                  ctypes.c_float(eps), _stream(device)),
               "clusten_add_layer_norm_forward")
    return total, out


def neighbour_lists_supported(pos: torch.Tensor, nearest: torch.Tensor) -> bool:
    """True when `neighbour_lists` takes this case: CUDA fp32 positions (B,N,2) and int64 cluster numbers (B,N,nnc)."""
    return (pos.is_cuda and nearest.is_cuda and pos.dtype == torch.float32 and nearest.dtype == torch.int64
            and pos.dim() == 3 and pos.shape[2] == 2 and nearest.dim() == 3 and nearest.shape[:2] == pos.shape[:2])


def neighbour_lists(pos: torch.Tensor, nearest: torch.Tensor, m: int, radius: int, table_width: int, with_mask: bool):
    """(member_idx, mask or None, pe_idx, cluster_idx) of a cluster-ordered sequence: the members of each token's
    nearest clusters (clusters of m consecutive rows; rows past the last token become index 0 / mask 0), the row of
    the relative-position table for every (token, member) pair, and the cluster numbers as int32
    (models/aff_transformer.py:476-487).  pos (B,N,2) fp32, nearest (B,N,nnc) int64."""
    lib = load()
    _require_cuda("pos", pos)
    device = pos.device
    _require_cuda("nearest", nearest, device)
    if not neighbour_lists_supported(pos, nearest):
        raise RuntimeError("neighbour_lists takes fp32 positions (B,N,2) and int64 cluster numbers (B,N,nnc)")
    b, n, nnc = nearest.shape
    pos = pos.contiguous()
    nearest = nearest.contiguous()
    member_idx = torch.empty(b, n, nnc * m, dtype=torch.int64, device=device)
    pe_idx = torch.empty_like(member_idx)
    mask = torch.empty_like(member_idx) if with_mask else None
    cluster_idx = torch.empty(b, n, nnc, dtype=torch.int32, device=device)
    if member_idx.numel() == 0:
        return member_idx, mask, pe_idx, cluster_idx
    with torch.cuda.device(device):
        _check(lib.clusten_neighbour_lists(_ptr(pos), _ptr(nearest), _ptr(member_idx), _ptr(mask), _ptr(pe_idx),
                                           _ptr(cluster_idx), b, n, nnc, m, int(radius), int(table_width),
                                           _stream(device)),
               "clusten_neighbour_lists")
    return member_idx, mask, pe_idx, cluster_idx


def add_row_score_supported(x: torch.Tensor, branch, weight: torch.Tensor) -> bool:
    """True when `add_row_score` takes this case: CUDA tensors, weight (1,C) or (C,) fp16 / bf16 with C in
    {64,128,256,512}, x (...,C) fp32 or of weight's type, branch None or of x's shape and weight's type."""
    if not (x.is_cuda and weight.is_cuda and weight.dtype in (torch.float16, torch.bfloat16)):
        return False
    if x.dim() < 1 or x.shape[-1] not in (64, 128, 256, 512) or weight.numel() != x.shape[-1]:
        return False
    if x.dtype not in (torch.float32, weight.dtype):
        return False
    return branch is None or (branch.is_cuda and branch.dtype == weight.dtype and branch.shape == x.shape)


def add_row_score(x: torch.Tensor, branch, weight: torch.Tensor, bias):
    """(x + branch, sigmoid(F.linear((x + branch).to(T), weight, bias))) with T = weight's 16-bit dtype — or
    (x, sigmoid(...)) when branch is None: the importance score of the tokens before a merge
    (models/aff_transformer.py:498) and the residual addition ahead of it, in one pass.  The score has shape
    x.shape[:-1] + (1,) and dtype T.  No autograd: for inference."""
    lib = load()
    _require_cuda("x", x)
    device = x.device
    _require_cuda("weight", weight, device)
    if not add_row_score_supported(x, branch, weight):
        raise RuntimeError("add_row_score: weight fp16 / bf16 of 64, 128, 256 or 512 elements, x fp32 or of weight's "
                           "type, branch of x's shape and weight's type")
    c = x.shape[-1]
    code = _DTYPE_CODES[weight.dtype]
    x = x.detach().contiguous()
    weight = weight.detach().contiguous()
    if bias is not None:
        _require_cuda("bias", bias, device)
        if bias.numel() != 1 or bias.dtype != weight.dtype:
            raise RuntimeError("bias must be one element of weight's dtype")
        bias = bias.detach().contiguous()
    total = x
    if branch is not None:
        branch = branch.detach().contiguous()
        total = torch.empty_like(x)
    score = torch.empty(x.shape[:-1] + (1,), dtype=weight.dtype, device=device)
    if score.numel() == 0:
        return total, score
    with torch.cuda.device(device):
        _check(lib.clusten_add_row_score_forward(_ptr(x), _DTYPE_CODES[x.dtype], _ptr(branch),
                                                 _ptr(total) if branch is not None else None, _ptr(weight), _ptr(bias),
                                                 _ptr(score), x.numel() // c, c, code, _stream(device)),
               "clusten_add_row_score_forward")
    return total, score


def bias_table_grad_supported(d_logit: torch.Tensor, rows: int) -> bool:
    """True when `bias_table_grad` takes this case: a CUDA fp32 / fp16 / bf16 (B,H,N,M) gradient and a table of any number of rows."""
    return d_logit.is_cuda and d_logit.dtype in _DTYPE_CODES and d_logit.dim() == 4 and 0 < rows < 2 ** 31


def bias_table_grad(d_logit: torch.Tensor, pe_idx: torch.Tensor, rows: int) -> torch.Tensor:
    """d_table (rows,H) fp32 with d_table[pe_idx[b,i,j], h] = sum of d_logit[b,h,i,j]: the backward of the position-bias
    lookup of an attention layer (models/aff_transformer.py:131-133).  d_logit (B,H,N,M), pe_idx (B,N,M) int64."""
    lib = load()
    _require_cuda("d_logit", d_logit)
    device = d_logit.device
    _require_cuda("pe_idx", pe_idx, device)
    if not bias_table_grad_supported(d_logit, rows):
        raise RuntimeError("bias_table_grad takes a CUDA fp32 / fp16 / bf16 (B,H,N,M) gradient and a table of 1 to 2^31 - 1 rows")
    B, H, N, M = d_logit.shape
    if pe_idx.shape != (B, N, M) or pe_idx.dtype != torch.int64:
        raise RuntimeError("pe_idx must be int64 of shape (B,N,M)")
    d_logit, pe_idx = d_logit.contiguous(), pe_idx.contiguous()
    d_table = torch.zeros(rows, H, dtype=torch.float32, device=device)
    if d_logit.numel() == 0:
        return d_table
    with torch.cuda.device(device):
        _check(lib.clusten_bias_table_grad(_ptr(d_logit), _ptr(pe_idx), _ptr(d_table), B, H, N, M, rows,
                                           _DTYPE_CODES[d_logit.dtype], _stream(device)),
               "clusten_bias_table_grad")
    return d_table


def merge_weights_supported(table_weights: torch.Tensor) -> bool:
    """True when `merge_weights` takes this case: a CUDA table of 4 weights per row."""
    return table_weights.is_cuda and table_weights.dim() == 2 and table_weights.shape[1] == 4


def merge_weights(table_weights: torch.Tensor, pe_idx: torch.Tensor, nbhd_idx: torch.Tensor, prob, mask):
    """table_weights[pe_idx] * prob.gather(nbhd_idx) * mask as one (B,N',M,4) fp32 tensor: the weights the WF
    operator takes (models/aff_transformer.py:340-358).  table_weights (rows,4); pe_idx, nbhd_idx (B,N',M) int64;
    prob (B,N) or (B,N,1) or None; mask (B,N',M) of 0/1 or None.  No autograd: for inference."""
    lib = load()
    _require_cuda("table_weights", table_weights)
    device = table_weights.device
    _require_cuda("pe_idx", pe_idx, device)
    _require_cuda("nbhd_idx", nbhd_idx, device)
    if pe_idx.dim() != 3 or pe_idx.dtype != torch.int64 or nbhd_idx.shape != pe_idx.shape or nbhd_idx.dtype != torch.int64:
        raise RuntimeError("pe_idx and nbhd_idx must be int64 of one shape (B,N',M)")
    b, n_out, m = pe_idx.shape
    table_weights = table_weights.detach().float().contiguous()
    n = 1
    if prob is not None:
        _require_cuda("prob", prob, device)
        prob = prob.detach().reshape(b, -1).float().contiguous()
        n = prob.shape[1]
    if mask is not None:
        _require_cuda("mask", mask, device)
        if mask.shape != pe_idx.shape:
            raise RuntimeError("mask must have the shape of pe_idx")
        mask = mask.to(torch.int64).contiguous()
    out = torch.empty(b, n_out, m, table_weights.shape[1], dtype=torch.float32, device=device)
    if out.numel() == 0:
        return out
    with torch.cuda.device(device):
        _check(lib.clusten_merge_weights_forward(_ptr(table_weights), _ptr(pe_idx.contiguous()),
                                                 _ptr(nbhd_idx.contiguous()), _ptr(prob), _ptr(mask), _ptr(out), b, n,
                                                 n_out, m, table_weights.shape[1], _stream(device)),
               "clusten_merge_weights_forward")
    return out


def scanline_rank_supported(pos: torch.Tensor, rows: int, cols: int) -> bool:
    """True when `scanline_rank` takes this case: CUDA (B,N,2) positions, at least two anchor cells, and a sequence
    that one compute unit's LDS sorts (16384 tokens on an MI355X)."""
    if not (pos.is_cuda and pos.dim() == 3 and pos.shape[2] == 2 and pos.shape[1] > 0 and rows * cols >= 2):
        return False
    with torch.cuda.device(pos.device):
        return pos.shape[1] <= load().clusten_scanline_rank_max_tokens()


def cluster_centres(pos: torch.Tensor, ranking: torch.Tensor, m: int):
    """(pos in ranking order (B,N,2), mean position of every cluster of m consecutive tokens of that order
    (B,ceil(N/m),2)): what `space_filling_cluster` derives from its ranking (point_utils.py:161-208), in one kernel."""
    lib = load()
    _require_cuda("pos", pos)
    device = pos.device
    _require_cuda("ranking", ranking, device)
    if pos.dim() != 3 or pos.shape[2] != 2 or ranking.shape != pos.shape[:2] or ranking.dtype != torch.int64:
        raise RuntimeError("pos must be (B,N,2) and ranking an int64 (B,N) tensor")
    pos = pos.detach().float().contiguous()
    ranking = ranking.contiguous()
    b, n, _ = pos.shape
    k = (n + m - 1) // m
    pos_sorted = torch.empty_like(pos)
    centres = torch.empty(b, k, 2, dtype=torch.float32, device=device)
    if pos.numel():
        with torch.cuda.device(device):
            _check(lib.clusten_cluster_centres(_ptr(pos), _ptr(ranking), _ptr(pos_sorted), _ptr(centres), b, n, m,
                                               _stream(device)), "clusten_cluster_centres")
    return pos_sorted, centres


def gather_rows_supported(x: torch.Tensor) -> bool:
    """True when `gather_rows` takes this case: a CUDA (B,N,C) tensor whose rows are whole 16-byte pieces."""
    return x.is_cuda and x.dim() == 3 and x.numel() > 0 and (x.shape[2] * x.element_size()) % 16 == 0


def gather_rows(x: torch.Tensor, order: torch.Tensor) -> torch.Tensor:
    """out[b,i,:] = x[b, order[b,i], :] for x (B,N,C) and order (B,N) int64 — or (N,), one order for every image:
    `x.gather(1, order.unsqueeze(2).expand(-1, -1, C))` without an index per element.  No autograd."""
    lib = load()
    _require_cuda("x", x)
    device = x.device
    _require_cuda("order", order, device)
    if not gather_rows_supported(x) or order.dtype != torch.int64:
        raise RuntimeError("gather_rows takes (B,N,C) rows of whole 16-byte pieces and an int64 order")
    b, n, c = x.shape
    shared = order.dim() == 1
    if tuple(order.shape) != ((n,) if shared else (b, n)):
        raise RuntimeError("order must be (B,N) or (N,)")
    x = x.detach().contiguous()
    order = order.contiguous()
    out = torch.empty_like(x)
    with torch.cuda.device(device):
        _check(lib.clusten_gather_rows(_ptr(x), _ptr(order), _ptr(out), b, n, c * x.element_size(), int(shared),
                                       _stream(device)), "clusten_gather_rows")
    return out


def merge_centres_supported(pos: torch.Tensor, learned_prob=None) -> bool:
    """True when `merge_centres` takes this case: CUDA (B,N,2) positions of a sequence the selecting workgroup holds
    in LDS, importance scores (if any) in fp32 / fp16 / bf16."""
    if not (pos.is_cuda and pos.dim() == 3 and pos.shape[2] == 2 and pos.numel() > 0):
        return False
    if learned_prob is not None and not (learned_prob.is_cuda and learned_prob.dtype in _DTYPE_CODES
                                         and learned_prob.numel() == pos.shape[0] * pos.shape[1]):
        return False
    return pos.shape[1] <= load().clusten_merge_centres_max_tokens()


def merge_centres(pos: torch.Tensor, min_dist, learned_prob, alpha: float, stride: int, sample_num: int,
                  reserve_num: int, reserve_on: bool) -> torch.Tensor:
    """(B, sample_num [+ reserve_num]) int64: the tokens `ClusterMerging` keeps (aff_transformer.py:296-334) — the
    sample_num tokens of highest score (grid prior + learned_prob * alpha, - 100 on the reserved coarse grid), those
    above the sample_num-th score by ascending index and then those equal to it, followed, with reserve_on, by the
    reserve_num tokens of the coarse grid by ascending index.  `min_dist` (B,N): distance of every token to its
    nearest other token, or None while the tokens still fill the grid of `stride`."""
    lib = load()
    _require_cuda("pos", pos)
    device = pos.device
    if not merge_centres_supported(pos, learned_prob):
        raise RuntimeError("merge_centres: unsupported positions or importance scores")
    b, n, _ = pos.shape
    pos = pos.detach().float().contiguous()
    if min_dist is not None:
        _require_cuda("min_dist", min_dist, device)
        if min_dist.numel() != b * n:
            raise RuntimeError("min_dist must be (B,N)")
        min_dist = min_dist.detach().float().contiguous()
    code = 0
    if learned_prob is not None:
        _require_cuda("learned_prob", learned_prob, device)
        learned_prob = learned_prob.detach().contiguous()
        code = _DTYPE_CODES[learned_prob.dtype]
    centre = torch.empty(b, sample_num + (reserve_num if reserve_on else 0), dtype=torch.int64, device=device)
    with torch.cuda.device(device):
        _check(lib.clusten_merge_centres(_ptr(pos), _ptr(min_dist), _ptr(learned_prob), code, _ptr(centre), b, n,
                                         sample_num, reserve_num, int(bool(reserve_on)), ctypes.c_float(alpha),
                                         stride, _stream(device)), "clusten_merge_centres")
    if reserve_on and debug_indices() and centre.numel() and int(centre.min()) < 0:
        # the kernel marks the slots of reserved tokens an image does not have with -1; the reference's
        # `reserve_mask.nonzero().reshape(b, reserve_num)` raises there (aff_transformer.py:323)
        raise RuntimeError("merge_centres: an image holds fewer than reserve_num = %d tokens on the coarse grid"
                           % reserve_num)
    return centre


def merge_rows_supported(*tensors) -> bool:
    """True when `merge_rows` takes these tensors: CUDA (B,N,.) with rows of whole 8-byte words, at most four."""
    return 1 <= len(tensors) <= 4 and all(
        t.is_cuda and t.dim() == 3 and t.numel() > 0 and (t.shape[2] * t.element_size()) % 8 == 0 for t in tensors)


def merge_rows(centre: torch.Tensor, *tensors):
    """The rows of up to four (B,N,.) tensors at centre (B,n') int64, in one launch:
    `t.gather(1, centre.unsqueeze(2).expand(-1, -1, t.shape[2]))` for each (aff_transformer.py:337-344)."""
    lib = load()
    if not merge_rows_supported(*tensors):
        raise RuntimeError("merge_rows takes one to four CUDA (B,N,.) tensors with rows of whole 8-byte words")
    device = tensors[0].device
    _require_cuda("centre", centre, device)
    b, n = tensors[0].shape[:2]
    if centre.dtype != torch.int64 or centre.dim() != 2 or centre.shape[0] != b:
        raise RuntimeError("centre must be (B,n') int64")
    centre = centre.contiguous()
    n_out = centre.shape[1]
    src, dst = [], []
    for t in tensors:
        _require_cuda("tensor", t, device)
        if tuple(t.shape[:2]) != (b, n):
            raise RuntimeError("every tensor must be (B,N,.)")
        src.append(t.detach().contiguous())
        dst.append(torch.empty(b, n_out, t.shape[2], dtype=t.dtype, device=device))
    if n_out == 0:
        return tuple(dst)
    k = len(src)
    srcs = (ctypes.c_void_p * k)(*[t.data_ptr() for t in src])
    dsts = (ctypes.c_void_p * k)(*[t.data_ptr() for t in dst])
    sizes = (ctypes.c_int * k)(*[t.shape[2] * t.element_size() for t in src])
    with torch.cuda.device(device):
        _check(lib.clusten_merge_rows(srcs, dsts, sizes, k, _ptr(centre), b, n, n_out, _stream(device)),
               "clusten_merge_rows")
    return tuple(dst)


def scanline_rank(pos: torch.Tensor, rows: int, cols: int, cell_w: float, cell_h: float) -> torch.Tensor:
    """(B,N) int64: per image the order of the tokens along the scan-line walk over the rows x cols anchor grid
    (cells of cell_w x cell_h), the ranking of the reference's `space_filling_cluster` (point_utils.py:139-159)."""
    lib = load()
    _require_cuda("pos", pos)
    if pos.dim() != 3 or pos.shape[2] != 2:
        raise RuntimeError("pos must be (B,N,2)")
    device = pos.device
    pos = pos.detach().float().contiguous()
    b, n, _ = pos.shape
    ranking = torch.empty(b, n, dtype=torch.int64, device=device)
    if ranking.numel() == 0:
        return ranking
    nbytes = lib.clusten_scanline_rank_workspace_bytes(b, n)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        _check(lib.clusten_scanline_rank(_ptr(pos), _ptr(ranking), _ptr(workspace), nbytes, b, n, rows, cols,
                                         ctypes.c_float(cell_w), ctypes.c_float(cell_h), _stream(device)),
               "clusten_scanline_rank")
    return ranking


def knn2d_supported(query: torch.Tensor, database: torch.Tensor, k: int) -> bool:
    """True when `knn2d` takes this case: CUDA tensors of 2-D points, 1 <= k <= 8, k <= number of database points."""
    return (query.is_cuda and database.is_cuda and query.shape[-1] == 2 and database.shape[-1] == 2
            and 1 <= k <= 8 and k <= database.shape[1])


def knn2d(query: torch.Tensor, database: torch.Tensor, k: int, return_dist: bool = False):
    """Indices (B,Nq,k) int64 [and distances (B,Nq,k) fp32] of the k database points nearest to each query point."""
    lib = load()
    _require_cuda("query", query)
    _require_cuda("database", database, query.device)
    if query.dim() != 3 or database.dim() != 3 or query.shape[2] != 2 or database.shape[2] != 2 \
            or query.shape[0] != database.shape[0]:
        raise RuntimeError("knn2d needs query (B,Nq,2) and database (B,N,2)")
    device = query.device
    query = query.detach().float().contiguous()
    database = database.detach().float().contiguous()
    b, nq, _ = query.shape
    n = database.shape[1]
    idx = torch.empty(b, nq, k, dtype=torch.int64, device=device)
    dist = torch.empty(b, nq, k, dtype=torch.float32, device=device) if return_dist else None
    if idx.numel():
        with torch.cuda.device(device):
            _check(lib.clusten_knn2d(_ptr(query), _ptr(database), _ptr(idx), _ptr(dist), b, nq, n, k, _stream(device)),
                   "clusten_knn2d")
    return (idx, dist) if return_dist else idx
