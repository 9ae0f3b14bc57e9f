"""Stand-in for the reference's `clustenqk_cuda` extension module (clusten/src/clustenqk_cuda.cpp:25-51) on top of
libclusten_hip.so: `forward(query, key_t, nbhd_idx) -> attn`, `backward(d_attn, query, key, nbhd_idx) -> [d_query, d_key]`."""
import torch

try:
    from . import clusten_hip_abi as A
except ImportError:  # imported as a top-level module, the way clusten/clusten.py:9-11 imports the compiled ones
    import clusten_hip_abi as A


def forward(query, key_t, nbhd_idx):
    """`key_t` is the (b,h,c,n) transposed copy clusten/clusten.py:30 makes; its (b,h,n,c) view is read in place."""
    A.check_cuda(query, key_t, nbhd_idx)
    key = A.rows_unit_stride(key_t.permute(0, 1, 3, 2))
    query, nbhd_idx = A.rows_unit_stride(query), nbhd_idx.contiguous()
    b, h, n, c = query.shape
    m = nbhd_idx.shape[2]
    attn = torch.empty(b, h, n, m, dtype=query.dtype, device=query.device)
    A.done("clusten_qk_forward", A.lib.clusten_qk_forward(
        A.ptr(query), A.strides(query), A.ptr(key), A.strides(key), A.ptr(nbhd_idx), A.ptr(attn),
        A.AttnShape(b, h, n, c, m), A.CODE[query.dtype], A.stream(query)))
    return attn


def backward(d_attn, query, key, nbhd_idx):
    """The saved key is the un-transposed one (clusten/clusten.py:32)."""
    A.check_cuda(d_attn, query, key, nbhd_idx)
    query, key = A.rows_unit_stride(query), A.rows_unit_stride(key)
    d_attn, nbhd_idx = d_attn.contiguous(), nbhd_idx.contiguous()
    b, h, n, c = query.shape
    shape, code = A.AttnShape(b, h, n, c, nbhd_idx.shape[2]), A.CODE[query.dtype]
    d_query = torch.empty(b, h, n, c, dtype=query.dtype, device=query.device)
    d_key = torch.empty(b, h, n, c, dtype=query.dtype, device=query.device)
    ws, nws, keep = A.workspace("qk", shape, code, query)
    A.done("clusten_qk_backward", A.lib.clusten_qk_backward(
        A.ptr(d_attn), A.ptr(query), A.strides(query), A.ptr(key), A.strides(key), A.ptr(nbhd_idx), A.ptr(d_query),
        A.ptr(d_key), ws, nws, shape, code, A.stream(query)))
    return [d_query, d_key]
