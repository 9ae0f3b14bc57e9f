"""Stand-in for the reference's `clustenav_cuda` extension module (clusten/src/clustenav_cuda.cpp:25-51) on top of
libclusten_hip.so: `forward(attn, v, nbhd_idx) -> feat`, `backward(d_feat, attn, v, nbhd_idx) -> [d_attn, d_v]`."""
import torch

try:
    from . import clusten_hip_abi as A
except ImportError:  # imported as a top-level module, the way clusten/clusten.py:9-11 imports the compiled ones
    import clusten_hip_abi as A


def forward(attn, v, nbhd_idx):
    A.check_cuda(attn, v, nbhd_idx)
    attn, v, nbhd_idx = attn.contiguous(), A.rows_unit_stride(v), nbhd_idx.contiguous()
    b, h, n, m = attn.shape
    c = v.shape[3]
    feat = torch.empty(b, h, n, c, dtype=attn.dtype, device=attn.device)
    A.done("clusten_av_forward", A.lib.clusten_av_forward(
        A.ptr(attn), A.ptr(v), A.strides(v), A.ptr(nbhd_idx), A.ptr(feat), A.strides(feat),
        A.AttnShape(b, h, n, c, m), A.CODE[attn.dtype], A.stream(attn)))
    return feat


def backward(d_feat, attn, v, nbhd_idx):
    A.check_cuda(d_feat, attn, v, nbhd_idx)
    attn, v, nbhd_idx = attn.contiguous(), A.rows_unit_stride(v), nbhd_idx.contiguous()
    d_feat = A.rows_unit_stride(d_feat)
    b, h, n, m = attn.shape
    c = v.shape[3]
    shape, code = A.AttnShape(b, h, n, c, m), A.CODE[attn.dtype]
    d_attn = torch.empty(b, h, n, m, dtype=attn.dtype, device=attn.device)
    d_v = torch.empty(b, h, n, c, dtype=attn.dtype, device=attn.device)
    ws, nws, keep = A.workspace("av", shape, code, attn)
    A.done("clusten_av_backward", A.lib.clusten_av_backward(
        A.ptr(d_feat), A.strides(d_feat), A.ptr(attn), A.ptr(v), A.strides(v), A.ptr(nbhd_idx), A.ptr(d_attn),
        A.ptr(d_v), ws, nws, shape, code, A.stream(attn)))
    return [d_attn, d_v]
