"""Stand-in for the reference's `clustenwf_cuda` extension module (clusten/src/clustenwf_cuda.cpp:25-51) on top of
libclusten_hip.so: `forward(weights, feat, nbhd_idx) -> feat_new`,
`backward(d_feat_new, weights, feat, nbhd_idx) -> [d_weights, d_feat]`; weights (b,n',m,ic), feat (b,n,c)."""
import torch

try:
    from . import clusten_hip_abi as A
except ImportError:  # imported as a top-level module, the way clusten/clusten.py:9-11 imports the compiled ones
    import clusten_hip_abi as A


def _shape(weights, feat):
    b, n_out, m, ic = weights.shape
    return A.WfShape(b, feat.shape[1], n_out, feat.shape[2], m, ic)


def forward(weights, feat, nbhd_idx):
    A.check_cuda(weights, feat, nbhd_idx)
    weights, feat, nbhd_idx = weights.contiguous(), feat.contiguous(), nbhd_idx.contiguous()
    shape = _shape(weights, feat)
    feat_new = torch.empty(shape.B, shape.Nout, shape.IC, shape.C, dtype=weights.dtype, device=weights.device)
    A.done("clusten_wf_forward", A.lib.clusten_wf_forward(
        A.ptr(weights), A.ptr(feat), A.ptr(nbhd_idx), A.ptr(feat_new), shape, A.CODE[weights.dtype],
        A.stream(weights)))
    return feat_new


def backward(d_feat_new, weights, feat, nbhd_idx):
    A.check_cuda(d_feat_new, weights, feat, nbhd_idx)
    weights, feat, nbhd_idx = weights.contiguous(), feat.contiguous(), nbhd_idx.contiguous()
    d_feat_new = d_feat_new.contiguous()
    shape, code = _shape(weights, feat), A.CODE[weights.dtype]
    d_weights, d_feat = torch.empty_like(weights), torch.empty_like(feat)
    ws, nws, keep = A.workspace("wf", shape, code, weights)
    A.done("clusten_wf_backward", A.lib.clusten_wf_backward(
        A.ptr(d_feat_new), A.ptr(weights), A.ptr(feat), A.ptr(nbhd_idx), A.ptr(d_weights), A.ptr(d_feat), ws, nws,
        shape, code, A.stream(weights)))
    return [d_weights, d_feat]
