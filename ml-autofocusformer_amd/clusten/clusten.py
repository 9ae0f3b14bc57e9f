"""The three CLUSTEN autograd Functions, with the reference's names, signatures and dtype rules
(clusten/clusten.py:17-92), on the gfx950 HIP kernels of libclusten_hip.so.

    CLUSTENQKFunction.apply(query, key, nbhd_idx)    -> attn      (b,h,n,m)
    CLUSTENAVFunction.apply(attn, v, nbhd_idx)       -> feat      (b,h,n,c)
    CLUSTENWFFunction.apply(weights, feat, nbhd_idx) -> feat_new  (b,n_,ic,c)

Same behaviour as the reference:
  * the second operand is cast to the first operand's dtype; the output has the first operand's dtype
    (clusten.py:25-26,52-53,78-79);
  * backward returns (grad_first, grad_second, None) (clusten.py:40,66,92);
  * non-CUDA tensors raise RuntimeError; importing the package without the compiled library raises
    RuntimeError (clusten.py:8-14).
Differences, none visible in results:
  * strided query / key / value views whose channel stride is 1 are read in place instead of being
    copied by `.contiguous()`, and key is not transposed;
  * fp32 attn with fp16 / bf16 v, and fp32 weights with fp16 / bf16 feat (what mixed precision produces), are
    computed from the 16-bit operand in place: bit-identical to the reference's cast-first forward, one pass less;
  * fp16 / bf16 sums are accumulated in fp32 and rounded once (the reference accumulates in half);
  * bfloat16 is accepted.
"""
from torch.autograd import Function

from . import _native

_native.load()  # fail at import time, like the reference, when the extension is missing


class CLUSTENQKFunction(Function):
    """
    query times key function
    """

    @staticmethod
    def forward(ctx, query, key, nbhd_idx):
        if key.dtype != query.dtype:
            key = key.to(query.dtype)
        attn = _native.qk_forward(query, key, nbhd_idx)
        ctx.save_for_backward(query, key, nbhd_idx)
        return attn

    @staticmethod
    def backward(ctx, grad_attn):
        query, key, nbhd_idx = ctx.saved_tensors
        d_query, d_key = _native.qk_backward(grad_attn, query, key, nbhd_idx)
        return d_query, d_key, None


class CLUSTENAVFunction(Function):
    """
    attention times value function
    """

    @staticmethod
    def forward(ctx, attn, v, nbhd_idx):
        if _native.mixed_supported(attn, v, attention=True):
            # fp32 weights over 16-bit values (mixed precision): the values are read in place; same result as the cast
            feat = _native.av_forward_mixed(attn, v, nbhd_idx)
        else:
            if attn.dtype != v.dtype:
                v = v.to(attn.dtype)
            feat = _native.av_forward(attn, v, nbhd_idx)
        ctx.save_for_backward(attn, v, nbhd_idx)
        return feat

    @staticmethod
    def backward(ctx, grad_feat):
        attn, v, nbhd_idx = ctx.saved_tensors
        if v.dtype != attn.dtype:
            v = v.to(attn.dtype)
        d_attn, d_v = _native.av_backward(grad_feat, attn, v, nbhd_idx)
        return d_attn, d_v, None


class CLUSTENWFFunction(Function):
    """
    weight times feature function
    """

    @staticmethod
    def forward(ctx, weights, feat, nbhd_idx):
        if _native.mixed_supported(weights, feat):
            # fp32 weights over 16-bit features: the features are read in place; same result as the cast
            feat_new = _native.wf_forward_mixed(weights, feat, nbhd_idx)
        else:
            if feat.dtype != weights.dtype:
                feat = feat.to(weights.dtype)
            feat_new = _native.wf_forward(weights, feat, nbhd_idx)
        ctx.save_for_backward(weights, feat, nbhd_idx)
        return feat_new

    @staticmethod
    def backward(ctx, grad_feat_new):
        weights, feat, nbhd_idx = ctx.saved_tensors
        if feat.dtype != weights.dtype:
            feat = feat.to(weights.dtype)
        d_weights, d_feat = _native.wf_backward(grad_feat_new, weights, feat, nbhd_idx)
        return d_weights, d_feat, None
