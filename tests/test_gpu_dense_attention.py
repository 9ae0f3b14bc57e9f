"""GPU parity of the one-kernel dense attention (`clusten_dense_attention_forward`) against the tensor expressions
the reference model writes for a stage that attends globally (models/aff_transformer.py:108-113, 125-155),
evaluated in fp32 from the same rounded inputs, and against the one-kernel local attention on lists that name
every cluster (two independent kernels, one function).

Bar: max|x - ref| / max|ref| <= 1e-2 (16-bit data; the probabilities are rounded to the storage type before they
weigh the values, the output is rounded once).
"""
import pytest
import torch

from clusten import _native
from conftest import TOL
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu

C = 32


def _reference(q, k, v, table, pe_idx, blank_k, blank_v, scale):
    """fp32 evaluation of the model's global branch; returns (B,N,H*C)."""
    b, h, n, c = q.shape
    q, k, v, table = q.float(), k.float(), v.float(), table.float()
    attn = (q @ k.transpose(-1, -2)) * scale + table[pe_idx].permute(0, 3, 1, 2)          # (b,h,n,n)
    blank = (q * blank_k.reshape(1, h, 1, c)).sum(-1, keepdim=True) * scale
    p = torch.softmax(torch.cat([attn, blank], dim=-1), dim=-1)
    out = p[..., :-1] @ v + p[..., -1:] * blank_v.reshape(1, h, 1, c)
    return out.permute(0, 2, 1, 3).reshape(b, n, h * c)


def _case(b, h, n, gen, dtype, rows=211):
    q = torch.randn(b, h, n, C, generator=gen).to(dtype)
    k = torch.randn(b, h, n, C, generator=gen).to(dtype)
    v = torch.randn(b, h, n, C, generator=gen).to(dtype)
    table = torch.randn(rows, h, generator=gen).to(dtype)
    pe_idx = torch.randint(rows, (b, n, n), generator=gen)
    blank_k = torch.randn(h * C, generator=gen)
    blank_v = torch.randn(h * C, generator=gen)
    return q, k, v, table, pe_idx, blank_k, blank_v


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_against_the_tensor_expressions(device, dtype):
    gen = torch.Generator().manual_seed(91)
    # 49: the last stage of the shipped models at 224 x 224; 64: the largest; 1, 16, 17, 33: block edges
    for b, h, n in ((3, 16, 49), (2, 3, 64), (2, 2, 1), (1, 1, 16), (2, 5, 17), (1, 2, 33), (2, 2, 48)):
        case = _case(b, h, n, gen, dtype)
        for scale in (C ** -0.5, 1.0):
            ref = _reference(*case, scale)
            out = _native.dense_attention(*[t.to(device) for t in case], scale=scale)
            assert out.dtype == dtype and out.shape == ref.shape and out.is_contiguous()
            err = oracle.rel_err(out, ref)
            assert err <= TOL[dtype], "%s b=%d h=%d n=%d scale=%.3g rel err %.3g" % (dtype, b, h, n, scale, err)


def test_strided_operands(device):
    """q as a view of the (B,N,H*C) projection, k / v as the views a fused kv projection leaves."""
    gen = torch.Generator().manual_seed(92)
    b, h, n = 2, 4, 49
    q, k, v, table, pe_idx, blank_k, blank_v = _case(b, h, n, gen, torch.float16)
    ref = _reference(q, k, v, table, pe_idx, blank_k, blank_v, 0.25)
    d = lambda x: x.to(device)
    q_view = d(q.permute(0, 2, 1, 3).contiguous()).permute(0, 2, 1, 3)                      # (b,n,h,c) memory
    kv = d(torch.stack([k, v], dim=0).permute(1, 3, 2, 0, 4).contiguous()).permute(3, 0, 2, 1, 4)   # (b,n,h,2,c) memory
    assert not q_view.is_contiguous() and not kv[0].is_contiguous()
    out = _native.dense_attention(q_view, kv[0], kv[1], d(table), d(pe_idx), d(blank_k), d(blank_v), scale=0.25)
    assert oracle.rel_err(out, ref) <= TOL[torch.float16]


def test_equals_the_local_kernel_on_lists_of_every_cluster(device):
    """48 tokens = six clusters of 8: with every cluster listed by every token the local attention is dense."""
    gen = torch.Generator().manual_seed(93)
    b, h, n = 3, 4, 48
    q, k, v, table, pe_idx, blank_k, blank_v = _case(b, h, n, gen, torch.float16)
    d = lambda x: x.to(device)
    cidx = torch.arange(6, dtype=torch.int32).expand(b, n, 6).contiguous()
    local = _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), None, d(blank_k), d(blank_v),
                                      scale=0.2)
    dense = _native.dense_attention(d(q), d(k), d(v), d(table), d(pe_idx), d(blank_k), d(blank_v), scale=0.2)
    assert oracle.rel_err(dense.float().cpu(), local.float().cpu()) <= 2e-3


def test_unsupported_cases_are_refused(device):
    gen = torch.Generator().manual_seed(94)
    q, k, v, table, pe_idx, blank_k, blank_v = _case(1, 2, 49, gen, torch.float16)
    d = lambda x: x.to(device)
    assert _native.dense_attention_supported(d(q))
    assert not _native.dense_attention_supported(d(q).float())
    assert not _native.dense_attention_supported(q)
    assert not _native.dense_attention_supported(d(torch.zeros(1, 2, 65, C, dtype=torch.float16)))
    assert not _native.dense_attention_supported(d(torch.zeros(1, 2, 49, 64, dtype=torch.float16)))
    with pytest.raises(RuntimeError):       # fp32 has no fused kernel
        _native.dense_attention(d(q).float(), d(k).float(), d(v).float(), d(table), d(pe_idx), d(blank_k), d(blank_v))
    with pytest.raises(RuntimeError):       # CPU tensors
        _native.dense_attention(q, k, v, table, pe_idx, blank_k, blank_v)
    big = _case(1, 1, 65, gen, torch.float16)
    with pytest.raises(RuntimeError):       # more than 64 tokens
        _native.dense_attention(*[d(t) for t in big])
    with pytest.raises(RuntimeError):       # pe_idx of the local form
        _native.dense_attention(d(q), d(k), d(v), d(table), d(pe_idx[:, :, :48]), d(blank_k), d(blank_v))
    empty = _native.dense_attention(d(q)[:0], d(k)[:0], d(v)[:0], d(table), d(pe_idx)[:0], d(blank_k), d(blank_v))
    assert empty.shape == (0, 49, 2 * C)
