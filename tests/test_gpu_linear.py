"""GPU parity of the small-weight Linear kernel (`clusten_linear_forward`) against `F.linear` (and `F.gelu`)
evaluated in fp32 from the same rounded operands (models/aff_transformer.py:60-68, 181-196 are plain `nn.Linear` /
`nn.GELU` layers).

Bar: the fp32 sum rounded once to the 16-bit storage type: max|x - ref| / max|ref| <= 2e-3 (fp16), 1e-2 (bf16).
"""
import pytest
import torch
import torch.nn.functional as F

from clusten import _native
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu

BAR = {torch.float16: 2e-3, torch.bfloat16: 1e-2}
SHAPES = [(64, 64, False), (64, 128, False), (64, 192, False), (128, 64, False), (192, 64, False),
          (64, 64, True), (64, 128, True), (64, 192, True)]


def _reference(x, w, b, gelu):
    y = F.linear(x.float(), w.float(), None if b is None else b.float())
    if gelu:
        y = F.gelu(y.to(x.dtype).float())
    return y


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,nout,gelu", SHAPES)
def test_against_f_linear(device, dtype, k, nout, gelu):
    gen = torch.Generator().manual_seed(101)
    for rows in (65536 + 5, 70001):           # partial last block of 16 rows; more blocks than waves
        x = torch.randn(rows, k, generator=gen).to(dtype)
        w = (torch.randn(nout, k, generator=gen) * k ** -0.5).to(dtype)
        b = torch.randn(nout, generator=gen).to(dtype)
        ref = _reference(x, w, b, gelu)
        assert _native.linear_supported(x.to(device), w.to(device), gelu)
        out = _native.linear(x.to(device), w.to(device), b.to(device), gelu)
        assert out.dtype == dtype and out.shape == ref.shape
        err = oracle.rel_err(out, ref)
        assert err <= BAR[dtype], "%s K=%d Nout=%d gelu=%s rows=%d rel err %.3g" % (dtype, k, nout, gelu, rows, err)


def test_without_bias_batched_shape_and_row_stride(device):
    gen = torch.Generator().manual_seed(102)
    x = torch.randn(4, 20000, 64, generator=gen).half()
    w = (torch.randn(128, 64, generator=gen) / 8).half()
    out = _native.linear(x.to(device), w.to(device), None)
    assert out.shape == (4, 20000, 128)
    assert oracle.rel_err(out, _reference(x, w, None, False)) <= BAR[torch.float16]
    # rows of a wider matrix, read in place (row stride 192 elements)
    wide = torch.randn(70000, 192, generator=gen).half()
    view = wide.to(device)[:, 64:128]
    assert not view.is_contiguous()
    out = _native.linear(view, w.to(device), None)
    assert oracle.rel_err(out, _reference(wide[:, 64:128], w, None, False)) <= BAR[torch.float16]
    # integer-valued operands: every product and sum is exact, so is the result
    xi = torch.randint(-4, 5, (65536, 64), generator=gen).half()
    wi = torch.randint(-3, 4, (64, 64), generator=gen).half()
    bi = torch.randint(-8, 9, (64,), generator=gen).half()
    out = _native.linear(xi.to(device), wi.to(device), bi.to(device))
    assert torch.equal(out.cpu().float(), F.linear(xi.float(), wi.float(), bi.float()))


def test_gelu_epilogue_on_every_fp16_value(device):
    """y = GELU(x I^T): every finite fp16 value through the activation of the epilogue, against the exactly rounded
    GELU (float64 erfc).  The epilogue approximates erfc to a relative bound, so it stays within one fp16 ulp
    everywhere, the negative tail included."""
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    vals = bits.view(torch.float16)
    vals = vals[torch.isfinite(vals)]
    assert vals.numel() == 63488
    x = vals.repeat(67)[:65536 * 64].reshape(65536, 64).contiguous()
    eye = torch.eye(64, dtype=torch.float16)
    out = _native.linear(x.to(device), eye.to(device), None, True).cpu()
    x64 = x.double()
    exact = (x64 * 0.5 * torch.special.erfc(-x64 * 2 ** -0.5)).half()

    def ordered(t):      # fp16 bit patterns as integers that order like the values
        i = t.view(torch.int16).int()
        return torch.where(i < 0, -32768 - i, i)

    ulps = (ordered(out) - ordered(exact)).abs()
    assert int(ulps.max()) <= 1
    assert int((ulps > 0).sum()) <= 2e-3 * ulps.numel()
    # and next to the framework's kernel (0.5 x (1 + erf(x / sqrt 2)) in fp32, which cancels in the negative tail)
    theirs = F.gelu(x.to(device)).cpu()
    apart = (ordered(out) - ordered(theirs)).abs()
    assert int(apart.max()) <= 8 and int(apart[x >= -2].max()) <= 1
    assert (out.float() - theirs.float())[x < -2].abs().max() <= 4e-6      # one ulp of values below 2^-7


def test_unsupported_cases_are_refused(device):
    x = torch.zeros(70000, 64, dtype=torch.float16, device=device)
    w = torch.zeros(64, 64, dtype=torch.float16, device=device)
    assert _native.linear_supported(x, w)
    assert not _native.linear_supported(x[:1000], w)                        # few rows: the framework's kernel
    assert not _native.linear_supported(x.float(), w.float())
    assert not _native.linear_supported(x.cpu(), w.cpu())
    assert not _native.linear_supported(x, torch.zeros(96, 64, dtype=torch.float16, device=device))
    assert not _native.linear_supported(torch.zeros(70000, 192, dtype=torch.float16, device=device),
                                        torch.zeros(64, 192, dtype=torch.float16, device=device), gelu=True)
    with pytest.raises(RuntimeError):
        _native.linear(x, torch.zeros(96, 64, dtype=torch.float16, device=device), None)
    with pytest.raises(RuntimeError):
        _native.linear(x.float(), w.float(), None)
    with pytest.raises(RuntimeError):
        _native.linear(x, w.bfloat16(), None)
    assert _native.linear(x[:0], w, None).shape == (0, 64)
