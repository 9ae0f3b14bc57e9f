"""fp32 attention weights over 16-bit values (AV) and fp32 merge weights over 16-bit features (WF), the operand pairs
mixed precision hands the operators (reference: clusten/clusten.py:52-53,78-79 cast the 16-bit operand up first).
`clusten_av_forward_mixed` / `clusten_wf_forward_mixed` read the 16-bit operand in place; the bar is bit equality
with the cast-first path through `clusten_av_forward` / `clusten_wf_forward`, and the oracle's tolerance (1e-5: the
arithmetic is fp32) against the CPU gather expression on the widened operand."""
import pytest
import torch

import workloads as wl
from clusten import CLUSTENAVFunction, CLUSTENWFFunction, _native
from conftest import TOL
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("lists", ["windowed", "model", "random", "runs:padded", "runs:repeated"])
def test_av_mixed_equals_the_cast_first_path(device, dtype, lists):
    g = torch.Generator().manual_seed(40)
    for B, H, N, C, M in ((2, 2, 200, 32, 48), (1, 3, 104, 16, 48), (2, 2, 136, 64, 32), (1, 2, 77, 32, 20), (1, 2, 160, 32, 64),
                          (2, 1, 50, 24, 8)):
        if lists == "model" and (M != 48 or N % 8):
            continue
        if lists.startswith("runs:") and (M % 8 or N < M or M > 64):
            continue
        case = wl.attn_case("mixed", 41, B=B, H=H, N=N, C=C, M=M, lists=lists)
        v = case.value.to(dtype).to(device)
        attn = torch.softmax(torch.randn(B, H, N, M, generator=g), dim=-1).to(device)
        idx = case.nbhd_idx.to(device)
        got = _native.av_forward_mixed(attn, v, idx)
        want = _native.av_forward(attn, v.float(), idx)
        assert got.dtype == torch.float32
        assert torch.equal(got, want), (lists, B, H, N, C, M)
        ref = oracle.av_gather(attn.cpu(), v.float().cpu(), case.nbhd_idx)
        assert oracle.rel_err(got, ref) <= TOL[torch.float32]


def test_av_mixed_leaves_long_lists_to_the_cast_first_path(device):
    from clusten import CLUSTENAVFunction
    g = torch.Generator().manual_seed(48)
    case = wl.attn_case("mixed", 49, B=1, H=2, N=160, C=32, M=144)
    v = case.value.half().to(device)
    attn = torch.softmax(torch.randn(1, 2, 160, 144, generator=g), dim=-1).to(device)
    idx = case.nbhd_idx.to(device)
    assert not _native.mixed_supported(attn, v, attention=True)
    with pytest.raises(RuntimeError):
        _native.av_forward_mixed(attn, v, idx)
    assert torch.equal(CLUSTENAVFunction.apply(attn, v, idx), _native.av_forward(attn, v.float(), idx))


def test_av_mixed_reads_strided_values_in_place(device):
    # the model's value view: (B,N,2,H,C) storage, permuted to (B,H,N,C)
    g = torch.Generator().manual_seed(42)
    B, H, N, C, M = 2, 4, 200, 32, 48
    kv = torch.randn(B, N, 2, H, C, generator=g).half().to(device)
    v = kv[:, :, 1].permute(0, 2, 1, 3)
    assert not v.is_contiguous()
    case = wl.attn_case("mixed", 43, B=B, H=H, N=N, C=C, M=M)
    attn = torch.softmax(torch.randn(B, H, N, M, generator=g), dim=-1).to(device)
    idx = case.nbhd_idx.to(device)
    assert torch.equal(_native.av_forward_mixed(attn, v, idx), _native.av_forward(attn, v.float().contiguous(), idx))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_wf_mixed_equals_the_cast_first_path(device, dtype):
    for B, N, C, IC, M in ((2, 196, 64, 4, 48), (1, 200, 128, 4, 48), (2, 64, 256, 1, 20), (1, 100, 96, 3, 48), (1, 400, 64, 4, 144)):
        case = wl.wf_case("mixed", 44, B=B, N=N, C=C, IC=IC, M=M)
        feat = case.feat.to(dtype).to(device)
        w, idx = case.weights.to(device), case.nbhd_idx.to(device)
        got = _native.wf_forward_mixed(w, feat, idx)
        want = _native.wf_forward(w, feat.float(), idx)
        assert got.dtype == torch.float32 and torch.equal(got, want), (B, N, C, IC, M)
        ref = oracle.wf_gather(case.weights, feat.float().cpu(), case.nbhd_idx)
        assert oracle.rel_err(got, ref) <= TOL[torch.float32]


def test_the_functions_take_the_mixed_path_and_their_gradients_match_the_oracle(device):
    """AV and WF through the autograd Functions with the operand types of mixed precision: forward bit-equal to the
    cast-first forward, gradients (fp32 for the first operand; for the 16-bit operand the fp32 gradient the reference
    returns, which autograd casts) against autograd through the oracle."""
    g = torch.Generator().manual_seed(45)
    B, H, N, C, M = 2, 2, 200, 32, 48
    case = wl.attn_case("mixed", 46, B=B, H=H, N=N, C=C, M=M, lists="model")
    idx = case.nbhd_idx.to(device)
    attn0 = torch.softmax(torch.randn(B, H, N, M, generator=g), dim=-1)
    v0 = case.value.half()
    up = torch.randn(B, H, N, C, generator=g)

    attn = attn0.to(device).requires_grad_(True)
    v = v0.to(device).requires_grad_(True)
    out = CLUSTENAVFunction.apply(attn, v, idx)
    assert out.dtype == torch.float32
    assert torch.equal(out.detach(), _native.av_forward(attn0.to(device), v0.float().to(device), idx))
    (out * up.to(device)).sum().backward()
    a_ref = attn0.clone().requires_grad_(True)
    v_ref = v0.float().requires_grad_(True)
    (oracle.av_gather(a_ref, v_ref, case.nbhd_idx) * up).sum().backward()
    assert v.grad.dtype == torch.float16
    assert oracle.rel_err(attn.grad, a_ref.grad) <= TOL[torch.float32]
    assert oracle.rel_err(v.grad, v_ref.grad) <= TOL[torch.float16]

    wcase = wl.wf_case("mixed", 47, B=2, N=200, C=64, IC=4)
    widx = wcase.nbhd_idx.to(device)
    w = wcase.weights.to(device).requires_grad_(True)
    f = wcase.feat.to(torch.bfloat16).to(device).requires_grad_(True)
    upw = torch.randn(2, 50, 4, 64, generator=g)
    outw = CLUSTENWFFunction.apply(w, f, widx)
    assert outw.dtype == torch.float32
    assert torch.equal(outw.detach(), _native.wf_forward(wcase.weights.to(device), f.detach().float(), widx))
    (outw * upw.to(device)).sum().backward()
    w_ref = wcase.weights.clone().requires_grad_(True)
    f_ref = wcase.feat.to(torch.bfloat16).float().requires_grad_(True)
    (oracle.wf_gather(w_ref, f_ref, wcase.nbhd_idx) * upw).sum().backward()
    assert oracle.rel_err(w.grad, w_ref.grad) <= TOL[torch.float32]
    assert oracle.rel_err(f.grad, f_ref.grad) <= TOL[torch.bfloat16]
