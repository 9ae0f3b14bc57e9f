"""`clusten_qk_backward_static` — the QK backward through the entry point that allocates nothing (its fp32 scratch is
a fixed device array of the library) — against `clusten_qk_backward` with a caller-provided workspace, both through
the C ABI: two calls in a row on the shared scratch, the second with a smaller input.

Bar: d_query (a gather) bit-equal; d_key bit-equal on integer-valued data (every sum exact in fp32, so the order of
the atomics cannot show) and within 1e-2 (fp16 / bf16) or 1e-4 (fp32) of the workspace entry point and of the CPU
oracle on random data.  This file is collected last on purpose.
"""
import ctypes

import pytest
import torch

import workloads as wl
from clusten import _native
from conftest import TOL, TOL_SCATTER_F32
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu


def _inputs(seed, B, H, N, C, M, dtype, lists, integer):
    case = wl.attn_case("static", seed, B=B, H=H, N=N, C=C, M=M, lists=lists)
    g = torch.Generator().manual_seed(seed + 1)
    if integer:
        q = torch.randint(-3, 4, (B, H, N, C), generator=g).to(dtype)
        k = torch.randint(-3, 4, (B, H, N, C), generator=g).to(dtype)
        d_attn = torch.randint(-2, 3, (B, H, N, M), generator=g).to(dtype)
    else:
        q, k = case.query.to(dtype), case.key.to(dtype)
        d_attn = torch.randn(B, H, N, M, generator=g).to(dtype)
    return d_attn, q, k, case.nbhd_idx


def _both(device, d_attn, q, k, idx):
    d_attn, q, k, idx = (t.to(device) for t in (d_attn, q, k, idx))
    want_q, want_k = _native.qk_backward(d_attn, q, k, idx)           # clusten_qk_backward + torch workspace
    got_q = torch.full_like(q, float("nan"))
    got_k = torch.full_like(q, float("nan"))
    _native.qk_backward_static(d_attn, q, k, idx, got_q, got_k)       # no allocation, the library's scratch
    return (got_q, got_k), (want_q, want_k)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_two_calls_in_a_row_the_second_smaller(device, dtype):
    tol = TOL_SCATTER_F32 if dtype == torch.float32 else TOL[dtype]
    # first call: pair-list scratch and 2*3*392*32 sums in the scratch; second: a smaller problem that reuses its first
    # part; third: lists made of whole clusters (the cluster-by-cluster kernel, its pair lists in the scratch)
    for step, (B, H, N, C, M, lists) in enumerate(((2, 3, 392, 32, 48, "windowed"), (1, 2, 104, 32, 48, "random"),
                                                   (1, 2, 64, 32, 48, "model"))):
        for integer in (True, False):
            d_attn, q, k, idx = _inputs(300 + step, B, H, N, C, M, dtype, lists, integer)
            (got_q, got_k), (want_q, want_k) = _both(device, d_attn, q, k, idx)
            assert torch.equal(got_q, want_q), "d_query step %d" % step
            ref_q, ref_k = oracle.qk_gather_backward(d_attn.float(), q.float(), k.float(), idx)
            if integer:
                assert torch.equal(got_k, want_k), "d_key step %d" % step
                assert torch.equal(got_k.float().cpu(), ref_k.to(dtype).float()), "d_key vs oracle step %d" % step
            else:
                assert oracle.rel_err(got_k, want_k.float().cpu()) <= tol, "d_key step %d" % step
                assert oracle.rel_err(got_k, ref_k) <= tol, "d_key vs oracle step %d" % step
                assert oracle.rel_err(got_q, ref_q) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_a_warmed_call_allocates_nothing_and_replays_from_a_graph(device, dtype):
    """After one call on the device (which looks the scratch array's address up) a call changes neither the device's
    free memory nor the framework's allocation count, and it can be recorded into a HIP graph: replays, with eager
    calls between them, equal the eager result (integer-valued data, so the order of the atomics cannot show)."""
    d_attn, q, k, idx = (t.to(device) for t in _inputs(310, 2, 2, 200, 32, 48, dtype, "windowed", True))
    got_q, got_k = torch.empty_like(q), torch.empty_like(q)
    _native.qk_backward_static(d_attn, q, k, idx, got_q, got_k)       # the first call on this device
    torch.cuda.synchronize()
    want_q, want_k = got_q.clone(), got_k.clone()
    free0 = torch.cuda.mem_get_info()[0]
    count0 = torch.cuda.memory_stats()["allocation.all.allocated"]
    segs0 = torch.cuda.memory_stats()["segment.all.allocated"]
    _native.qk_backward_static(d_attn, q, k, idx, got_q, got_k)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == count0
    assert torch.cuda.memory_stats()["segment.all.allocated"] == segs0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _native.qk_backward_static(d_attn, q, k, idx, got_q, got_k)   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _native.qk_backward_static(d_attn, q, k, idx, got_q, got_k)
    for _ in range(3):
        got_q.fill_(float("nan"))
        got_k.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got_q, want_q) and torch.equal(got_k, want_k)
        small = [t.to(device) for t in _inputs(311, 1, 2, 64, 32, 48, dtype, "random", True)]   # eager work between
        sq, sk = torch.empty_like(small[1]), torch.empty_like(small[1])
        _native.qk_backward_static(*small, sq, sk)
        assert torch.equal(sk, _native.qk_backward(*small)[1])


def test_a_problem_beyond_the_scratch_is_refused(device):
    lib = _native.load()
    # 16-bit data: at least 4 bytes of scratch per d_key element
    elems = _native.STATIC_SCRATCH_BYTES // 4
    shape = _native.AttnShape(1, 1, elems // 32 + 8, 32, 8)
    rows = _native.Strides(shape.N * 32, shape.N * 32, 32)
    fake = ctypes.c_void_p(0x1000)      # never dereferenced: the size check comes before any launch
    st = lib.clusten_qk_backward_static(fake, fake, rows, fake, rows, fake, fake, fake, shape, 1, ctypes.c_void_p(0))
    assert st == 8
    assert b"scratch" in lib.clusten_status_string(st)
    q = torch.zeros(1, 1, shape.N, 32, dtype=torch.float16, device=device)
    with pytest.raises(RuntimeError, match="scratch"):
        _native.qk_backward_static(torch.zeros(1, 1, shape.N, 8, dtype=torch.float16, device=device), q, q,
                                   torch.zeros(1, shape.N, 8, dtype=torch.int64, device=device),
                                   torch.empty_like(q), torch.empty_like(q))
