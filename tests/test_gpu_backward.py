"""GPU parity of the backward kernels and of the drop-in autograd surface against autograd through
the CPU gather oracle, with RANDOM upstream gradients (the reference's scripts use `.mean()`, whose
constant gradient cannot detect a mis-indexed d_attn / d_feat).

Bar: <= 1e-5 (fp32) for the gather-type gradients d_query, d_attn, d_weights; <= 1e-4 for the
scatter-type gradients d_key, d_value, d_feat, whose fp32 atomics arrive in arbitrary order;
<= 1e-2 for fp16/bf16.
"""
import pytest
import torch

import workloads as wl
from clusten import CLUSTENAVFunction, CLUSTENQKFunction, CLUSTENWFFunction, _native
from conftest import TOL, TOL_SCATTER_F32
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu


def _scatter_tol(dtype):
    return TOL_SCATTER_F32 if dtype == torch.float32 else TOL[dtype]


def _ref(t):
    return t.double() if t.dtype == torch.float64 else t.float()


def _check_attn_backward(case, device, dtype):
    g = torch.Generator().manual_seed(70)
    q, k, v, idx = case.query.to(dtype), case.key.to(dtype), case.value.to(dtype), case.nbhd_idx
    B, H, N, C = q.shape
    M = idx.shape[-1]
    d_attn = torch.randn(B, H, N, M, generator=g).to(dtype)
    d_feat = torch.randn(B, H, N, C, generator=g).to(dtype)
    p = torch.softmax(torch.randn(B, H, N, M, generator=g), dim=-1).to(dtype)

    dq_ref, dk_ref = oracle.qk_gather_backward(_ref(d_attn), _ref(q), _ref(k), idx)
    dq, dk = _native.qk_backward(d_attn.to(device), q.to(device), k.to(device), idx.to(device))
    assert dq.dtype == dtype and dk.dtype == dtype
    assert oracle.rel_err(dq, dq_ref) <= TOL[dtype], "d_query %s" % case.name
    assert oracle.rel_err(dk, dk_ref) <= _scatter_tol(dtype), "d_key %s" % case.name

    da_ref, dv_ref = oracle.av_gather_backward(_ref(d_feat), _ref(p), _ref(v), idx)
    da, dv = _native.av_backward(d_feat.to(device), p.to(device), v.to(device), idx.to(device))
    assert oracle.rel_err(da, da_ref) <= TOL[dtype], "d_attn %s" % case.name
    assert oracle.rel_err(dv, dv_ref) <= _scatter_tol(dtype), "d_value %s" % case.name


def _check_wf_backward(case, device, dtype):
    g = torch.Generator().manual_seed(71)
    w, f, idx = case.weights.to(dtype), case.feat.to(dtype), case.nbhd_idx
    B, Nout, M, IC = w.shape
    C = f.shape[-1]
    d_out = torch.randn(B, Nout, IC, C, generator=g).to(dtype)
    dw_ref, df_ref = oracle.wf_gather_backward(_ref(d_out), _ref(w), _ref(f), idx)
    dw, df = _native.wf_backward(d_out.to(device), w.to(device), f.to(device), idx.to(device))
    assert dw.dtype == dtype and df.dtype == dtype and dw.shape == w.shape and df.shape == f.shape
    assert oracle.rel_err(dw, dw_ref) <= TOL[dtype], "d_weights %s" % case.name
    assert oracle.rel_err(df, df_ref) <= _scatter_tol(dtype), "d_feat %s" % case.name


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_attn_backward_cluster_shared(device, dtype):
    _check_attn_backward(wl.attn_case("shared", 72, B=2, H=2, N=200, C=32), device, dtype)


@pytest.mark.parametrize("lists", ["random", "model", "model_built"])
def test_attn_backward_per_token_lists(device, lists):
    _check_attn_backward(wl.attn_case(lists, 73, B=2, H=4, N=392, C=32, lists=lists), device, torch.float32)


@pytest.mark.parametrize("kind", ["clusters", "unaligned", "padded", "scattered", "repeated"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_attn_backward_lists_made_of_runs(device, kind, dtype):
    # the scatter's union path (and its fall-back for tiles with more than 16 distinct runs: "scattered");
    # N = 396 leaves a partial last tile, "repeated" makes a token list a run twice
    for c, h, m in ((32, 3, 48), (64, 2, 32), (16, 5, 64)):
        _check_attn_backward(wl.attn_case("runs", 77, B=2, H=h, N=396, C=c, M=m, lists="runs:" + kind), device, dtype)


def _whole(idx, device, n_rows=None):
    """True when the library finds `idx` to be lists made of whole clusters (reads the device flag: test only)."""
    block = _native.cluster_pairs(idx.to(device), n_rows)
    return block is not None and int(_native.pairs_not_whole(block)) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_attn_backward_cluster_by_cluster(device, dtype):
    """Lists made of whole clusters: d_key / d_value as a gather over the pairs of every cluster (no atomics)."""
    g = torch.Generator().manual_seed(79)
    for B, H, N, nnc, C in ((2, 3, 200, 6, 32), (1, 2, 392, 6, 32), (3, 1, 64, 8, 32), (2, 2, 24, 3, 32), (2, 2, 200, 6, 16),
                            (1, 3, 136, 6, 64)):
        idx = wl.model_like_lists(B, N, g, nnc=min(nnc, N // 8))
        assert _whole(idx, device)
        case = wl.attn_case("model", 80, B=B, H=H, N=N, C=C, M=idx.shape[-1])
        case.nbhd_idx = idx
        _check_attn_backward(case, device, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attn_backward_cluster_by_cluster_on_the_long_lists_of_the_384_models(device, dtype):
    """Clusters of 24 tokens, the members of the 6 nearest = 144 slots (configs/aff_base_22kto1k_384.yaml:10-11): every
    run of 8 slots of such a list is a whole cluster of 8 rows too, 18 runs per token, so the scatters run as gathers;
    a sequence that does not end on a cluster of 24 has runs of pad slots only and keeps the atomic kernels."""
    g = torch.Generator().manual_seed(83)
    for B, H, N, whole in ((2, 2, 240, True), (1, 4, 576, True), (2, 2, 250, False)):
        idx = wl.model_built_lists(B, N, g, cluster=24, nnc=6)
        assert idx.shape[-1] == 144 and _whole(idx, device) == whole
        case = wl.attn_case("long", 84, B=B, H=H, N=N, C=32, M=144, lists="random")
        case.nbhd_idx = idx
        _check_attn_backward(case, device, dtype)
    # the same lists for a merge: WF feature gradient by cluster
    idx = wl.model_built_lists(2, 240, g, cluster=24, nnc=6)[:, ::4].contiguous()
    wcase = wl.wf_case("long_wf", 85, B=2, N=240, C=64, M=144)
    wcase.nbhd_idx = idx
    assert _whole(idx, device, n_rows=240)
    _check_wf_backward(wcase, device, dtype)


def _padded_model_lists(B, N, nnc, gen):
    """Lists over a sequence whose last cluster is short: (B,N,8*nnc), clusters chosen at random per token, the
    slots past the last row hold index 0 (as the model pads them)."""
    K = (N + 7) // 8
    pick = torch.rand(B, N, K, generator=gen).argsort(dim=2)[:, :, :nnc]
    rows = pick.unsqueeze(3) * 8 + torch.arange(8)
    return torch.where(rows < N, rows, torch.zeros_like(rows)).reshape(B, N, nnc * 8)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_backward_cluster_by_cluster_with_a_short_last_cluster(device, dtype):
    """196 tokens = 24 clusters and one of 4: the lists that name it hold row 0 in their last slots, and those slots'
    contributions must reach row 0 (attention scatters and the WF feature gradient)."""
    g = torch.Generator().manual_seed(88)
    for B, H, N in ((2, 2, 196), (1, 3, 100), (2, 1, 13)):
        idx = _padded_model_lists(B, N, min(6, (N + 7) // 8), g)
        assert (idx == 0).sum() > B * N // 8
        assert _whole(idx, device)
        case = wl.attn_case("padded", 89, B=B, H=H, N=N, C=32, M=idx.shape[-1], lists="random")
        case.nbhd_idx = idx
        _check_attn_backward(case, device, dtype)
    B, N, Nout, C = 2, 196, 49, 64
    K = (N + 7) // 8
    pick = torch.rand(B, Nout, K, generator=g).argsort(dim=2)[:, :, :6]
    rows = pick.unsqueeze(3) * 8 + torch.arange(8)
    idx = torch.where(rows < N, rows, torch.zeros_like(rows)).reshape(B, Nout, 48)
    assert _whole(idx, device, N)
    case = wl.wf_case("padded", 90, B=B, N=N, C=C, IC=4, M=48, Nout=Nout)
    case.nbhd_idx = idx
    _check_wf_backward(case, device, dtype)


def test_cluster_by_cluster_scatter_properties(device):
    g = torch.Generator().manual_seed(81)
    B, H, N, C = 2, 3, 200, 32
    idx = wl.model_like_lists(B, N, g).to(device)
    M = idx.shape[-1]
    lists = _native.cluster_pairs(idx)
    assert lists.dtype == torch.uint8 and int(_native.pairs_not_whole(lists)) == 0
    # integer-valued data: every product and sum exact, so the result equals the oracle's bit for bit
    q = torch.randint(-4, 5, (B, H, N, C), generator=g).float()
    k = torch.randint(-4, 5, (B, H, N, C), generator=g).float()
    d_attn = torch.randint(-4, 5, (B, H, N, M), generator=g).float()
    dq_ref, dk_ref = oracle.qk_gather_backward(d_attn, q, k, idx.cpu())
    dq, dk = _native.qk_backward(d_attn.to(device), q.to(device), k.to(device), idx)
    assert torch.equal(dq.cpu(), dq_ref) and torch.equal(dk.cpu(), dk_ref)
    # no atomics: two runs on random data give the same bits, through the optional entry point and through the
    # drop-in backward (whose first call takes the same kernels as every later one)
    x = torch.randn(B, H, N, C, generator=g).to(device)
    p = torch.randn(B, H, N, M, generator=g).to(device)
    first = _native.scatter_rows_by_cluster(p, x, lists)
    assert torch.equal(first, _native.scatter_rows_by_cluster(p, x, lists))
    assert torch.equal(first, _native.scatter_rows_by_cluster(p, x, _native.cluster_pairs(idx)))   # a stable sort
    assert torch.equal(first, _native.qk_backward(p, x, x, idx)[1])
    assert torch.equal(first, _native.qk_backward(p, x, x, idx)[1])
    # a cluster nobody lists receives zeros; one listed by more pairs than a wave holds at once is taken in segments
    # (16-bit data too: the sum over all segments is rounded once)
    lone = torch.zeros(1, 2400, 48, dtype=torch.int64)
    lone[:] = (torch.arange(48) % 8) + 8 * (torch.arange(48) // 8 + 1)          # everybody lists clusters 1..6
    lone = lone.to(device)
    lists2 = _native.cluster_pairs(lone)
    x2 = torch.randn(1, 2, 2400, C, generator=g)
    p2 = torch.randn(1, 2, 2400, 48, generator=g)
    for dtype, tol in ((torch.float32, TOL_SCATTER_F32), (torch.float16, TOL[torch.float16]),
                       (torch.bfloat16, TOL[torch.bfloat16])):
        xs, ps = x2.to(dtype), p2.to(dtype)
        want = oracle.qk_gather_backward(ps.float(), xs.float(), xs.float(), lone.cpu())[1]
        got = _native.scatter_rows_by_cluster(ps.to(device), xs.to(device), lists2)
        assert oracle.rel_err(got, want) <= tol and float(got[:, :, :8].float().abs().max()) == 0.0
        if dtype != torch.float32:
            # one rounding of the fp32 sum: at most half a unit in the last place from the oracle's fp32 result
            assert oracle.rel_err(got, want.to(dtype).float()) <= (2e-3 if dtype == torch.float16 else 1.6e-2) * 0.51
    # lists that are not whole clusters: the flag is up, the optional entry point leaves its output alone, the drop-in
    # backward takes the atomic kernels
    for other in (torch.randint(N, (B, N, M), generator=g).to(device),
                  (idx + (torch.arange(M, device=device) < 8)).clamp_(max=N - 1)):
        block = _native.cluster_pairs(other)
        assert int(_native.pairs_not_whole(block)) == 1
        marker = torch.full((B, H, N, C), 7.0, device=device)
        _native.scatter_rows_by_cluster(p, x, block, out=marker)
        assert bool((marker == 7.0).all())
        want = oracle.qk_gather_backward(p.cpu(), x.cpu(), x.cpu(), other.cpu())[1]
        assert oracle.rel_err(_native.qk_backward(p, x, x, other)[1], want) <= TOL_SCATTER_F32
    assert _native.cluster_pairs(idx[:, :, :44].contiguous()) is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_backward_of_the_cluster_number_forms(device, dtype):
    """`qk_backward_clusters` / `av_backward_clusters`: the lists as (b,n,nnc) int32 cluster numbers in the backward too
    (pair lists straight from the numbers, `clusten_cluster_pairs_from_numbers`).  Against the oracle's backward on the
    expanded lists and bit for bit against the row-list backward (same kernels, same pair lists); a short last cluster;
    a number outside the sequence raises the block's flag."""
    g = torch.Generator().manual_seed(86)
    tol = TOL_SCATTER_F32 if dtype == torch.float32 else TOL[dtype]
    for B, H, N, C, nnc in ((2, 2, 203, 32, 6), (1, 3, 96, 64, 4), (2, 1, 400, 16, 8)):
        if C == 16 and dtype != torch.float32:
            continue
        idx = wl.model_built_lists(B, N, g, cluster=8, nnc=nnc)
        cidx = (idx[:, :, ::8] // 8).to(torch.int32).contiguous()
        q = torch.randn(B, H, N, C, generator=g).to(dtype)
        k = torch.randn(B, H, N, C, generator=g).to(dtype)
        p = torch.randn(B, H, N, 8 * nnc, generator=g).to(dtype)
        qd, kd, pd, idxd, cd = q.to(device), k.to(device), p.to(device), idx.to(device), cidx.to(device)
        pairs = _native.cluster_pairs_from_numbers(cd)
        assert int(_native.pairs_not_whole(pairs)) == 0
        want_dq, want_dk = oracle.qk_gather_backward(p.float(), q.float(), k.float(), idx)
        dq, dk = _native.qk_backward_clusters(pd, qd, kd, cd)
        what = "%s N=%d C=%d nnc=%d" % (dtype, N, C, nnc)
        assert oracle.rel_err(dq, want_dq) <= tol and oracle.rel_err(dk, want_dk) <= tol, what
        dq0, dk0 = _native.qk_backward(pd, qd, kd, idxd)
        assert torch.equal(dk, dk0) and oracle.rel_err(dq, dq0.float().cpu()) <= tol, what
        da, dv = _native.av_backward_clusters(qd, pd, kd, cd, pairs=pairs)
        da0, dv0 = _native.av_backward(qd, pd, kd, idxd)
        assert torch.equal(dv, dv0) and oracle.rel_err(da, da0.float().cpu()) <= tol, what
    stray = cd.clone()
    stray[0, 5, 1] = (N + 7) // 8
    assert int(_native.pairs_not_whole(_native.cluster_pairs_from_numbers(stray))) == 1
    stray[0, 5, 1] = -1
    assert int(_native.pairs_not_whole(_native.cluster_pairs_from_numbers(stray))) == 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_scatter_alone_with_the_callers_pair_lists(device, dtype):
    """`clusten_scatter_rows`: the scatter of the attention backward passes by itself, with pair lists the caller keeps.
    On lists made of whole clusters it is the gather over those lists (bit-equal to the entry point that only does
    that, and to the drop-in backward); on any other list the block's flag sends it to the atomic kernels, so the
    output is the full sum either way - nothing is left unwritten.  `qk_backward` / `av_backward` with `pairs=` are
    the same kernels as without."""
    g = torch.Generator().manual_seed(84)
    B, H, N, C = 2, 2, 203, 32                       # a short last cluster: 3 rows and 5 pad slots
    tol = TOL_SCATTER_F32 if dtype == torch.float32 else TOL[dtype]
    x = torch.randn(B, H, N, C, generator=g).to(dtype)
    k = torch.randn(B, H, N, C, generator=g).to(dtype)
    for kind in ("runs:padded", "model_built", "random", "windowed"):
        idx = wl.attn_case("s", 85, B=B, H=H, N=N, C=C, lists=kind).nbhd_idx
        M = idx.shape[-1]
        p = torch.randn(B, H, N, M, generator=g).to(dtype)
        xd, kd, pd, idxd = x.to(device), k.to(device), p.to(device), idx.to(device)
        pairs = _native.cluster_pairs(idxd)
        whole = int(_native.pairs_not_whole(pairs)) == 0
        assert whole == (kind in ("runs:padded", "model_built")), kind
        want_dq, want_dk = oracle.qk_gather_backward(p.float(), x.float(), k.float(), idx)
        got = _native.scatter_rows(pd, xd, idxd, pairs)
        assert got.dtype == dtype and oracle.rel_err(got, want_dk) <= tol, kind
        assert oracle.rel_err(_native.scatter_rows(pd, xd, idxd), want_dk) <= tol, kind      # pair lists built inside
        dq, dk = _native.qk_backward(pd, xd, kd, idxd, pairs=pairs)
        dq0, dk0 = _native.qk_backward(pd, xd, kd, idxd)
        assert torch.equal(dq, dq0) and oracle.rel_err(dq, want_dq) <= tol
        da, dv = _native.av_backward(xd, pd, kd, idxd, pairs=pairs)
        da0, dv0 = _native.av_backward(xd, pd, kd, idxd)
        assert torch.equal(da, da0)
        if whole:   # fixed summation order: the same bits through every door
            assert torch.equal(got, _native.scatter_rows_by_cluster(pd, xd, pairs))
            assert torch.equal(got, dk0) and torch.equal(dk, dk0) and torch.equal(dv, dv0)
        else:
            assert oracle.rel_err(dk, want_dk) <= tol and oracle.rel_err(dv, dv0.float().cpu()) <= 2 * tol
    with pytest.raises(RuntimeError, match="does not belong"):
        _native.scatter_rows(pd, xd, idxd, pairs[:-256])


def test_backward_never_reads_the_device_from_the_host(device):
    """The drop-in backward of the three operators recorded into a HIP graph (a capture fails on any synchronisation or
    read-back) and replayed with eager work between the replays: every replay equals the eager result bit for bit on
    lists made of whole clusters."""
    g = torch.Generator().manual_seed(93)
    B, H, N, C = 2, 2, 200, 32
    idx = wl.model_like_lists(B, N, g).to(device)
    M = idx.shape[-1]
    q, k = (torch.randn(B, H, N, C, generator=g).to(device) for _ in range(2))
    d_attn = torch.randn(B, H, N, M, generator=g).to(device)
    widx = _wf_cluster_lists(B, N, 50, 6, g).to(device)
    w = torch.randn(B, 50, 48, 4, generator=g).to(device)
    f = torch.randn(B, N, 64, generator=g).to(device)
    d_out = torch.randn(B, 50, 4, 64, generator=g).to(device)

    def step():
        return (_native.qk_backward(d_attn, q, k, idx) + _native.av_backward(q, d_attn, k, idx)
                + _native.wf_backward(d_out, w, f, widx))

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for _ in range(3):
        for t in outs:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want)
        again = step()                           # eager work between the replays
        for got, want in zip(again, eager):
            assert torch.equal(got, want)


def _wf_cluster_lists(B, N, Nout, nnc, gen):
    """(B,Nout,8*nnc) int64: every output token lists nnc distinct clusters of 8 consecutive feature rows."""
    K = N // 8
    pick = torch.rand(B, Nout, K, generator=gen).argsort(dim=2)[:, :, :nnc]
    return (pick.unsqueeze(3) * 8 + torch.arange(8)).reshape(B, Nout, nnc * 8)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_wf_backward_cluster_by_cluster(device, dtype):
    """WF lists made of whole clusters: d_feat as a gather over the pairs of every cluster (no atomics)."""
    g = torch.Generator().manual_seed(83)
    for B, N, Nout, C, nnc in ((2, 200, 50, 64, 6), (1, 392, 98, 128, 6), (2, 64, 16, 32, 8), (1, 48, 12, 96, 3)):
        idx = _wf_cluster_lists(B, N, Nout, nnc, g)
        assert _whole(idx, device, N)
        case = wl.wf_case("clusters", 84, B=B, N=N, C=C, IC=4, M=idx.shape[-1], Nout=Nout)
        case.nbhd_idx = idx
        _check_wf_backward(case, device, dtype)


def test_wf_cluster_by_cluster_properties(device):
    g = torch.Generator().manual_seed(85)
    B, N, Nout, C, IC = 2, 200, 50, 64, 4
    idx = _wf_cluster_lists(B, N, Nout, 6, g)
    M = idx.shape[-1]
    # integer-valued data: the result equals the oracle's bit for bit; a second run gives the same bits
    w = torch.randint(-3, 4, (B, Nout, M, IC), generator=g).float()
    f = torch.randint(-3, 4, (B, N, C), generator=g).float()
    d_out = torch.randint(-3, 4, (B, Nout, IC, C), generator=g).float()
    dw_ref, df_ref = oracle.wf_gather_backward(d_out, w, f, idx)
    dw, df = _native.wf_backward(d_out.to(device), w.to(device), f.to(device), idx.to(device))
    assert torch.equal(dw.cpu(), dw_ref) and torch.equal(df.cpu(), df_ref)
    # a cluster listed by more pairs than a wave holds at once (every output token lists clusters 0..5), and
    # clusters nobody lists
    many = (torch.arange(48) % 8 + 8 * (torch.arange(48) // 8)).expand(1, 600, 48).contiguous()
    w2 = torch.randn(1, 600, 48, IC, generator=g)
    f2 = torch.randn(1, 160, 32, generator=g)
    d2 = torch.randn(1, 600, IC, 32, generator=g)
    want = oracle.wf_gather_backward(d2, w2, f2, many)[1]
    got = _native.wf_backward(d2.to(device), w2.to(device), f2.to(device), many.to(device))[1]
    assert oracle.rel_err(got, want) <= TOL_SCATTER_F32 and float(got[:, 48:].abs().max()) == 0.0
    got16 = _native.wf_backward(d2.half().to(device), w2.half().to(device), f2.half().to(device), many.to(device))[1]
    want16 = oracle.wf_gather_backward(d2.half().float(), w2.half().float(), f2.half().float(), many)[1]
    assert oracle.rel_err(got16, want16.half().float()) <= 2e-3 * 0.51          # the fp32 sum rounded once
    # the optional entry point on the same pair lists gives the same bits as the drop-in backward
    block = _native.cluster_pairs(many.to(device), 160)
    assert torch.equal(_native.wf_backward_by_cluster(d2.to(device), w2.to(device), f2.to(device), many.to(device),
                                                      block)[1], got)
    # other inner channel counts and lists that are not whole clusters keep the atomic kernel
    case = wl.wf_case("knn", 86, B=2, N=200, C=64, IC=4)
    assert not _whole(case.nbhd_idx, device, 200)
    _check_wf_backward(case, device, torch.float32)
    case1 = wl.wf_case("ic1", 87, B=1, N=64, C=64, IC=1, M=48, Nout=16)
    case1.nbhd_idx = _wf_cluster_lists(1, 64, 16, 6, g)
    _check_wf_backward(case1, device, torch.float32)


def test_wf_feature_gradient_on_any_list_is_a_gather_in_a_fixed_order(device):
    """Lists that are not made of whole clusters (nearest-neighbour lists, random lists): the entries are sorted by the
    row they name on the device and every row is summed by one wave in ascending entry order — two runs give the same
    bits, integer-valued data the oracle's bits, rows nobody lists zeros, and a row half the entries name the right sum."""
    g = torch.Generator().manual_seed(94)
    case = wl.wf_case("knn", 95, B=3, N=200, C=64, IC=4)
    d_out = torch.randn(3, 50, 4, 64, generator=g)
    args = [t.to(device) for t in (d_out, case.weights, case.feat, case.nbhd_idx)]
    first = _native.wf_backward(*args)[1]
    for _ in range(3):
        assert torch.equal(_native.wf_backward(*args)[1], first)
    assert oracle.rel_err(first, oracle.wf_gather_backward(d_out, case.weights, case.feat, case.nbhd_idx)[1]) <= 1e-5
    # integer-valued data, random lists with repeats, odd sizes, fewer inner channels
    for B, N, Nout, C, IC, M in ((2, 77, 19, 32, 4, 20), (1, 130, 40, 96, 3, 48), (2, 64, 16, 128, 1, 7)):
        idx = torch.randint(N, (B, Nout, M), generator=g)
        idx[:, :, 0] = 5                                               # every output token names row 5
        w = torch.randint(-3, 4, (B, Nout, M, IC), generator=g).float()
        f = torch.randint(-3, 4, (B, N, C), generator=g).float()
        d2 = torch.randint(-3, 4, (B, Nout, IC, C), generator=g).float()
        dw_ref, df_ref = oracle.wf_gather_backward(d2, w, f, idx)
        dw, df = _native.wf_backward(d2.to(device), w.to(device), f.to(device), idx.to(device))
        assert torch.equal(dw.cpu(), dw_ref) and torch.equal(df.cpu(), df_ref), (B, N, Nout, C, IC, M)
    # rows nobody lists are zero; 16-bit data is summed in fp32 and rounded once
    idx = torch.randint(100, 200, (2, 50, 48), generator=g)
    w16, f16, d16 = case.weights[:2].half(), case.feat[:2].half(), d_out[:2].half()
    got = _native.wf_backward(d16.to(device), w16.to(device), f16.to(device), idx.to(device))[1]
    want = oracle.wf_gather_backward(d16.float(), w16.float(), f16.float(), idx)[1]
    assert float(got[:, :100].float().abs().max()) == 0.0
    assert oracle.rel_err(got, want.half().float()) <= 2e-3 * 0.51


def test_scatter_union_path_is_bit_exact_on_integer_data(device):
    g = torch.Generator().manual_seed(78)
    B, H, N, C = 2, 3, 200, 32
    idx = wl.model_like_lists(B, N, g)
    M = idx.shape[-1]
    q = torch.randint(-4, 5, (B, H, N, C), generator=g).float()
    k = torch.randint(-4, 5, (B, H, N, C), generator=g).float()
    d_attn = torch.randint(-4, 5, (B, H, N, M), generator=g).float()
    dq_ref, dk_ref = oracle.qk_gather_backward(d_attn, q, k, idx)
    dq, dk = _native.qk_backward(d_attn.to(device), q.to(device), k.to(device), idx.to(device))
    assert torch.equal(dq.cpu(), dq_ref) and torch.equal(dk.cpu(), dk_ref)


@pytest.mark.parametrize("c,h,m,n", [(16, 3, 48, 104), (64, 2, 48, 100), (24, 2, 48, 64), (32, 2, 20, 77),
                                     (32, 5, 144, 160), (32, 2, 5, 40)])
def test_attn_backward_shapes(device, c, h, m, n):
    _check_attn_backward(wl.attn_case("shape", 74, B=2, H=h, N=n, C=c, M=m), device, torch.float32)


def test_attn_backward_aff_base_384_shape_fp32(device):
    # configuration 3's backward check at its real token count and head layout, batch reduced so the
    # CPU autograd reference stays small
    _check_attn_backward(wl.config3_attn(dtype=torch.float32, B=1), device, torch.float32)


def test_scatter_integer_valued_data_is_bit_exact(device):
    g = torch.Generator().manual_seed(75)
    B, H, N, C, M = 2, 2, 136, 32, 48
    q = torch.randint(-4, 5, (B, H, N, C), generator=g).float()
    k = torch.randint(-4, 5, (B, H, N, C), generator=g).float()
    d_attn = torch.randint(-4, 5, (B, H, N, M), generator=g).float()
    for idx in (wl.windowed_cluster_lists(B, N, M, g), torch.randint(N, (B, N, M), generator=g)):
        dq_ref, dk_ref = oracle.qk_gather_backward(d_attn, q, k, idx)
        dq, dk = _native.qk_backward(d_attn.to(device), q.to(device), k.to(device), idx.to(device))
        assert torch.equal(dq.cpu(), dq_ref) and torch.equal(dk.cpu(), dk_ref)


def _tile_shared_lists(B, N, M, gen, kind):
    """(B,N,M) lists in which the 8 tokens of a tile share one list (`mixed`: every other tile does)."""
    tiles = (N + 7) // 8
    if kind == "near":
        return wl.windowed_cluster_lists(B, N, M, gen)
    per_tile = torch.randint(N, (B, tiles, M), generator=gen)                  # rows anywhere in the image
    if kind == "repeats":
        per_tile[:, :, M // 2:] = per_tile[:, :, :M - M // 2]                   # every row named twice
    idx = per_tile.repeat_interleave(8, dim=1)[:, :N].contiguous()
    if kind == "mixed":
        own = torch.randint(N, (B, N, M), generator=gen)
        odd = (torch.arange(N) // 8) % 2 == 1
        idx[:, odd] = own[:, odd]
    return idx


@pytest.mark.parametrize("kind", ["near", "far", "repeats", "mixed"])
@pytest.mark.parametrize("c,m,n,dtype", [(32, 48, 1501, torch.float32), (32, 48, 1501, torch.bfloat16),
                                         (16, 20, 1100, torch.float32), (64, 64, 613, torch.float16),
                                         (32, 4, 37, torch.float32), (64, 12, 300, torch.float32)])
def test_scatter_of_tiles_that_share_a_list(device, kind, c, m, n, dtype):
    """The tiles whose tokens share one list are summed in an LDS window of destination rows before they reach
    memory (rows outside the window are added directly), the other tiles by the tile kernel: sequences longer than
    one window, rows far from their tile, rows named twice, tiles of both sorts side by side, a short last tile."""
    g = torch.Generator().manual_seed(79)
    B, H = 2, 3
    idx = _tile_shared_lists(B, n, m, g, kind)
    q = torch.randn(B, H, n, c, generator=g).to(dtype)
    k = torch.randn(B, H, n, c, generator=g).to(dtype)
    d_attn = torch.randn(B, H, n, m, generator=g).to(dtype)
    dq_ref, dk_ref = oracle.qk_gather_backward(_ref(d_attn), _ref(q), _ref(k), idx)
    dq, dk = _native.qk_backward(d_attn.to(device), q.to(device), k.to(device), idx.to(device))
    assert oracle.rel_err(dq, dq_ref) <= TOL[dtype]
    assert oracle.rel_err(dk, dk_ref) <= _scatter_tol(dtype)
    # integer-valued data: every sum is exact in fp32, whatever the order of the additions
    qi = torch.randint(-4, 5, (B, H, n, c), generator=g).to(dtype)
    di = torch.randint(-4, 5, (B, H, n, m), generator=g).to(dtype)
    _, dk_ref = oracle.qk_gather_backward(_ref(di), _ref(qi), _ref(qi), idx)
    _, dk = _native.qk_backward(di.to(device), qi.to(device), qi.to(device), idx.to(device))
    assert torch.equal(dk.float().cpu(), dk_ref.to(dtype).float())


def test_scatter_conserves_mass_at_full_size(device):
    """Configuration 3's backward shape at full size (B64 H4 N9216 C32, fp32): the sum of d_key over
    destination rows equals the sum of all products whatever the indices are, and three batch
    elements are compared with the oracle."""
    case = wl.config3_attn(dtype=torch.float32, B=64)
    d = case.to(device)
    g = torch.Generator(device="cpu").manual_seed(76)
    d_attn = torch.randn(64, 4, 9216, 48, generator=g).to(device)
    dq, dk = _native.qk_backward(d_attn, d.query, d.key, d.nbhd_idx)
    lhs = dk.double().sum(2)
    rhs = (d_attn.double().sum(-1, keepdim=True) * d.query.double()).sum(2)
    assert oracle.rel_err(lhs, rhs) <= 1e-6
    for b in (0, 63):
        dq_ref, dk_ref = oracle.qk_gather_backward(d_attn[b:b + 1].cpu(), case.query[b:b + 1], case.key[b:b + 1],
                                                   case.nbhd_idx[b:b + 1])
        assert oracle.rel_err(dq[b:b + 1], dq_ref) <= TOL[torch.float32]
        assert oracle.rel_err(dk[b:b + 1], dk_ref) <= TOL_SCATTER_F32


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_wf_backward_dtypes(device, dtype):
    _check_wf_backward(wl.wf_case("wf", 77, B=2, N=196, C=64, dtype=dtype), device, dtype)


@pytest.mark.parametrize("c,ic,m", [(128, 4, 48), (256, 1, 48), (32, 4, 48), (96, 3, 20), (512, 4, 16)])
def test_wf_backward_shapes(device, c, ic, m):
    _check_wf_backward(wl.wf_case("wf", 78, B=2, N=196, C=c, IC=ic, M=m, Nout=40), device, torch.float32)


def test_wf_backward_aff_base_384_shape(device):
    _check_wf_backward(wl.config3_wf(dtype=torch.float32, B=1), device, torch.float32)


# ---- the drop-in autograd surface ------------------------------------------------------------------------

def test_autograd_functions_match_oracle_autograd(device):
    """The three Functions used the way the model uses them: QK -> softmax -> AV, and WF, with a loss
    that gives every output element its own random weight."""
    g = torch.Generator().manual_seed(79)
    case = wl.attn_case("auto", 79, B=2, H=2, N=200, C=32)
    loss_w = torch.randn(2, 2, 200, 32, generator=g)

    def run(qk, av, dev):
        q = case.query.to(dev).requires_grad_(True)
        k = case.key.to(dev).requires_grad_(True)
        v = case.value.to(dev).requires_grad_(True)
        idx = case.nbhd_idx.to(dev)
        attn = torch.softmax(qk(q, k, idx), dim=-1)
        feat = av(attn, v, idx)
        (feat * loss_w.to(dev)).sum().backward()
        return feat.detach(), q.grad, k.grad, v.grad

    got = run(CLUSTENQKFunction.apply, CLUSTENAVFunction.apply, device)
    ref = run(oracle.qk_gather, oracle.av_gather, "cpu")
    for name, x, y, tol in zip(("feat", "d_query", "d_key", "d_value"), got, ref,
                               (1e-5, 2e-5, TOL_SCATTER_F32, TOL_SCATTER_F32)):
        assert oracle.rel_err(x, y) <= tol, name

    wcase = wl.wf_case("auto_wf", 80, B=2, N=196, C=64)
    wloss = torch.randn(2, 49, 4, 64, generator=g)

    def run_wf(fn, dev):
        w = wcase.weights.to(dev).requires_grad_(True)
        f = wcase.feat.to(dev).requires_grad_(True)
        out = fn(w, f, wcase.nbhd_idx.to(dev))
        (out * wloss.to(dev)).sum().backward()
        return out.detach(), w.grad, f.grad

    got = run_wf(CLUSTENWFFunction.apply, device)
    ref = run_wf(oracle.wf_gather, "cpu")
    for name, x, y, tol in zip(("feat_new", "d_weights", "d_feat"), got, ref, (1e-5, 1e-5, TOL_SCATTER_F32)):
        assert oracle.rel_err(x, y) <= tol, name


def test_dtype_rules_of_the_reference_wrappers(device):
    """Second operand is cast to the first operand's dtype; output has the first operand's dtype
    (clusten/clusten.py:25-26,52-53,78-79) — the mixed dtypes fp16 autocast produces."""
    case = wl.attn_case("mixed", 81, B=2, H=2, N=104, C=32).to(device)
    attn16 = CLUSTENQKFunction.apply(case.query.half(), case.key, case.nbhd_idx)         # fp16 q, fp32 k
    assert attn16.dtype == torch.float16
    ref = oracle.qk_gather(case.query.half().float().cpu(), case.key.half().float().cpu(), case.nbhd_idx.cpu())
    assert oracle.rel_err(attn16, ref) <= 1e-2
    p = torch.softmax(attn16.float(), dim=-1)                                             # fp32 attn, fp16 v
    feat = CLUSTENAVFunction.apply(p, case.value.half(), case.nbhd_idx)
    assert feat.dtype == torch.float32
    ref = oracle.av_gather(p.cpu(), case.value.half().float().cpu(), case.nbhd_idx.cpu())
    assert oracle.rel_err(feat, ref) <= 1e-5
    wcase = wl.wf_case("mixed_wf", 82, B=2, N=196, C=64).to(device)
    out = CLUSTENWFFunction.apply(wcase.weights, wcase.feat.half(), wcase.nbhd_idx)      # fp32 w, fp16 feat
    assert out.dtype == torch.float32
    ref = oracle.wf_gather(wcase.weights.cpu(), wcase.feat.half().float().cpu(), wcase.nbhd_idx.cpu())
    assert oracle.rel_err(out, ref) <= 1e-5


def test_backward_returns_none_for_indices_and_accepts_noncontiguous_grads(device):
    case = wl.attn_case("nc", 83, B=2, H=2, N=104, C=32).to(device)
    q = case.query.clone().requires_grad_(True)
    k = case.key.clone().requires_grad_(True)
    attn = CLUSTENQKFunction.apply(q, k, case.nbhd_idx)
    up = torch.randn(2, 2, 48, 104, device=device).transpose(2, 3)                        # non-contiguous upstream
    attn.backward(up)
    dq_ref, dk_ref = oracle.qk_gather_backward(up.cpu(), case.query.cpu(), case.key.cpu(), case.nbhd_idx.cpu())
    assert oracle.rel_err(q.grad, dq_ref) <= 1e-5 and oracle.rel_err(k.grad, dk_ref) <= TOL_SCATTER_F32
    assert not case.nbhd_idx.requires_grad
