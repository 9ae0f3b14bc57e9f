"""GPU parity of the forward kernels against the CPU gather oracle, through the C ABI.

Bar: bit-exact for index handling (integer-valued data), max|x-ref|/max|ref| <= 1e-5 for fp32,
<= 1e-2 for fp16/bf16 (oracle evaluated in fp32 from the same rounded inputs), 1e-12 for fp64.
"""
import pytest
import torch

import workloads as wl
from clusten import _native
from conftest import TOL
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu


def _ref_inputs(*tensors):
    """The oracle sees the same rounded values, in fp32 (fp64 stays fp64)."""
    return [t.double() if t.dtype == torch.float64 else t.float() for t in tensors]


def _check_attn(case, device, dtype, check_av=True):
    q, k, v, idx = case.query.to(dtype), case.key.to(dtype), case.value.to(dtype), case.nbhd_idx
    qr, kr, vr = _ref_inputs(q, k, v)
    attn_ref = oracle.qk_gather_chunked(qr, kr, idx)
    attn = _native.qk_forward(q.to(device), k.to(device), idx.to(device))
    assert attn.dtype == dtype and attn.shape == attn_ref.shape and attn.is_contiguous()
    err = oracle.rel_err(attn, attn_ref)
    assert err <= TOL[dtype], "QK %s %s rel err %.3g" % (case.name, dtype, err)
    if check_av:
        p = torch.softmax(attn_ref, dim=-1).to(dtype)
        feat_ref = oracle.av_gather_chunked(_ref_inputs(p)[0], vr, idx)
        feat = _native.av_forward(p.to(device), v.to(device), idx.to(device))
        assert feat.dtype == dtype and feat.shape == feat_ref.shape and feat.is_contiguous()
        err = oracle.rel_err(feat, feat_ref)
        assert err <= TOL[dtype], "AV %s %s rel err %.3g" % (case.name, dtype, err)


def _check_wf(case, device, dtype):
    w, f, idx = case.weights.to(dtype), case.feat.to(dtype), case.nbhd_idx
    wr, fr = _ref_inputs(w, f)
    ref = oracle.wf_gather_chunked(wr, fr, idx)
    out = _native.wf_forward(w.to(device), f.to(device), idx.to(device))
    assert out.dtype == dtype and out.shape == ref.shape and out.is_contiguous()
    err = oracle.rel_err(out, ref)
    assert err <= TOL[dtype], "WF %s %s rel err %.3g" % (case.name, dtype, err)


# ---- QK / AV -----------------------------------------------------------------------------------------

def test_config0_fp32(device):
    _check_attn(wl.config0(), device, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_cluster_shared_lists_all_dtypes(device, dtype):
    _check_attn(wl.attn_case("shared", 50, B=3, H=2, N=392, C=32), device, dtype)


@pytest.mark.parametrize("lists", ["random", "model", "model_canonical", "model_built"])
def test_per_token_lists(device, lists):
    # random lists hold duplicates, like the reference's own test scripts (torch.randint)
    _check_attn(wl.attn_case(lists, 51, B=2, H=4, N=784 if lists != "random" else 196, C=32, lists=lists), device,
                torch.float32)


def test_reference_script_shape(device):
    # clusten/test_qk_kernel.py:14-18 (b reduced from 256 so the CPU oracle stays fast)
    _check_attn(wl.attn_case("refscript", 52, B=16, H=4, N=196, C=32, lists="random", scale_q=False), device,
                torch.float32)


@pytest.mark.parametrize("kind", ["clusters", "unaligned", "padded", "scattered", "repeated"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_lists_made_of_runs_of_eight(device, kind, dtype):
    # the tokens of a tile share most of their runs (not "scattered": up to 48 distinct runs, several passes);
    # N = 396 leaves a partial last tile, "padded" puts index 0 into the runs of a short last cluster
    _check_attn(wl.attn_case("runs", 61, B=2, H=3, N=396, C=32, lists="runs:" + kind), device, dtype)


@pytest.mark.parametrize("c,m", [(16, 48), (64, 48), (32, 16), (32, 64), (64, 64), (16, 8)])
def test_lists_made_of_runs_other_head_dims_and_lengths(device, c, m):
    _check_attn(wl.attn_case("runs", 62, B=2, H=2, N=200, C=c, M=m, lists="runs:clusters"), device, torch.float32)
    _check_attn(wl.attn_case("runs", 63, B=1, H=2, N=200, C=c, M=m, lists="runs:scattered"), device, torch.bfloat16)


@pytest.mark.parametrize("n", [49, 197, 8, 5])
def test_partial_tiles(device, n):
    m = min(48, n) if n >= 48 else 4
    lists = "windowed" if n >= 48 else "random"
    _check_attn(wl.attn_case("ragged", 53, B=2, H=2, N=n, C=32, M=m, lists=lists), device, torch.float32)


@pytest.mark.parametrize("c", [16, 64, 24, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_head_dims(device, c, dtype):
    # 16/32/64 take the tile kernels, anything else the element kernels
    _check_attn(wl.attn_case("c%d" % c, 54, B=2, H=3, N=200, C=c), device, dtype)


@pytest.mark.parametrize("m", [4, 16, 20, 32, 64, 144, 5])
def test_list_lengths(device, m):
    # 48 is the unguarded kernel; others are range-checked; 144 (the 384x384 models) spans three chunks;
    # 5 is not a multiple of 4 (element kernel for AV)
    _check_attn(wl.attn_case("m%d" % m, 55, B=2, H=2, N=320, C=32, M=m), device, torch.float32)


def _cluster_lists(B, N, cluster, nnc, gen, kind="model"):
    """Lists of nnc runs of `cluster` slots: the members of a token's nearest clusters ("model", nearest first, as the
    reference builds them), with the short last cluster padded by row 0 ("padded"), with runs of other rows mixed in
    ("irregular": some runs are not consecutive rows, one token repeats a run), or runs scattered over the whole sequence
    so that a tile holds more distinct runs than the kernel keeps ("scattered")."""
    if kind == "model":
        return wl.model_like_lists(B, N, gen, cluster=cluster, nnc=nnc)
    K = (N + cluster - 1) // cluster
    own = torch.arange(N) // cluster
    if kind == "scattered":
        pick = torch.rand(B, N, K, generator=gen).argsort(dim=2)[:, :, :nnc]
    else:
        lo = (own - 4).clamp(min=0, max=max(K - 9, 0))
        pick = torch.rand(B, N, min(9, K), generator=gen).argsort(dim=2)[:, :, :nnc] + lo.view(1, N, 1)
    rows = pick.unsqueeze(3) * cluster + torch.arange(cluster)
    idx = torch.where(rows < N, rows, torch.zeros_like(rows)).reshape(B, N, nnc * cluster)
    if kind == "irregular":
        idx[:, 5::7, cluster:2 * cluster] = torch.randint(N, (B, len(range(5, N, 7)), cluster), generator=gen)
        idx[:, 3::11, 2 * cluster:3 * cluster] = idx[:, 3::11, :cluster]            # a run held twice by one token
        idx[:, 2::13, 0] = idx[:, 2::13, 1]                                         # a duplicate inside a run
    return idx


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind", ["model", "padded", "irregular", "scattered"])
def test_long_lists_made_of_long_runs(device, dtype, kind):
    """The neighbourhoods of the 384 x 384 models (configs/aff_base_22kto1k_384.yaml:10-11): 6 clusters of 24 tokens, 144
    slots — and other run lengths the kernels for long runs take (32, 16)."""
    g = torch.Generator().manual_seed(57)
    # 620 tokens: the last tile of 24 holds 20 (and, padded, a short last cluster)
    for N, cluster, nnc, C, H in ((2304, 24, 6, 32, 2), (600, 24, 6, 64, 1), (620, 24, 6, 32, 2), (400, 32, 4, 32, 3),
                                  (328, 16, 5, 32, 2)):
        if kind == "model" and N % cluster:
            N -= N % cluster
        if kind != "padded" and kind != "model":
            N -= N % 8
        idx = _cluster_lists(1 if N > 1000 else 2, N, cluster, nnc, g, kind)
        case = wl.attn_case("runs%d" % cluster, 58, B=idx.shape[0], H=H, N=N, C=C, M=idx.shape[-1], lists="random")
        case.nbhd_idx = idx
        _check_attn(case, device, dtype)


def test_long_runs_integer_valued_data_is_bit_exact(device):
    g = torch.Generator().manual_seed(59)
    N, H, C = 960, 2, 32
    for kind in ("model", "padded", "irregular", "scattered"):
        idx = _cluster_lists(2, N, 24, 6, g, kind)
        q = torch.randint(-4, 5, (2, H, N, C), generator=g).float()
        k = torch.randint(-4, 5, (2, H, N, C), generator=g).float()
        p = torch.randint(-3, 4, (2, H, N, 144), generator=g).float()
        assert torch.equal(_native.qk_forward(q.to(device), k.to(device), idx.to(device)).cpu(),
                           oracle.qk_gather_chunked(q, k, idx)), kind
        assert torch.equal(_native.av_forward(p.to(device), k.to(device), idx.to(device)).cpu(),
                           oracle.av_gather_chunked(p, k, idx)), kind


@pytest.mark.parametrize("h", [1, 3, 5, 16])
def test_head_counts(device, h):
    _check_attn(wl.attn_case("h%d" % h, 56, B=2, H=h, N=104, C=32), device, torch.float32)


def test_head_dim_16_with_odd_head_count(device):
    _check_attn(wl.attn_case("c16h3", 57, B=2, H=3, N=104, C=16), device, torch.float32)


def test_integer_valued_data_is_bit_exact(device):
    # products and partial sums of small integers are exact in fp32, so any summation order gives the
    # same bits: a wrong index, offset or stride cannot hide inside a tolerance
    g = torch.Generator().manual_seed(58)
    B, H, N, C, M = 3, 4, 136, 32, 48
    q = torch.randint(-8, 9, (B, H, N, C), generator=g).float()
    k = torch.randint(-8, 9, (B, H, N, C), generator=g).float()
    v = torch.randint(-8, 9, (B, H, N, C), generator=g).float()
    p = torch.randint(-4, 5, (B, H, N, M), generator=g).float()
    for idx in (wl.windowed_cluster_lists(B, N, M, g), torch.randint(N, (B, N, M), generator=g)):
        attn = _native.qk_forward(q.to(device), k.to(device), idx.to(device))
        assert torch.equal(attn.cpu(), oracle.qk_gather(q, k, idx))
        feat = _native.av_forward(p.to(device), v.to(device), idx.to(device))
        assert torch.equal(feat.cpu(), oracle.av_gather(p, v, idx))


def test_strided_views_are_read_in_place(device):
    # the model hands over permuted views of (b,n,h,c) / (b,n,h,2,c) storage (aff_transformer.py:117-119)
    g = torch.Generator().manual_seed(59)
    B, H, N, C, M = 2, 4, 200, 32, 48
    q_store = torch.randn(B, N, H, C, generator=g)
    kv_store = torch.randn(B, N, H, 2, C, generator=g)
    idx = wl.windowed_cluster_lists(B, N, M, g)
    qd, kvd = q_store.to(device), kv_store.to(device)
    q = qd.permute(0, 2, 1, 3)
    kv = kvd.permute(3, 0, 2, 1, 4)
    key, val = kv[0], kv[1]
    assert not q.is_contiguous() and not key.is_contiguous()
    attn = _native.qk_forward(q, key, idx.to(device))
    attn_ref = oracle.qk_gather(q.cpu(), key.cpu(), idx)
    assert oracle.rel_err(attn, attn_ref) <= TOL[torch.float32]
    p = torch.softmax(attn_ref, dim=-1)
    feat = _native.av_forward(p.to(device), val, idx.to(device))
    assert oracle.rel_err(feat, oracle.av_gather(p, val.cpu(), idx)) <= TOL[torch.float32]
    # token-major output: same values, storage laid out (b,n,h,c)
    feat_tm = _native.av_forward(p.to(device), val, idx.to(device), token_major=True)
    assert feat_tm.shape == feat.shape and feat_tm.permute(0, 2, 1, 3).is_contiguous()
    assert torch.equal(feat_tm, feat)
    # a transposed channel axis cannot be read in place and is copied
    qt = torch.randn(B, H, C, N, generator=g).to(device).transpose(2, 3)
    attn_t = _native.qk_forward(qt, key, idx.to(device))
    assert oracle.rel_err(attn_t, oracle.qk_gather(qt.cpu(), key.cpu(), idx)) <= TOL[torch.float32]


def test_unaligned_rows_take_the_element_kernels(device):
    g = torch.Generator().manual_seed(60)
    B, H, N, C, M = 2, 2, 64, 32, 48
    store = torch.randn(B, H, N, C + 1, generator=g)          # row pitch 33 floats: rows are not 16-byte aligned
    idx = wl.windowed_cluster_lists(B, N, M, g)
    k = store.to(device)[..., 1:]
    q = torch.randn(B, H, N, C, generator=g)
    attn = _native.qk_forward(q.to(device), k, idx.to(device))
    assert oracle.rel_err(attn, oracle.qk_gather(q, store[..., 1:], idx)) <= TOL[torch.float32]


def test_aff_mini_stage1_shape_fp32_fp16(device):
    # configuration 1 at a batch the CPU oracle handles in seconds
    for dtype in (torch.float32, torch.float16):
        _check_attn(wl.config1(dtype=dtype, B=4), device, dtype)


@pytest.mark.parametrize("stage", [1, 2, 3, 4])
def test_aff_tiny_stage_shapes(device, stage):
    # configuration 2 (all four stages) at batch 4
    _check_attn(wl.config2_attn(stage, B=4), device, torch.float32)


def test_aff_base_384_shape_bf16(device):
    _check_attn(wl.config3_attn(B=2), device, torch.bfloat16)


def test_full_size_stage1_batch_slices_and_linearity(device):
    """Configuration 2 stage 1 at its full batch of 128: three batch elements against the oracle, and
    two properties that hold for every element: out(2a) == 2*out(a) bit for bit (scaling by a power of
    two commutes with every rounding), and the batch elements are independent of each other."""
    case = wl.config2_attn(1, B=128)
    d = case.to(device)
    attn = _native.qk_forward(d.query, d.key, d.nbhd_idx)
    for b in (0, 63, 127):
        ref = oracle.qk_gather(case.query[b:b + 1], case.key[b:b + 1], case.nbhd_idx[b:b + 1])
        assert oracle.rel_err(attn[b:b + 1], ref) <= TOL[torch.float32]
    assert torch.equal(_native.qk_forward(2 * d.query, d.key, d.nbhd_idx), 2 * attn)
    sub = _native.qk_forward(d.query[100:104], d.key[100:104], d.nbhd_idx[100:104])
    assert torch.equal(sub, attn[100:104])
    p = torch.softmax(attn, dim=-1)
    feat = _native.av_forward(p, d.value, d.nbhd_idx)
    for b in (0, 63, 127):
        ref = oracle.av_gather(p[b:b + 1].cpu(), case.value[b:b + 1], case.nbhd_idx[b:b + 1])
        assert oracle.rel_err(feat[b:b + 1], ref) <= TOL[torch.float32]
    assert torch.equal(_native.av_forward(p, 2 * d.value, d.nbhd_idx), 2 * feat)
    # softmax rows sum to one, so every output lies inside the range of the gathered values
    assert feat.abs().max() <= d.value.abs().max()


# ---- WF ----------------------------------------------------------------------------------------------

@pytest.mark.parametrize("stage", [1, 2, 3, 4])
@pytest.mark.parametrize("ic", [4, 1])
def test_wf_aff_tiny_stages(device, stage, ic):
    _check_wf(wl.config2_wf(stage, IC=ic, B=4), device, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("c", [64, 128, 256, 512])
def test_wf_dtypes_and_channel_counts(device, dtype, c):
    _check_wf(wl.wf_case("wf", 61, B=2, N=196, C=c, dtype=dtype), device, dtype)


@pytest.mark.parametrize("c,ic,m", [(32, 4, 48), (96, 4, 48), (64, 3, 48), (64, 2, 48), (64, 4, 16), (64, 4, 144),
                                    (128, 1, 20), (64, 1, 5)])
def test_wf_other_shapes(device, c, ic, m):
    # (32,4,48) is the reference script's shape family (test_wf_kernel.py:14-19) and AFF-Mini stage 1
    _check_wf(wl.wf_case("wf", 62, B=2, N=196, C=c, IC=ic, M=m, Nout=64), device, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,ic,m", [(128, 4, 48), (128, 3, 48), (256, 2, 48), (128, 1, 48), (128, 4, 16), (128, 4, 144),
                                    (128, 4, 20), (128, 2, 100), (512, 4, 52), (64, 4, 48)])
def test_wf_16_bit_rows_on_the_16_bit_matrix_path(device, dtype, c, ic, m):
    """fp16 / bf16 weights over rows of the same type: four slots per matrix instruction.  Lists of 48 slots (no range
    checks) and other lengths (64 slots at a time, the tail of the last four-slot group zeroed), 1 to 4 inner channels,
    rows of 128 bytes (element kernel) to 1 KiB; sums of small integers must come out exactly rounded."""
    _check_wf(wl.wf_case("wf16", 64, B=2, N=196, C=c, IC=ic, M=m, Nout=50, dtype=dtype), device, dtype)
    g = torch.Generator().manual_seed(65)
    w = torch.randint(-4, 5, (2, 50, m, ic), generator=g).float()
    f = torch.randint(-8, 9, (2, 196, c), generator=g).float()
    idx = torch.randint(196, (2, 50, m), generator=g)
    out = _native.wf_forward(w.to(dtype).to(device), f.to(dtype).to(device), idx.to(device))
    # the fp32 sums of these integers are exact, so the result is their one rounding to the storage type
    assert torch.equal(out.cpu(), oracle.wf_gather(w, f, idx).to(dtype))


def test_wf_integer_valued_data_is_bit_exact(device):
    g = torch.Generator().manual_seed(63)
    B, N, Nout, C, M, IC = 2, 196, 49, 128, 48, 4
    w = torch.randint(-4, 5, (B, Nout, M, IC), generator=g).float()
    f = torch.randint(-8, 9, (B, N, C), generator=g).float()
    idx = torch.randint(N, (B, Nout, M), generator=g)
    out = _native.wf_forward(w.to(device), f.to(device), idx.to(device))
    assert torch.equal(out.cpu(), oracle.wf_gather(w, f, idx))


def test_wf_aff_base_384_shape_bf16(device):
    _check_wf(wl.config3_wf(B=2), device, torch.bfloat16)


def test_wf_full_size_stage1(device):
    case = wl.config2_wf(1, IC=4, B=128)
    d = case.to(device)
    out = _native.wf_forward(d.weights, d.feat, d.nbhd_idx)
    for b in (0, 77, 127):
        ref = oracle.wf_gather(case.weights[b:b + 1], case.feat[b:b + 1], case.nbhd_idx[b:b + 1])
        assert oracle.rel_err(out[b:b + 1], ref) <= TOL[torch.float32]
    assert torch.equal(_native.wf_forward(d.weights, 2 * d.feat, d.nbhd_idx), 2 * out)
    # rows of the weights are non-negative and sum to one: outputs are convex combinations
    assert out.abs().max() <= d.feat.abs().max() * (1 + 1e-6)


def _cluster_numbers(b, n, nnc, gen, kind):
    """(B,N,nnc) int32 cluster numbers: clusters = ceil(N/8); the last one may be short (its pad slots list row 0)."""
    k = (n + 7) // 8
    own = torch.arange(n) // 8
    if kind == "shared":          # every token of a cluster lists the same clusters in the same order
        per_cluster = torch.stack([torch.randperm(k, generator=gen)[:nnc] for _ in range(b * k)]).reshape(b, k, nnc)
        return per_cluster[:, own].to(torch.int32).contiguous()
    width = k if kind == "scattered" else min(12, k)
    lo = torch.zeros(n, dtype=torch.int64) if kind == "scattered" else (own - width // 2).clamp(0, k - width)
    pick = torch.rand(b, n, width, generator=gen).argsort(dim=2)[:, :, :nnc] + lo.view(1, n, 1)
    return pick.to(torch.int32).contiguous()


def _expand_clusters(cidx, n):
    rows = cidx.long().unsqueeze(3) * 8 + torch.arange(8)
    rows = torch.where(rows < n, rows, torch.zeros_like(rows))
    return rows.reshape(cidx.shape[0], cidx.shape[1], -1).contiguous()


@pytest.mark.parametrize("kind", ["near", "shared", "scattered"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_lists_given_as_cluster_numbers(device, kind, dtype):
    gen = torch.Generator().manual_seed(71)
    for n, c, nnc in ((396, 32, 6), (200, 64, 8), (64, 16, 2)):
        b, h = 2, 3
        q = (torch.randn(b, h, n, c, generator=gen) * c ** -0.5).to(dtype)
        k = torch.randn(b, h, n, c, generator=gen).to(dtype)
        v = torch.randn(b, h, n, c, generator=gen).to(dtype)
        cidx = _cluster_numbers(b, n, nnc, gen, kind)
        idx = _expand_clusters(cidx, n)
        assert idx.max() < n and idx.shape == (b, n, 8 * nnc)
        # against the oracle on the expanded lists ...
        qr, kr, vr = _ref_inputs(q, k, v)
        attn_ref = oracle.qk_gather_chunked(qr, kr, idx)
        attn = _native.qk_forward_clusters(q.to(device), k.to(device), cidx.to(device))
        assert attn.dtype == dtype and oracle.rel_err(attn, attn_ref) <= TOL[dtype]
        p = torch.softmax(attn_ref, dim=-1).to(dtype)
        feat_ref = oracle.av_gather_chunked(_ref_inputs(p)[0], vr, idx)
        feat = _native.av_forward_clusters(p.to(device), v.to(device), cidx.to(device))
        assert feat.dtype == dtype and oracle.rel_err(feat, feat_ref) <= TOL[dtype]
        # ... and against the row-list entry points on the same lists
        assert oracle.rel_err(attn, _native.qk_forward(q.to(device), k.to(device), idx.to(device)).cpu()) <= TOL[dtype]
        assert oracle.rel_err(feat, _native.av_forward(p.to(device), v.to(device), idx.to(device)).cpu()) <= TOL[dtype]
    assert not _native.clusters_supported(q.to(device), 9)
    with pytest.raises(RuntimeError):
        _native.qk_forward_clusters(q.to(device), k.to(device), cidx.long().to(device))


def _cluster_numbers_of(b, n, nnc, cs, gen, kind):
    """(B,N,nnc) int32 numbers of clusters of `cs` rows; tokens of one cluster pick theirs from the same dozen."""
    k = (n + cs - 1) // cs
    own = torch.arange(n) // cs
    if kind == "shared":
        per_cluster = torch.stack([torch.randperm(k, generator=gen)[:nnc] for _ in range(b * k)]).reshape(b, k, nnc)
        return per_cluster[:, own].to(torch.int32).contiguous()
    width = k if kind == "scattered" else min(9, k)
    lo = torch.zeros(n, dtype=torch.int64) if kind == "scattered" else (own - width // 2).clamp(0, k - width)
    pick = torch.rand(b, n, width, generator=gen).argsort(dim=2)[:, :, :nnc] + lo.view(1, n, 1)
    return pick.to(torch.int32).contiguous()


@pytest.mark.parametrize("kind", ["near", "shared", "scattered", "outside"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_long_lists_given_as_numbers_of_larger_clusters(device, kind, dtype):
    """The cluster-number forms on lists of more than 64 slots: clusters of 24 rows (6 of them: the 144 slots of the
    384 x 384 models), of 32 and of 16, against the oracle and against the row-list entry points on the expanded lists
    (bit for bit: same kernels, same order of sums).  A short last cluster, tiles of 20 tokens, and cluster numbers
    whose rows lie outside the sequence (they stand for row 0)."""
    gen = torch.Generator().manual_seed(72)
    for n, c, nnc, cs in ((596, 32, 6, 24), (240, 64, 6, 24), (300, 32, 4, 32), (212, 32, 5, 16), (148, 32, 4, 24)):
        b, h = 2, 3
        q = (torch.randn(b, h, n, c, generator=gen) * c ** -0.5).to(dtype)
        k = torch.randn(b, h, n, c, generator=gen).to(dtype)
        v = torch.randn(b, h, n, c, generator=gen).to(dtype)
        assert _native.cluster_size_for(cs * nnc) == cs
        cidx = _cluster_numbers_of(b, n, nnc, cs, gen, "near" if kind == "outside" else kind)
        if kind == "outside":
            far = torch.rand(b, n, nnc, generator=gen) < 0.1
            cidx = torch.where(far, torch.full_like(cidx, (n + cs - 1) // cs + 3), cidx)
            cidx[:, ::17, 0] = -2
        rows = cidx.long().unsqueeze(3) * cs + torch.arange(cs)
        idx = torch.where((rows >= 0) & (rows < n), rows, torch.zeros_like(rows)).reshape(b, n, cs * nnc).contiguous()
        qr, kr, vr = _ref_inputs(q, k, v)
        attn_ref = oracle.qk_gather_chunked(qr, kr, idx)
        attn = _native.qk_forward_clusters(q.to(device), k.to(device), cidx.to(device), cluster_size=cs)
        what = "%s %s n=%d c=%d %dx%d" % (kind, dtype, n, c, nnc, cs)
        assert attn.dtype == dtype and oracle.rel_err(attn, attn_ref) <= TOL[dtype], what
        p = torch.softmax(attn_ref, dim=-1).to(dtype)
        feat_ref = oracle.av_gather_chunked(_ref_inputs(p)[0], vr, idx)
        feat = _native.av_forward_clusters(p.to(device), v.to(device), cidx.to(device), cluster_size=cs)
        assert feat.dtype == dtype and oracle.rel_err(feat, feat_ref) <= TOL[dtype], what
        assert oracle.rel_err(attn, _native.qk_forward(q.to(device), k.to(device), idx.to(device)).cpu()) <= TOL[dtype], what
        assert oracle.rel_err(feat, _native.av_forward(p.to(device), v.to(device), idx.to(device)).cpu()) <= TOL[dtype], what
    assert _native.clusters_supported(q.to(device), 6, 24) and not _native.clusters_supported(q.to(device), 9, 24)
    assert not _native.clusters_supported(q.to(device), 6, 20)
    with pytest.raises(RuntimeError):   # 6 clusters of 20 rows: no such form
        _native.qk_forward_clusters(q.to(device), k.to(device), cidx.to(device)[:, :, :6].contiguous(), cluster_size=20)


def test_empty_inputs_give_empty_or_zero_outputs(device):
    # no batch elements, no tokens, or empty lists: nothing is launched
    for b, n, m in ((0, 16, 8), (2, 0, 8), (2, 16, 0)):
        q = torch.randn(b, 2, n, 32, device=device)
        idx = torch.zeros(b, n, m, dtype=torch.int64, device=device)
        attn = _native.qk_forward(q, q, idx)
        assert attn.shape == (b, 2, n, m)
        feat = _native.av_forward(attn, q, idx)
        assert feat.shape == (b, 2, n, 32) and (feat == 0).all()
        w = torch.randn(b, n, m, 4, device=device)
        f = torch.randn(b, max(n, 1) * 4, 64, device=device)
        out = _native.wf_forward(w, f, idx)
        assert out.shape == (b, n, 4, 64) and (out == 0).all()
        d_q, d_k = _native.qk_backward(torch.zeros_like(attn), q, q, idx)
        assert d_q.shape == q.shape and (d_q == 0).all() and (d_k == 0).all()


def test_copy_probe(device):
    import probe
    src = torch.randn(1 << 20, device=device)
    dst = torch.zeros_like(src)
    probe.copy_probe(src, dst)
    assert torch.equal(src, dst)


def test_replay_probes_run_at_the_operators_shapes(device):
    """The measurement kernels (the forward kernels without their arithmetic) live in their own library and take the
    operators' arguments; their outputs mean nothing, so only shapes and a clean launch are checked."""
    import probe
    case = wl.attn_case("replay", 77, B=2, H=2, N=200, C=32).to(device)
    attn = _native.qk_forward(case.query, case.key, case.nbhd_idx)
    assert probe.qk_forward_replay(case.query, case.key, case.nbhd_idx).shape == attn.shape
    assert probe.av_forward_replay(attn, case.value, case.nbhd_idx).shape == case.value.shape
    w = wl.wf_case("replay_wf", 78, B=2, N=200, C=64).to(device)
    assert probe.wf_forward_replay(w.weights, w.feat, w.nbhd_idx).shape == (2, 50, 4, 64)
    torch.cuda.synchronize()


def test_debug_index_check_on_the_device_and_no_synchronisation_without_it(device, monkeypatch):
    """With CLUSTEN_DEBUG_INDICES=1 a stray index raises before any kernel is launched (QK / AV lists against the
    token count, WF lists against the rows of feat); without it nothing is read back: the three forwards can be
    recorded into a HIP graph, which a host read of device memory would break."""
    case = wl.attn_case("dbg", 79, B=2, H=2, N=64, C=32).to(device)
    w = wl.wf_case("dbg_wf", 80, B=2, N=64, C=64).to(device)
    monkeypatch.setenv("CLUSTEN_DEBUG_INDICES", "1")
    attn = _native.qk_forward(case.query, case.key, case.nbhd_idx)      # good lists pass
    bad = case.nbhd_idx.clone()
    bad[1, 5, 7] = 64
    with pytest.raises(RuntimeError, match=r"outside \[0, 64\)"):
        _native.qk_forward(case.query, case.key, bad)
    with pytest.raises(RuntimeError, match=r"outside \[0, 64\)"):
        _native.av_forward(attn, case.value, bad)
    wbad = w.nbhd_idx.clone()
    wbad[0, 0, 0] = -1
    with pytest.raises(RuntimeError, match="min -1"):
        _native.wf_forward(w.weights, w.feat, wbad)
    assert int(w.nbhd_idx.max()) >= w.weights.shape[1]                  # WF lists exceed Nout and are fine: they index feat
    _native.wf_forward(w.weights, w.feat, w.nbhd_idx)
    monkeypatch.delenv("CLUSTEN_DEBUG_INDICES")

    def step():
        a_ = _native.qk_forward(case.query, case.key, case.nbhd_idx)
        return a_, _native.av_forward(a_, case.value, case.nbhd_idx), _native.wf_forward(w.weights, w.feat, w.nbhd_idx)

    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        a, f, o = step()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(a, attn)
    assert torch.equal(f, _native.av_forward(attn, case.value, case.nbhd_idx))
    assert torch.equal(o, _native.wf_forward(w.weights, w.feat, w.nbhd_idx))
