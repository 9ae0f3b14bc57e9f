"""GPU parity of the one-kernel local attention (`clusten_cluster_attention_forward`) against the composition
of the CPU gather oracles and the tensor expressions the reference model writes between its two operators
(models/aff_transformer.py:120-155), evaluated in fp32 from the same rounded inputs.

Bar: max|x - ref| / max|ref| <= 1e-2 (16-bit data; the probabilities are rounded to the storage type before they
weigh the values, the output is rounded once).
"""
import pytest
import torch

from clusten import _native
from conftest import TOL
from oracle import clusten_oracle as oracle

pytestmark = pytest.mark.gpu

C, NNC, M = 32, 6, 48


def _cluster_numbers(b, n, gen, kind, cs=8):
    """(B,N,6) int32 cluster numbers out of ceil(N/cs) clusters (the last may be short: its pad slots list row 0)."""
    k = (n + cs - 1) // cs
    own = torch.arange(n) // cs
    if kind == "shared":        # the 8 tokens of a cluster list the same clusters
        per = torch.stack([torch.randperm(k, generator=gen)[:NNC] for _ in range(b * k)]).reshape(b, k, NNC)
        return per[:, own].to(torch.int32).contiguous()
    width = k if kind == "scattered" else min(12, k)       # scattered: up to 48 distinct clusters per tile
    lo = torch.zeros(n, dtype=torch.int64) if kind == "scattered" else (own - width // 2).clamp(0, k - width)
    pick = torch.rand(b, n, width, generator=gen).argsort(dim=2)[:, :, :NNC] + lo.view(1, n, 1)
    if kind == "repeated":      # a cluster listed twice by a token
        pick[:, :, 3] = pick[:, :, 1]
    return pick.to(torch.int32).contiguous()


def _expand(cidx, n, cs=8):
    rows = cidx.long().unsqueeze(3) * cs + torch.arange(cs)
    rows = torch.where((rows < n) & (rows >= 0), rows, torch.zeros_like(rows))
    return rows.reshape(cidx.shape[0], cidx.shape[1], -1).contiguous()


def _reference(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, scale):
    """fp32 evaluation of the model's attention on the expanded lists; returns (B,N,H*C)."""
    b, h, n, c = q.shape
    q, k, v, table = q.float(), k.float(), v.float(), table.float()
    attn = oracle.qk_gather_chunked(q, k, idx) * scale                      # (b,h,n,m)
    attn = attn + table[pe_idx].permute(0, 3, 1, 2)
    if mask is not None:
        attn = attn + (1 - mask.reshape(b, 1, n, -1)) * (-100.0)
    blank = (q * blank_k.reshape(1, h, 1, c)).sum(-1, keepdim=True) * scale
    p = torch.softmax(torch.cat([attn, blank], dim=-1), dim=-1)
    out = oracle.av_gather_chunked(p[..., :-1].contiguous(), v, idx) + p[..., -1:] * blank_v.reshape(1, h, 1, c)
    return out.permute(0, 2, 1, 3).reshape(b, n, h * c)


def _case(b, h, n, gen, kind, dtype, with_mask, rows=97, cs=8):
    m = NNC * cs
    q = torch.randn(b, h, n, C, generator=gen).to(dtype)
    k = torch.randn(b, h, n, C, generator=gen).to(dtype)
    v = torch.randn(b, h, n, C, generator=gen).to(dtype)
    cidx = _cluster_numbers(b, n, gen, kind, cs)
    table = torch.randn(rows, h, generator=gen).to(dtype)
    pe_idx = torch.randint(rows, (b, n, m), generator=gen)
    idx = _expand(cidx, n, cs)
    mask = None
    if with_mask:
        # pad slots of a short last cluster are masked, as the model's cluster mask does, plus a few others
        mask = ((cidx.long().unsqueeze(3) * cs + torch.arange(cs)) < n).reshape(b, n, m).long()
        mask = mask * (torch.rand(b, n, m, generator=gen) > 0.05).long()
    blank_k = torch.randn(h * C, generator=gen)
    blank_v = torch.randn(h * C, generator=gen)
    return q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v


def _run(device, case, scale):
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = case
    ref = _reference(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, scale)
    out = _native.cluster_attention(q.to(device), k.to(device), v.to(device), cidx.to(device), table.to(device),
                                    pe_idx.to(device), None if mask is None else mask.to(device),
                                    blank_k.to(device), blank_v.to(device), scale=scale)
    assert out.dtype == q.dtype and out.shape == ref.shape and out.is_contiguous()
    return oracle.rel_err(out, ref)


@pytest.mark.parametrize("kind", ["near", "shared", "scattered", "repeated"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_against_the_oracle_composition(device, kind, dtype):
    gen = torch.Generator().manual_seed(81)
    # 396 = 49 whole clusters and one of 4 tokens (a partial tile whose pad rows list row 0); 64: few clusters
    for b, h, n in ((2, 3, 396), (1, 1, 64), (3, 4, 200)):
        for with_mask in (False, True):
            err = _run(device, _case(b, h, n, gen, kind, dtype, with_mask), scale=C ** -0.5)
            assert err <= TOL[dtype], "%s %s n=%d mask=%s rel err %.3g" % (kind, dtype, n, with_mask, err)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_on_the_lists_and_position_indices_the_benchmark_measures(device, dtype):
    """The benchmark's attention legs take lists and position indices from `workloads.model_built_geometry` (tokens
    on a canvas, clustered as the model clusters them, indices = offsets between positions): the same generator at a
    small batch, through the tensors and through a plan, per-tile kernel and the one for short sequences, against the
    oracle composition; clusters of 8 in all three types, clusters of 24 in the 16-bit ones."""
    import workloads as wl
    d = lambda x: None if x is None else x.to(device)
    gen = torch.Generator().manual_seed(97)
    for cs, b, h, n in ((8, 2, 2, 784), (8, 64, 8, 196), (8, 2, 4, 100), (24, 2, 4, 600)):   # (64 x 8 heads: the short-sequence kernel)
        if cs == 24 and dtype == torch.float32:
            continue
        idx, pe_idx, rows = wl.model_built_geometry(b, n, wl.generator(41), cluster=cs, nnc=NNC)
        cidx = (idx[:, :, ::cs] // cs).to(torch.int32).contiguous()
        # the pad slots of a short last cluster hold row 0 in the lists; as cluster numbers they are the last cluster
        assert torch.equal(_expand(cidx, n, cs), idx)
        q, k, v = (torch.randn(b, h, n, C, generator=gen).to(dtype) for _ in range(3))
        table = torch.randn(rows, h, generator=gen).to(dtype)
        blank_k, blank_v = torch.randn(h * C, generator=gen), torch.randn(h * C, generator=gen)
        mask = ((cidx.long().unsqueeze(3) * cs + torch.arange(cs)) < n).reshape(b, n, NNC * cs).long() if n % cs else None
        ref = _reference(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, C ** -0.5)
        out = _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), d(mask), d(blank_k), d(blank_v),
                                        scale=C ** -0.5)
        err = oracle.rel_err(out, ref)
        assert err <= TOL[dtype], "clusters of %d, n=%d, %s: rel err %.3g" % (cs, n, dtype, err)
        plan = _native.cluster_attention_plan(d(cidx), d(pe_idx), d(mask))
        planned = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                            scale=C ** -0.5, plan=plan)
        assert torch.equal(planned, out)


@pytest.mark.parametrize("kind", ["near", "shared", "scattered", "repeated"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_clusters_of_24_against_the_oracle_composition(device, kind, dtype):
    """Clusters of 24 tokens, the members of the 6 nearest = 144 neighbours (the 384 x 384 models,
    configs/aff_base_22kto1k_384.yaml:10-11): three runs of 8 rows per cluster, two or three passes per head on lists
    like the model's, up to twelve on lists with nothing in common.  With and without a mask, a short last cluster
    (400 = 16 clusters and one of 16 tokens; 148: a last cluster of 4), partial tiles, through the tensors and through
    a plan (bit-equal), per-image lists and one image's lists for the batch."""
    gen = torch.Generator().manual_seed(91)
    d = lambda x: None if x is None else x.to(device)
    for b, h, n in ((2, 3, 400), (1, 2, 148), (2, 4, 192)):
        for with_mask in (False, True):
            case = _case(b, h, n, gen, kind, dtype, with_mask, cs=24)
            q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = case
            assert idx.shape == (b, n, 144)
            ref = _reference(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, C ** -0.5)
            out = _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), d(mask), d(blank_k),
                                            d(blank_v), scale=C ** -0.5)
            err = oracle.rel_err(out, ref)
            assert err <= TOL[dtype], "%s %s n=%d mask=%s rel err %.3g" % (kind, dtype, n, with_mask, err)
            plan = _native.cluster_attention_plan(d(cidx), d(pe_idx), d(mask))
            assert plan.numel() == _native.load().clusten_cluster_attention_plan_bytes(b, n, 144)
            planned = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                                scale=C ** -0.5, plan=plan)
            assert torch.equal(planned, out)
    # one image's lists for the whole batch
    b, h, n = 3, 2, 240
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, kind, dtype, True, cs=24)
    c1, p1, m1 = cidx[:1].contiguous(), pe_idx[:1].contiguous(), mask[:1].contiguous()
    full = _native.cluster_attention(d(q), d(k), d(v), d(c1.expand(b, -1, -1).contiguous()), d(table),
                                     d(p1.expand(b, -1, -1).contiguous()), d(m1.expand(b, -1, -1).contiguous()),
                                     d(blank_k), d(blank_v), scale=0.25)
    shared = _native.cluster_attention(d(q), d(k), d(v), d(c1), d(table), d(p1), d(m1), d(blank_k), d(blank_v), scale=0.25)
    assert torch.equal(shared, full)
    plan1 = _native.cluster_attention_plan(d(c1), d(p1), d(m1))
    assert torch.equal(_native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                                 scale=0.25, plan=plan1), full)
    # fp32 data has no kernel for clusters of 24
    assert not _native.cluster_attention_supported(d(q).float(), 6, 24) and _native.cluster_attention_supported(d(q), 6, 24)
    with pytest.raises(RuntimeError):
        _native.cluster_attention(d(q).float(), d(k).float(), d(v).float(), d(c1), d(table), d(p1), d(m1), d(blank_k),
                                  d(blank_v))


def test_clusters_of_24_equal_the_operators_on_the_expanded_lists(device):
    """The same attention through QK on the 144-slot lists, the softmax kernel and AV (the path the 384 x 384 models took
    before): equal within the 16-bit tolerance."""
    gen = torch.Generator().manual_seed(92)
    b, h, n = 2, 4, 480
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "near", torch.float16, True, cs=24)
    d = lambda x: x.to(device)
    attn = _native.qk_forward(d(q), d(k), d(idx))
    probs, blank = _native.attn_softmax(attn, d(table), d(pe_idx), d(mask), query=d(q), blank_key=d(blank_k))
    three = _native.av_forward(probs.to(torch.float16), d(v), d(idx)).float() + blank * d(blank_v).reshape(1, h, 1, C)
    three = three.permute(0, 2, 1, 3).reshape(b, n, h * C)
    one = _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), d(mask), d(blank_k), d(blank_v))
    assert oracle.rel_err(one.float().cpu(), three.cpu()) <= TOL[torch.float16]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_strided_operands_and_unit_scale(device, dtype):
    """q / k / v as the views a fused qkv projection leaves (channel stride 1, token stride 3*H*C)."""
    gen = torch.Generator().manual_seed(82)
    b, h, n = 2, 2, 136
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "near", dtype, True)
    packed = torch.stack([q, k, v], dim=0).permute(1, 3, 0, 2, 4).contiguous()        # (b, n, 3, h, c)
    views = packed.to(device).permute(2, 0, 3, 1, 4)                                  # (3, b, h, n, c) views
    assert not views[0].is_contiguous()
    ref = _reference(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, 1.0)
    out = _native.cluster_attention(views[0], views[1], views[2], cidx.to(device), table.to(device), pe_idx.to(device),
                                    mask.to(device), blank_k.to(device), blank_v.to(device))
    assert oracle.rel_err(out, ref) <= TOL[dtype]


def test_equals_the_three_kernel_path(device):
    """Same lists through qk_forward_clusters + attn_softmax + av_forward_clusters."""
    gen = torch.Generator().manual_seed(83)
    b, h, n = 2, 2, 392
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "near", torch.float16, True)
    d = lambda x: x.to(device)
    attn = _native.qk_forward_clusters(d(q), d(k), d(cidx))
    probs, blank = _native.attn_softmax(attn, d(table), d(pe_idx), d(mask), query=d(q), blank_key=d(blank_k))
    three = _native.av_forward_clusters(probs, d(v), d(cidx)) + blank * d(blank_v).reshape(1, h, 1, C)
    three = three.permute(0, 2, 1, 3).reshape(b, n, h * C)
    one = _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), d(mask), d(blank_k), d(blank_v))
    assert oracle.rel_err(one.float().cpu(), three.float().cpu()) <= TOL[torch.float16]


def test_unsupported_cases_are_refused(device):
    gen = torch.Generator().manual_seed(84)
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(1, 2, 64, gen, "near", torch.float16, False)
    d = lambda x: x.to(device)
    assert _native.cluster_attention_supported(d(q), 6)
    assert _native.cluster_attention_supported(d(q).float(), 6)
    assert not _native.cluster_attention_supported(d(q).double(), 6)
    assert not _native.cluster_attention_supported(d(q), 8)
    assert not _native.cluster_attention_supported(q, 6)
    with pytest.raises(RuntimeError):       # fp64 has no fused kernel
        _native.cluster_attention(d(q).double(), d(k).double(), d(v).double(), d(cidx), d(table), d(pe_idx), None,
                                  d(blank_k), d(blank_v))
    with pytest.raises(RuntimeError):       # CPU tensors
        _native.cluster_attention(q, k, v, cidx, table, pe_idx, None, blank_k, blank_v)
    empty = _native.cluster_attention(d(q)[:0], d(k)[:0], d(v)[:0], d(cidx)[:0], d(table), d(pe_idx)[:0], None,
                                      d(blank_k), d(blank_v))
    assert empty.shape == (0, 64, 2 * C)


def test_lists_shared_by_the_batch(device):
    """(1,N,.) lists (the tokens of a regular grid) give what their batch-sized copies give."""
    gen = torch.Generator().manual_seed(85)
    b, h, n = 3, 2, 200
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "near", torch.float16, True)
    d = lambda x: x.to(device)
    c1, p1, m1 = cidx[:1].contiguous(), pe_idx[:1].contiguous(), mask[:1].contiguous()
    full = _native.cluster_attention(d(q), d(k), d(v), d(c1.expand(b, -1, -1).contiguous()), d(table),
                                     d(p1.expand(b, -1, -1).contiguous()), d(m1.expand(b, -1, -1).contiguous()),
                                     d(blank_k), d(blank_v), scale=0.25)
    shared = _native.cluster_attention(d(q), d(k), d(v), d(c1), d(table), d(p1), d(m1), d(blank_k), d(blank_v), scale=0.25)
    assert torch.equal(shared, full)
    no_mask = _native.cluster_attention(d(q), d(k), d(v), d(c1), d(table), d(p1), None, d(blank_k), d(blank_v))
    assert no_mask.shape == full.shape and torch.isfinite(no_mask.float()).all()
    with pytest.raises(RuntimeError):       # shared cluster numbers need shared pe_idx
        _native.cluster_attention(d(q), d(k), d(v), d(c1), d(table), d(pe_idx), None, d(blank_k), d(blank_v))


def test_cluster_numbers_out_of_range_read_row_zero(device):
    """Negative numbers and numbers past the last cluster list row 0, as the expanded lists of the operators do."""
    gen = torch.Generator().manual_seed(86)
    b, h, n = 2, 2, 100                                   # 12 whole clusters and one of 4 tokens
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "near", torch.float16, False)
    wild = cidx.clone()
    hit = torch.rand(wild.shape, generator=gen) < 0.1
    wild[hit] = torch.tensor([-1, -7, 13, 500, 1 << 20], dtype=torch.int32)[torch.randint(5, (int(hit.sum()),), generator=gen)]
    idx = _expand(wild, n)
    assert (idx == 0).sum() > hit.sum()
    ref = _reference(q, k, v, idx, table, pe_idx, None, blank_k, blank_v, 0.2)
    d = lambda x: x.to(device)
    out = _native.cluster_attention(d(q), d(k), d(v), d(wild), d(table), d(pe_idx), None, d(blank_k), d(blank_v), scale=0.2)
    assert oracle.rel_err(out, ref) <= TOL[torch.float16]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("kind", ["near", "shared", "scattered", "repeated"])
def test_plan_built_once_gives_the_same_bits(device, kind, dtype):
    """What the kernel works out from the index tensors, handed over as a plan (one per stage, read by every layer):
    the result is bit-equal to the call that reads the tensors, for every kind of list, with and without a mask, on
    partial tiles, and for lists shared by the batch."""
    gen = torch.Generator().manual_seed(87)
    d = lambda x: None if x is None else x.to(device)
    for b, h, n in ((2, 3, 396), (1, 1, 64), (3, 4, 200)):
        for with_mask in (False, True):
            q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, kind, dtype, with_mask)
            plain = _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), d(mask), d(blank_k),
                                              d(blank_v), scale=0.2)
            plan = _native.cluster_attention_plan(d(cidx), d(pe_idx), d(mask))
            assert plan.dtype == torch.uint8 and plan.numel() == _native.load().clusten_cluster_attention_plan_bytes(b, n, 48)
            for _ in range(2):      # the plan serves any number of calls
                planned = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                                    scale=0.2, plan=plan)
                assert torch.equal(planned, plain)
    # one image's lists for the whole batch
    b, h, n = 3, 2, 200
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, kind, torch.bfloat16 if dtype == torch.float16 else dtype, True)
    c1, p1, m1 = cidx[:1].contiguous(), pe_idx[:1].contiguous(), mask[:1].contiguous()
    plain = _native.cluster_attention(d(q), d(k), d(v), d(c1), d(table), d(p1), d(m1), d(blank_k), d(blank_v))
    plan1 = _native.cluster_attention_plan(d(c1), d(p1), d(m1))
    assert torch.equal(_native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                                 plan=plan1), plain)
    with pytest.raises(RuntimeError):       # a plan of other lists
        _native.cluster_attention(d(q)[:, :, :64], d(k)[:, :, :64], d(v)[:, :, :64], None, d(table), None, None,
                                  d(blank_k), d(blank_v), plan=plan1)


@pytest.mark.parametrize("kind", ["near", "scattered", "repeated"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_short_sequences_with_the_rows_of_a_head_resident_in_lds(device, kind, dtype):
    """512 or more (image, head) pairs of at most 256 tokens go to the kernel that keeps the K and V rows of a head in
    LDS (the 196-token stage of the 224 x 224 models): against the oracle composition, and bit for bit against the same
    images computed a quarter of the batch at a time, which the kernel with one workgroup per tile takes - with and
    without plan, masks, a short last cluster (196 = 24 clusters and 4 tokens), the training forward's denominators."""
    gen = torch.Generator().manual_seed(95)
    d = lambda x: None if x is None else x.to(device)
    scale = C ** -0.5
    for b, h, n, with_mask in ((64, 8, 196, True), (128, 4, 104, False), (32, 16, 250, True)):
        q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, kind, dtype, with_mask)
        ref = _reference(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, scale)
        out = _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), d(mask), d(blank_k), d(blank_v),
                                        scale=scale)
        what = "%s %s b=%d h=%d n=%d" % (kind, dtype, b, h, n)
        assert oracle.rel_err(out, ref) <= TOL[dtype], what
        plan = _native.cluster_attention_plan(d(cidx), d(pe_idx), d(mask))
        planned, lse = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                                 scale=scale, plan=plan, return_lse=True)
        assert torch.equal(planned, out), what
        quarter = b // 4
        parts, lses = [], []
        for lo in range(0, b, quarter):
            sl = slice(lo, lo + quarter)
            assert quarter * h < 512
            pl = _native.cluster_attention_plan(d(cidx[sl]), d(pe_idx[sl]), d(None if mask is None else mask[sl]))
            o, l = _native.cluster_attention(d(q[sl]), d(k[sl]), d(v[sl]), None, d(table), None, None, d(blank_k),
                                             d(blank_v), scale=scale, plan=pl, return_lse=True)
            parts.append(o)
            lses.append(l)
        assert torch.equal(torch.cat(parts), out), what
        assert torch.equal(torch.cat(lses), lse), what


def _reference_grads(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, scale, d_out):
    """Gradients of `_reference` by autograd, in fp32 from the same rounded inputs."""
    b, h, n, c = q.shape
    leaves = [t.float().clone().requires_grad_(True) for t in (q, k, v, table, blank_k, blank_v)]
    qf, kf, vf, tf, bkf, bvf = leaves
    rows = idx[:, None, :, :, None].expand(b, h, n, idx.shape[2], c)
    kg = kf[:, :, :, None, :].expand(b, h, n, idx.shape[2], c).gather(2, rows)           # (b,h,n,m,c)
    vg = vf[:, :, :, None, :].expand(b, h, n, idx.shape[2], c).gather(2, rows)
    attn = (qf[:, :, :, None, :] * kg).sum(-1) * scale + tf[pe_idx].permute(0, 3, 1, 2)
    if mask is not None:
        attn = attn + (1 - mask.reshape(b, 1, n, -1)) * (-100.0)
    blank = (qf * bkf.reshape(1, h, 1, c)).sum(-1, keepdim=True) * scale
    p = torch.softmax(torch.cat([attn, blank], dim=-1), dim=-1)
    out = (p[..., :-1, None] * vg).sum(3) + p[..., -1:] * bvf.reshape(1, h, 1, c)
    out = out.permute(0, 2, 1, 3).reshape(b, n, h * c)
    out.backward(d_out.float())
    return [t.grad for t in leaves]


@pytest.mark.parametrize("kind", ["near", "shared", "scattered", "repeated"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_backward_against_autograd_through_the_composition(device, kind, dtype):
    """`cluster_attention_backward` (d_query, the recomputed probabilities and the logit gradients in one kernel) with
    the sums that complete it - the scatters over sorted pair lists, the bias table's gradient, the blank token's -
    against autograd through the fp32 composition, with a random upstream gradient."""
    gen = torch.Generator().manual_seed(88)
    d = lambda x: None if x is None else x.to(device)
    scale = C ** -0.5
    for b, h, n in ((2, 3, 392), (1, 1, 64), (2, 4, 396)):
        for with_mask in (False, True):
            q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, kind, dtype, with_mask)
            d_out = torch.randn(b, n, h * C, generator=gen).to(dtype)
            ref = _reference_grads(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, scale, d_out)
            plan = _native.cluster_attention_plan(d(cidx), d(pe_idx), d(mask))
            out, lse = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                                 scale=scale, plan=plan, return_lse=True)
            plain = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                              scale=scale, plan=plan)
            assert torch.equal(out, plain) and lse.shape == (b, h, n) and bool(torch.isfinite(lse).all())
            dq, probs, d_logit, p_b, ds_b = _native.cluster_attention_backward(
                d(q), d(k), d(v), d(d_out), out, lse, plan, d(table), d(blank_k), d(blank_v), scale=scale)
            pairs = _native.cluster_pairs(d(idx))
            assert int(_native.pairs_not_whole(pairs)) == 0
            g_view = d(d_out).view(b, n, h, C).permute(0, 2, 1, 3)
            dv = _native.scatter_rows_by_cluster(probs, g_view.contiguous(), pairs)
            dk = _native.scatter_rows_by_cluster(d_logit, d(q), pairs).float() * scale
            d_table = _native.bias_table_grad(d_logit, d(pe_idx), table.shape[0])
            d_bk = (ds_b.unsqueeze(-1) * d(q).float()).sum((0, 2)).reshape(-1) * scale
            d_bv = (p_b.unsqueeze(-1) * g_view.float()).sum((0, 2)).reshape(-1)
            tol = TOL[dtype]
            what = "%s %s n=%d mask=%s" % (kind, dtype, n, with_mask)
            for name, got, want in (("d_query", dq, ref[0]), ("d_key", dk, ref[1]), ("d_value", dv, ref[2]),
                                    ("d_table", d_table, ref[3]), ("d_blank_key", d_bk, ref[4]),
                                    ("d_blank_value", d_bv, ref[5])):
                err = oracle.rel_err(got.float().cpu(), want)
                assert err <= 2 * tol, "%s %s rel err %.3g" % (name, what, err)


def test_backward_of_tiles_that_take_several_passes_in_bf16(device):
    """Lists with nothing in common (up to 48 distinct clusters per tile: four passes) on short sequences in bf16, where
    delta taken from the saved 16-bit output cost the blank key's gradient several per cent: the kernel adds up p * dP
    over a sweep of its own instead, and every gradient stays within the 16-bit tolerance itself (not twice it)."""
    gen = torch.Generator().manual_seed(93)
    d = lambda x: None if x is None else x.to(device)
    scale = C ** -0.5
    dtype = torch.bfloat16
    for b, h, n in ((4, 2, 64), (2, 2, 128), (2, 3, 392)):
        q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "scattered", dtype, True)
        distinct = max(len(set(cidx[0, 8 * g:8 * g + 8].reshape(-1).tolist())) for g in range(n // 8))
        assert distinct > 12 or n == 64                     # several passes (64 tokens hold 8 clusters: one pass)
        d_out = torch.randn(b, n, h * C, generator=gen).to(dtype)
        ref = _reference_grads(q, k, v, idx, table, pe_idx, mask, blank_k, blank_v, scale, d_out)
        plan = _native.cluster_attention_plan(d(cidx), d(pe_idx), d(mask))
        out, lse = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                             scale=scale, plan=plan, return_lse=True)
        dq, probs, d_logit, p_b, ds_b = _native.cluster_attention_backward(
            d(q), d(k), d(v), d(d_out), out, lse, plan, d(table), d(blank_k), d(blank_v), scale=scale)
        pairs = _native.cluster_pairs(d(idx))
        g_view = d(d_out).view(b, n, h, C).permute(0, 2, 1, 3)
        dv = _native.scatter_rows(probs, g_view, d(idx), pairs)
        dk = _native.scatter_rows(d_logit, d(q), d(idx), pairs).float() * scale
        d_table = _native.bias_table_grad(d_logit, d(pe_idx), table.shape[0])
        d_bk = (ds_b.unsqueeze(-1) * d(q).float()).sum((0, 2)).reshape(-1) * scale
        d_bv = (p_b.unsqueeze(-1) * g_view.float()).sum((0, 2)).reshape(-1)
        for name, got, want in (("d_query", dq, ref[0]), ("d_key", dk, ref[1]), ("d_value", dv, ref[2]),
                                ("d_table", d_table, ref[3]), ("d_blank_key", d_bk, ref[4]),
                                ("d_blank_value", d_bv, ref[5])):
            err = oracle.rel_err(got.float().cpu(), want)
            assert err <= TOL[dtype], "%s n=%d rel err %.3g" % (name, n, err)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_softmax_denominators_of_the_training_forward(device, dtype):
    """`return_lse=True`: the same result bit for bit, and log(sum of exp(logit)) over the 48 neighbours and the
    blank token for every (image, head, token)."""
    gen = torch.Generator().manual_seed(89)
    d = lambda x: None if x is None else x.to(device)
    b, h, n = 2, 3, 204
    scale = C ** -0.5
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "near", dtype, True)
    plan = _native.cluster_attention_plan(d(cidx), d(pe_idx), d(mask))
    out, lse = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                         scale=scale, plan=plan, return_lse=True)
    plain = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                      scale=scale, plan=plan)
    assert torch.equal(out, plain)
    qf, kf, tf = q.float(), k.float(), table.float()
    attn = oracle.qk_gather_chunked(qf, kf, idx) * scale + tf[pe_idx].permute(0, 3, 1, 2)
    attn = attn + (1 - mask.reshape(b, 1, n, -1)) * (-100.0)
    blank = (qf * blank_k.reshape(1, h, 1, C)).sum(-1, keepdim=True) * scale
    want = torch.logsumexp(torch.cat([attn, blank], dim=-1), dim=-1)
    assert lse.shape == (b, h, n) and lse.dtype == torch.float32
    assert float((lse.cpu() - want).abs().max()) <= (1e-4 if dtype == torch.float32 else 2e-3)
    with pytest.raises(RuntimeError):       # the denominators are written by the planned kernel only
        _native.cluster_attention(d(q), d(k), d(v), d(cidx), d(table), d(pe_idx), d(mask), d(blank_k), d(blank_v),
                                  return_lse=True)


def test_backward_with_lists_shared_by_the_batch(device):
    """One image's lists (and plan) for the whole batch, as a grid stage hands them over: the backward kernel gives the
    same bits as with the lists repeated for every image."""
    gen = torch.Generator().manual_seed(90)
    d = lambda x: None if x is None else x.to(device)
    b, h, n = 3, 2, 200
    q, k, v, cidx, idx, table, pe_idx, mask, blank_k, blank_v = _case(b, h, n, gen, "near", torch.float16, True)
    c1, p1, m1 = cidx[:1].contiguous(), pe_idx[:1].contiguous(), mask[:1].contiguous()
    d_out = torch.randn(b, n, h * C, generator=gen).half()
    results = []
    for lists in ((c1, p1, m1), (c1.expand(b, -1, -1).contiguous(), p1.expand(b, -1, -1).contiguous(),
                                  m1.expand(b, -1, -1).contiguous())):
        plan = _native.cluster_attention_plan(d(lists[0]), d(lists[1]), d(lists[2]))
        out, lse = _native.cluster_attention(d(q), d(k), d(v), None, d(table), None, None, d(blank_k), d(blank_v),
                                             plan=plan, return_lse=True)
        results.append((out, lse) + tuple(_native.cluster_attention_backward(
            d(q), d(k), d(v), d(d_out), out, lse, plan, d(table), d(blank_k), d(blank_v))))
    for one, every in zip(*results):
        assert torch.equal(one, every)
