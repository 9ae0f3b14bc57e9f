"""The callers of the operators (ClusterAttention, ClusterMerging, BasicLayer) and the classifier built from them.

On the CPU the modules run on the oracle's gather expressions; on the GPU the same modules, same weights and
same input run once on the HIP operators and once on the oracle, and the logits must agree.
"""
import math
from types import SimpleNamespace

import pytest
import torch

from aff.model import (AutoFocusFormer, BasicLayer, ClusterAttention, ClusterMerging, aff_tiny,
                       relative_position_table)
from oracle import clusten_oracle as oracle


def oracle_ops():
    """The reference wrappers' dtype rule (second operand cast to the first's) around the gather expressions."""
    return SimpleNamespace(
        qk=lambda q, k, idx: oracle.qk_gather(q, k.to(q.dtype), idx),
        av=lambda a, v, idx: oracle.av_gather(a, v.to(a.dtype), idx),
        wf=lambda w, f, idx: oracle.wf_gather(w, f.to(w.dtype), idx))


TOL_16 = 1e-2


def small_model(ops, **kw):
    cfg = dict(embed_dim=(32, 64, 128, 256), depths=(1, 2, 1, 1), num_heads=(2, 4, 8, 16), mlp_ratio=2.0,
               num_classes=10, img_size=128, drop_path_rate=0.0, ops=ops)
    cfg.update(kw)
    torch.manual_seed(0)
    return AutoFocusFormer(**cfg).eval()


def test_relative_position_table_rows():
    table, r = relative_position_table(224)
    assert r == 55 and table.shape == (111 * 111, 5)
    row = lambda dx, dy: table[(dy + r) * 111 + (dx + r)]
    assert row(0, 0).tolist() == [0, 0, 0, 0, 0]
    got = row(3, -4)
    assert torch.allclose(got, torch.tensor([3.0, -4.0, 5.0, -0.8, 0.6]))
    assert torch.isfinite(table).all()


def test_parameter_names_follow_the_reference_layout():
    names = set(small_model(oracle_ops()).state_dict().keys())
    for key in ["patch_embed.proj1.weight", "patch_embed.bn.running_mean", "patch_embed.proj2.bias",
                "patch_embed.norm.weight", "layers.0.blocks.0.norm1.weight", "layers.0.blocks.0.attn.q.weight",
                "layers.0.blocks.0.attn.kv.bias", "layers.0.blocks.0.attn.blank_k", "layers.0.blocks.0.attn.blank_v",
                "layers.0.blocks.0.attn.pos_embed.weight", "layers.0.blocks.0.attn.proj.weight",
                "layers.0.blocks.0.mlp.fc1.weight", "layers.0.blocks.0.mlp.fc2.bias",
                "layers.0.downsample.weight_net.0.weight", "layers.0.downsample.weight_net.1.bias",
                "layers.0.downsample.norm.weight", "layers.0.downsample.linear.weight", "layers.0.prob_net.weight",
                "layers.3.blocks.0.attn.q.weight", "norm.weight", "head.bias"]:
        assert key in names, key
    assert not any(k.startswith("layers.3.downsample") or "pre_table" in k for k in names)


def test_classifier_runs_on_the_oracle_and_is_deterministic():
    model = small_model(oracle_ops())
    x = torch.randn(2, 3, 128, 128, generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        y1, y2 = model(x), model(x)
    assert y1.shape == (2, 10) and torch.isfinite(y1).all()
    assert torch.equal(y1, y2)
    # images of a batch do not interact
    with torch.no_grad():
        y_first = model(x[:1])
    assert torch.allclose(y_first, y1[:1], atol=1e-5)


def test_classifier_trains_through_the_oracle():
    model = small_model(oracle_ops()).train()
    x = torch.randn(2, 3, 128, 128, generator=torch.Generator().manual_seed(2))
    model(x).square().mean().backward()
    missing = [n for n, p in model.named_parameters() if p.grad is None]
    assert missing == []


def _stage_inputs(b, side, c, gen):
    ys, xs = torch.meshgrid(torch.arange(side), torch.arange(side), indexing="ij")
    pos = torch.stack([xs, ys], 2).reshape(1, -1, 2).expand(b, -1, -1).float()
    return pos, torch.randn(b, side * side, c, generator=gen)


def test_neighbourhood_lists_are_runs_of_whole_clusters_nearest_first():
    layer = BasicLayer(32, 64, 8, 48, 1, 2, 2.0, ops=oracle_ops())
    pos, _ = _stage_inputs(2, 14, 32, torch.Generator().manual_seed(0))         # 196 tokens: 25 clusters, 4 pads
    new_pos, ranking, member_idx, mask, pe_idx, cluster_idx = layer.neighbourhoods(pos, 14, 14, 55, 111)
    b, n, m = member_idx.shape
    assert (n, m) == (196, 48) and mask is not None
    runs = member_idx.reshape(b, n, 6, 8)
    start = runs[..., 0]
    full = mask.reshape(b, n, 6, 8).all(-1)
    # a run is cluster g's members 8g..8g+7; in the padded last cluster the pad slots hold 0 and mask 0
    assert torch.equal(runs[full], (start[full][:, None] + torch.arange(8)))
    assert (start % 8 == 0).all()
    padded = runs[~full]
    assert padded.numel() > 0 and (padded[:, :4] == torch.arange(192, 196)).all() and (padded[:, 4:] == 0).all()
    assert (mask.reshape(b, n, 6, 8)[~full][:, 4:] == 0).all()
    # a token's first run is its own cluster or one at least as near
    centres = new_pos.new_zeros(b, 25, 2)
    for g in range(25):
        centres[:, g] = new_pos[:, 8 * g:min(8 * g + 8, 196)].mean(1)
    d_first = (new_pos - centres.gather(1, (start[..., 0] // 8)[..., None].expand(-1, -1, 2))).norm(dim=-1)
    d_own = (new_pos - centres[:, torch.arange(196) // 8]).norm(dim=-1)
    assert (d_first <= d_own + 1e-6).all()
    # the cluster numbers alone describe the lists: row 8g+t of cluster g, row 0 past the last token
    rows = cluster_idx.long().unsqueeze(3) * 8 + torch.arange(8)
    assert cluster_idx.dtype == torch.int32 and cluster_idx.shape == (b, n, 6)
    assert torch.equal(torch.where(rows < n, rows, torch.zeros_like(rows)).reshape(b, n, m), member_idx)
    # position-table index = (dy + R) * width + (dx + R) of neighbour minus token
    nb = new_pos.gather(1, member_idx.reshape(b, -1, 1).expand(-1, -1, 2)).reshape(b, n, m, 2)
    rel = nb - new_pos[:, :, None]
    assert torch.equal(pe_idx, ((rel[..., 1] + 55) * 111 + rel[..., 0] + 55).long())


def test_attention_with_every_token_as_neighbour_equals_the_dense_branch():
    torch.manual_seed(0)
    attn = ClusterAttention(32, 2, ops=oracle_ops()).eval()
    table, r = relative_position_table(64)
    b, n = 2, 24
    feat = torch.randn(b, n, 32)
    pos = torch.stack([torch.randperm(225)[:n] for _ in range(b)])
    pos = torch.stack([pos % 15, pos // 15], 2).float()
    rel = (pos[:, None] + r) - pos[:, :, None]
    pe_idx = (rel[..., 1] * (2 * r + 1) + rel[..., 0]).long()
    member_idx = torch.arange(n).expand(b, n, n).contiguous()
    with torch.no_grad():
        local = attn(feat, member_idx, None, pe_idx, False, table)
        dense = attn(feat, None, None, pe_idx, True, table)
    assert torch.allclose(local, dense, atol=1e-5)
    # masked neighbours get no weight: masking a column equals removing it
    mask = torch.ones(b, n, n, dtype=torch.int64)
    mask[:, :, -3:] = 0
    with torch.no_grad():
        masked = attn(feat, member_idx, mask, pe_idx, False, table)
        dropped = attn(feat, member_idx[:, :, :-3].contiguous(), None, pe_idx[:, :, :-3], False, table)
    assert torch.allclose(masked, dropped, atol=1e-5)


def test_merging_keeps_a_quarter_with_reserved_tokens_last_and_orders_channels_ic_major():
    torch.manual_seed(0)
    ops = oracle_ops()
    layer = BasicLayer(16, 32, 8, 48, 1, 2, 2.0, ops=ops).eval()
    table, r = relative_position_table(64)
    pos, feat = _stage_inputs(2, 16, 16, torch.Generator().manual_seed(4))
    new_pos, ranking, member_idx, mask, pe_idx, _ = layer.neighbourhoods(pos, 16, 16, r, 2 * r + 1)
    feat = feat.gather(1, ranking.expand(-1, -1, 16))
    merge = layer.downsample
    prob = torch.rand(2, 256, 1)
    centre = merge.select(new_pos, prob, 2, 16)
    assert centre.shape == (2, 64)
    for b in range(2):
        assert len(set(centre[b].tolist())) == 64
        kept = new_pos[b, centre[b, -16:]]
        assert (kept % 4 == 0).all() and len({tuple(p.tolist()) for p in kept}) == 16
        assert centre[b, -16:].tolist() == sorted(centre[b, -16:].tolist())
        # the sampled ones are the best-scored unreserved tokens
        score = ((new_pos[b] % 2).sum(-1) == 0).float() + 4.0 * prob[b, :, 0]
        score[(new_pos[b] % 4).sum(-1) == 0] -= 100
        assert set(centre[b, :48].tolist()) == set(score.topk(48)[1].tolist())
    with torch.no_grad():
        out_pos, out = merge(new_pos, feat, member_idx, mask, prob, 2, pe_idx, 16, table)
        # the same merge spelled out: out[b,i, ic*c + ch] = sum_j w[b,i,j,ic] * feat[b, idx[b,i,j], ch]
        rows = centre.unsqueeze(2).expand(-1, -1, 48)
        idx = member_idx.gather(1, rows)
        w = merge.weight_net(table)[pe_idx.gather(1, rows)] * prob.gather(1, idx.reshape(2, -1, 1)).reshape(2, 64, 48, 1)
        g = feat.gather(1, idx.reshape(2, -1, 1).expand(-1, -1, 16)).reshape(2, 64, 48, 16)
        flat = torch.einsum("bijk,bijc->bikc", w, g).reshape(2, 64, 64)
        assert torch.allclose(out, merge.linear(merge.norm(flat)), atol=1e-5)
    assert torch.equal(out_pos, new_pos.gather(1, centre.unsqueeze(2).expand(-1, -1, 2)))


# ----------------------------------------------------------------------------------------------- GPU

@pytest.mark.gpu
@pytest.mark.parametrize("amp", [False, True])
def test_logits_equal_with_hip_operators_and_with_the_oracle(device, amp):
    from aff.model import default_ops
    hip = small_model(default_ops(), img_size=128, num_classes=16).to(device)
    ref = small_model(oracle_ops(), img_size=128, num_classes=16).to(device)
    ref.load_state_dict(hip.state_dict())
    x = torch.randn(4, 3, 128, 128, generator=torch.Generator().manual_seed(7)).to(device)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16, enabled=amp):
        y_hip, y_ref = hip(x), ref(x)
    assert torch.isfinite(y_hip).all()
    tol = 2e-2 if amp else 1e-4
    assert oracle.rel_err(y_hip.float(), y_ref.float()) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("amp", [False, True])
def test_clusters_of_24_with_144_neighbours_as_in_the_384_models(device, amp):
    """configs/aff_base_22kto1k_384.yaml:10-11: CLUSTER_SIZE 24, NBHD_SIZE 144.  A 192 x 192 image gives 2304 and 576
    tokens in the first two stages (local attention over 144-slot lists: the kernels for long runs, the softmax kernel
    with a wave per token) and 144 / 36 in the last two (global attention).  Logits and parameter gradients against the
    same model on the oracle."""
    from aff.model import default_ops
    kw = dict(img_size=192, num_classes=12, embed_dim=(64, 128, 256, 512), cluster_size=24, nbhd_size=(144, 144, 144, 144))
    ops = default_ops()
    fused_calls = []
    one_kernel = ops.cluster_attention

    def counted(q, *a, **k):
        fused_calls.append(tuple(q.shape))
        return one_kernel(q, *a, **k)

    ops.cluster_attention = counted
    numbered_calls = []
    qk_numbers = ops.qk_clusters

    def counted_numbers(q, k, cidx, **k2):
        numbered_calls.append((q.shape[2], cidx.shape[2], k2.get("cluster_size", 8)))
        return qk_numbers(q, k, cidx, **k2)

    ops.qk_clusters = counted_numbers
    hip = small_model(ops, **kw).to(device)
    ref = small_model(oracle_ops(), **kw).to(device)
    ref.load_state_dict(hip.state_dict())
    x = torch.randn(2, 3, 192, 192, generator=torch.Generator().manual_seed(17)).to(device)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16, enabled=amp):
        y_hip, y_ref = hip(x), ref(x)
    assert torch.isfinite(y_hip).all()
    assert oracle.rel_err(y_hip.float(), y_ref.float()) < (2e-2 if amp else 1e-4)
    if amp:
        # under mixed precision the local attention of the first two stages (1 + 2 blocks) ran as one kernel each
        assert [s[2] for s in fused_calls] == [2304, 576, 576] and all(s[3] == 32 for s in fused_calls)
        return
    # fp32 data: clusters of 24 go through the three operators, in inference on (b,n,6) cluster numbers
    assert not fused_calls and numbered_calls == [(2304, 6, 24), (576, 6, 24), (576, 6, 24)]
    hip.train(), ref.train()
    target = torch.randn(2, 12, generator=torch.Generator().manual_seed(18)).to(device)
    for model in (hip, ref):
        ((model(x) - target) ** 2).mean().backward()
    for (name, p), (_, q) in zip(hip.named_parameters(), ref.named_parameters()):
        assert p.grad is not None and torch.isfinite(p.grad).all(), name
        assert float((p.grad - q.grad).abs().max()) <= 1e-3 * float(q.grad.abs().max()) + 1e-7, name


@pytest.mark.gpu
@pytest.mark.parametrize("embed_dim", [(32, 64, 128, 256), (64, 128, 256, 512)])
def test_parameter_gradients_with_the_cluster_by_cluster_backward(device, monkeypatch, embed_dim):
    """A training step of the model with the backward scatters (d_key, d_value, WF d_feat) running as gathers over
    sorted pair lists — the model's own lists are made of whole clusters — against the same step on the oracle,
    at head dim 16 and 32."""
    from aff.model import default_ops
    from clusten import _native
    seen = {"qk": [], "av": [], "wf": []}

    def watched(name, fn, n_rows):
        def call(*a):
            block = _native.cluster_pairs(a[3], n_rows(a))
            seen[name].append(block is not None and int(_native.pairs_not_whole(block)) == 0)
            return fn(*a)
        return call

    monkeypatch.setattr(_native, "qk_backward", watched("qk", _native.qk_backward, lambda a: None))
    monkeypatch.setattr(_native, "av_backward", watched("av", _native.av_backward, lambda a: None))
    monkeypatch.setattr(_native, "wf_backward", watched("wf", _native.wf_backward, lambda a: a[2].shape[1]))
    ops = dict(vars(default_ops()))
    ops.pop("cluster_attention_backward")      # the three operators, not the one-kernel attention (head dim 32 would take it)
    hip = small_model(SimpleNamespace(**ops), img_size=128, num_classes=16, embed_dim=embed_dim).to(device).train()
    ref = small_model(oracle_ops(), img_size=128, num_classes=16, embed_dim=embed_dim).to(device).train()
    ref.load_state_dict(hip.state_dict())
    x = torch.randn(4, 3, 128, 128, generator=torch.Generator().manual_seed(8)).to(device)
    target = torch.randn(4, 16, generator=torch.Generator().manual_seed(9)).to(device)
    for model in (hip, ref):
        ((model(x) - target) ** 2).mean().backward()
    # every local attention layer and every merge handed over lists made of whole clusters
    for name, flags in seen.items():
        assert flags and all(flags), "%s: %s" % (name, flags)
    for (name, p), (_, q) in zip(hip.named_parameters(), ref.named_parameters()):
        assert p.grad is not None and torch.isfinite(p.grad).all(), name
        # 1e-7: the bias ahead of the BatchNorm has a gradient of zero, both sides hold rounding noise there
        assert float((p.grad - q.grad).abs().max()) <= 1e-3 * float(q.grad.abs().max()) + 1e-7, name


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("with_mask", [False, True])
def test_fused_bias_mask_blank_softmax_equals_the_tensor_expressions(device, dtype, with_mask):
    from clusten import _native
    gen = torch.Generator().manual_seed(11)
    b, h, n, m, rows = 3, 4, 197, 48, 111 * 111
    attn = (torch.randn(b, h, n, m, generator=gen) * 2).to(dtype).to(device)
    table = torch.randn(rows, h, generator=gen).to(dtype).to(device)
    pe_idx = torch.randint(rows, (b, n, m), generator=gen).to(device)
    blank = torch.randn(b, h, n, 1, generator=gen).to(device)
    mask = None
    if with_mask:
        mask = (torch.rand(b, n, m, generator=gen) > 0.2).long().to(device)
        mask[0, 5] = 0                      # a token whose neighbours are all padding: only the blank token is left
    probs, blank_p = _native.attn_softmax(attn, table, pe_idx, mask, blank)
    # aff_transformer.py:122-147 in fp32 from the same rounded inputs
    logits = attn.float() + table.float()[pe_idx].permute(0, 3, 1, 2)
    if mask is not None:
        logits = logits + (1 - mask.reshape(b, 1, n, m)) * (-100)
    ref = torch.softmax(torch.cat([logits, blank], dim=-1), dim=-1)
    assert probs.dtype == torch.float32 and probs.shape == (b, h, n, m) and blank_p.shape == (b, h, n, 1)
    assert oracle.rel_err(probs, ref[..., :-1]) < 1e-5
    assert oracle.rel_err(blank_p, ref[..., -1:]) < 1e-5
    assert torch.allclose(probs.sum(-1, keepdim=True) + blank_p, torch.ones_like(blank_p), atol=1e-5)
    # the blank logit computed in the same pass from a (permuted-view) query and the blank key
    c = 32
    qsrc = (torch.randn(b, n, h, c, generator=gen) * 0.3).to(dtype).to(device)
    query = qsrc.permute(0, 2, 1, 3)
    blank_key = torch.randn(h * c, generator=gen).to(device)
    probs_q, blank_q = _native.attn_softmax(attn, table, pe_idx, mask, query=query, blank_key=blank_key)
    blank_ref = (query.float() * blank_key.reshape(1, h, 1, c)).sum(-1, keepdim=True)
    ref_q = torch.softmax(torch.cat([logits, blank_ref], dim=-1), dim=-1)
    assert oracle.rel_err(probs_q, ref_q[..., :-1]) < 1e-5 and oracle.rel_err(blank_q, ref_q[..., -1:]) < 1e-5
    # the 144 neighbours of the 384 x 384 models (configs/aff_base_22kto1k_384.yaml:11): a wave per token
    m3 = 144
    attn3 = (torch.randn(2, h, 50, m3, generator=gen) * 2).to(dtype).to(device)
    pe3 = torch.randint(rows, (2, 50, m3), generator=gen).to(device)
    mask3 = (torch.rand(2, 50, m3, generator=gen) > 0.2).long().to(device) if with_mask else None
    q3 = (torch.randn(2, 50, h, c, generator=gen) * 0.3).to(dtype).to(device).permute(0, 2, 1, 3)
    p3, b3 = _native.attn_softmax(attn3, table, pe3, mask3, query=q3, blank_key=blank_key)
    logits3 = attn3.float() + table.float()[pe3].permute(0, 3, 1, 2)
    if mask3 is not None:
        logits3 = logits3 + (1 - mask3.reshape(2, 1, 50, m3)) * (-100)
    ref3 = torch.softmax(torch.cat([logits3, (q3.float() * blank_key.reshape(1, h, 1, c)).sum(-1, keepdim=True)], -1), -1)
    assert oracle.rel_err(p3, ref3[..., :-1]) < 1e-5 and oracle.rel_err(b3, ref3[..., -1:]) < 1e-5
    # ... and the backward of the softmax at that length
    dp, dpb = torch.randn_like(p3), torch.randn_like(b3)
    d_logit, d_blank = _native.attn_softmax_backward(p3, b3, dp, dpb, dtype)
    s3 = (p3 * dp).sum(-1, keepdim=True) + b3 * dpb
    assert oracle.rel_err(d_logit.float(), p3 * (dp - s3)) < (1e-5 if dtype == torch.float32 else 1e-2)
    assert oracle.rel_err(d_blank, b3 * (dpb - s3)) < 1e-5
    # other list lengths, and the refusals
    for m2 in (4, 16, 64, 256):
        p2, b2 = _native.attn_softmax(attn[..., :1].expand(-1, -1, -1, m2).contiguous(), table,
                                      pe_idx[..., :1].expand(-1, -1, m2).contiguous(), None, blank)
        assert torch.allclose(p2.sum(-1, keepdim=True) + b2, torch.ones_like(b2), atol=1e-5)
        assert torch.allclose(p2, p2[..., :1].expand_as(p2))
    assert not _native.attn_softmax_supported(attn, 260) and not _native.attn_softmax_supported(attn, 50)
    with pytest.raises(RuntimeError):
        _native.attn_softmax(attn.cpu(), table, pe_idx, mask, blank)


@pytest.mark.gpu
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_layer_norm_kernel_equals_torch(device, out_dtype):
    """fp32 statistics and affine transform, one rounding to the output type: F.layer_norm in fp32, then .to()."""
    from clusten import _native
    gen = torch.Generator().manual_seed(17)
    for rows, c in (((5, 37), 64), ((3, 200), 128), ((2, 49), 256), ((1, 7), 384), ((4, 13), 512), ((2, 3), 768),
                    ((3, 5), 1024), ((1,), 64)):
        x = (torch.randn(*rows, c, generator=gen) * 3 + 1.5).to(device)
        w = torch.randn(c, generator=gen).to(device)
        b = torch.randn(c, generator=gen).to(device)
        ref = torch.nn.functional.layer_norm(x, (c,), w, b, 1e-5)
        out = _native.layer_norm(x, w, b, 1e-5, out_dtype)
        assert out.dtype == out_dtype and out.shape == x.shape
        if out_dtype == torch.float32:
            assert oracle.rel_err(out, ref) <= 1e-5
        else:
            # the fp32 result rounded once: at most one unit in the last place of the 16-bit type from torch's
            assert oracle.rel_err(out.float(), ref.to(out_dtype).float()) <= (2e-3 if out_dtype == torch.float16 else 1.6e-2)
            assert oracle.rel_err(out.float(), ref) <= TOL_16
        # 16-bit input: widened, as mixed precision does before a normalisation
        for in_dtype in (torch.float16, torch.bfloat16):
            xin = x.to(in_dtype)
            ref16 = torch.nn.functional.layer_norm(xin.float(), (c,), w, b, 1e-5)
            out16 = _native.layer_norm(xin, w, b, 1e-5, out_dtype)
            assert out16.dtype == out_dtype
            assert oracle.rel_err(out16.float(), ref16) <= (1e-5 if out_dtype == torch.float32 else TOL_16)
    assert not _native.layer_norm_supported(x[..., :40].contiguous())
    assert not _native.layer_norm_supported(x.double())
    assert not _native.layer_norm_supported(x.cpu())
    with pytest.raises(RuntimeError):
        _native.layer_norm(x[..., :40].contiguous(), w[:40], b[:40])


@pytest.mark.gpu
@pytest.mark.parametrize("branch_dtype", [torch.float16, torch.bfloat16])
def test_add_layer_norm_kernel_equals_the_separate_addition_and_norm(device, branch_dtype):
    """The residual addition ahead of a norm and the norm in one pass: the sum equals the framework's addition bit
    for bit (fp32 + 16-bit -> fp32; 16-bit + 16-bit -> 16-bit, rounded before it is normalised), the normalised rows
    are F.layer_norm of that sum in fp32, rounded once."""
    from clusten import _native
    gen = torch.Generator().manual_seed(23)
    for x_dtype in (torch.float32, branch_dtype):
        for rows, c in ((1003, 64), (517, 128), (260, 256), (130, 384), (70, 512), (35, 768), (9, 1024)):
            x = (torch.randn(rows, c, generator=gen) * 2 + 0.5).to(x_dtype).to(device)
            branch = torch.randn(rows, c, generator=gen).to(branch_dtype).to(device)
            w = (torch.rand(c, generator=gen) + 0.5).to(device)
            b = torch.randn(c, generator=gen).to(device)
            assert _native.add_layer_norm_supported(x, branch)
            total, out = _native.add_layer_norm(x, branch, w, b, 1e-5)
            want_total = x + branch
            assert total.dtype == want_total.dtype and torch.equal(total, want_total)
            want = torch.nn.functional.layer_norm(want_total.float(), (c,), w, b, 1e-5)
            assert out.dtype == branch_dtype
            err = oracle.rel_err(out.float().cpu(), want.cpu())
            assert err <= (1e-3 if branch_dtype == torch.float16 else 8e-3), (x_dtype, rows, c, err)
    x = torch.zeros(4, 3, 64, device=device)
    assert not _native.add_layer_norm_supported(x, x)                               # fp32 branch
    assert not _native.add_layer_norm_supported(x.half(), x.bfloat16())             # mixed 16-bit types
    assert not _native.add_layer_norm_supported(x[..., :48], x[..., :48].half())    # width without a kernel
    with pytest.raises(RuntimeError):
        _native.add_layer_norm(x, x, torch.ones(64, device=device), torch.zeros(64, device=device))
    t, o = _native.add_layer_norm(x[:0], x[:0].half(), torch.ones(64, device=device), torch.zeros(64, device=device))
    assert t.shape == (0, 3, 64) and o.shape == (0, 3, 64)


@pytest.mark.gpu
def test_neighbour_lists_kernel_equals_the_tensor_expressions(device):
    """member_idx, mask, pe_idx and the int32 cluster numbers in one kernel: equal, element for element, to the gather
    and the tensor operations of BasicLayer.neighbourhoods (whole-number and fractional positions, a short last
    cluster, clusters of 8 and of 5)."""
    from clusten import _native
    gen = torch.Generator().manual_seed(29)
    for b, n, nnc, m, radius, frac in ((3, 196, 6, 8, 55, False), (2, 784, 6, 8, 55, False), (2, 203, 4, 5, 30, True),
                                       (1, 8, 1, 8, 3, False)):
        k = (n + m - 1) // m
        pos = torch.randint(0, radius + 1, (b, n, 2), generator=gen).float()
        if frac:
            pos = pos + torch.rand(b, n, 2, generator=gen)
        pos = pos.to(device)
        nearest = torch.randint(0, k, (b, n, nnc), generator=gen).to(device)
        width = 2 * radius + 1
        rows = nearest.unsqueeze(3) * m + torch.arange(m, device=device)
        valid = rows < n
        want_members = torch.where(valid, rows, torch.zeros_like(rows)).reshape(b, n, nnc * m)
        nb_pos = pos.gather(1, want_members.reshape(b, -1, 1).expand(-1, -1, 2)).reshape(b, n, nnc * m, 2)
        rel = nb_pos - (pos.unsqueeze(2) - radius)
        want_pe = (rel[..., 1] * width + rel[..., 0]).long()
        members, mask, pe_idx, cidx = _native.neighbour_lists(pos, nearest, m, radius, width, True)
        assert torch.equal(members, want_members)
        assert torch.equal(mask, valid.reshape(b, n, nnc * m).long())
        assert torch.equal(pe_idx, want_pe)
        assert cidx.dtype == torch.int32 and torch.equal(cidx.long(), nearest)
        assert _native.neighbour_lists(pos, nearest, m, radius, width, False)[1] is None
    assert not _native.neighbour_lists_supported(pos.cpu(), nearest.cpu())
    assert not _native.neighbour_lists_supported(pos.double(), nearest)
    assert not _native.neighbour_lists_supported(pos, nearest.int())
    with pytest.raises(RuntimeError):
        _native.neighbour_lists(pos.double(), nearest, 8, 3, 7, False)


@pytest.mark.gpu
def test_layer_norm_kernel_with_row_order_and_bias(device):
    """The norm that ends the patch embedding with the reordering of the tokens and the convolution's bias taken
    along: row i of every image is the norm of (row order[i] + bias), the sum rounded to the input's type."""
    from clusten import _native
    gen = torch.Generator().manual_seed(31)
    for in_dtype in (torch.float16, torch.bfloat16, torch.float32):
        for b, n, c in ((3, 200, 64), (2, 49, 128), (1, 7, 256)):
            x = (torch.randn(b, n, c, generator=gen) * 2).to(in_dtype).to(device)
            bias = torch.randn(c, generator=gen).to(device)
            w = (torch.rand(c, generator=gen) + 0.5).to(device)
            beta = torch.randn(c, generator=gen).to(device)
            order = torch.randperm(n, generator=gen).to(device)
            summed = (x + bias.to(in_dtype)).float()
            want = torch.nn.functional.layer_norm(summed, (c,), w, beta, 1e-5)
            tol = 1e-5
            assert oracle.rel_err(_native.layer_norm(x, w, beta, 1e-5, None, order, bias).cpu(), want[:, order].cpu()) <= tol
            assert oracle.rel_err(_native.layer_norm(x, w, beta, 1e-5, None, None, bias).cpu(), want.cpu()) <= tol
            plain = torch.nn.functional.layer_norm(x.float(), (c,), w, beta, 1e-5)
            assert oracle.rel_err(_native.layer_norm(x, w, beta, 1e-5, None, order).cpu(), plain[:, order].cpu()) <= tol
    with pytest.raises(RuntimeError):
        _native.layer_norm(x, w, beta, 1e-5, None, order[:3])
    with pytest.raises(RuntimeError):
        _native.layer_norm(x, w, beta, 1e-5, None, None, bias[:5])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_channel_affine_gelu_kernel_equals_bias_batch_norm_gelu(device, dtype):
    """Convolution bias, inference BatchNorm and GELU as one affine map per channel and one activation."""
    from clusten import _native
    gen = torch.Generator().manual_seed(37)
    b, c, h, w = 3, 32, 20, 12
    x = torch.randn(b, c, h, w, generator=gen).to(dtype).to(device)
    conv_bias = torch.randn(c, generator=gen).to(device)
    bn = torch.nn.BatchNorm2d(c).to(device).eval()
    with torch.no_grad():
        bn.weight.copy_(torch.rand(c, generator=gen) + 0.5)
        bn.bias.copy_(torch.randn(c, generator=gen))
        bn.running_mean.copy_(torch.randn(c, generator=gen))
        bn.running_var.copy_(torch.rand(c, generator=gen) + 0.3)
        want = torch.nn.functional.gelu(bn(x.float() + conv_bias.view(1, c, 1, 1)))
    scale = bn.weight / torch.sqrt(bn.running_var + bn.eps)
    shift = (conv_bias - bn.running_mean) * scale + bn.bias
    assert _native.channel_affine_gelu_supported(x)
    out = _native.channel_affine_gelu(x, scale, shift)
    assert out.dtype == dtype and out.shape == x.shape
    assert oracle.rel_err(out.float().cpu(), want.cpu()) <= (1e-3 if dtype == torch.float16 else 8e-3)
    assert not _native.channel_affine_gelu_supported(x[:, :, :, :5])
    assert not _native.channel_affine_gelu_supported(x.float())
    with pytest.raises(RuntimeError):
        _native.channel_affine_gelu(x.float(), scale, shift)
    with pytest.raises(RuntimeError):
        _native.channel_affine_gelu(x, scale[:4], shift)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_add_row_score_kernel_equals_addition_linear_sigmoid(device, dtype):
    """The importance score of the tokens with the residual addition ahead of it: the sum equals the framework's
    addition bit for bit, the score is sigmoid(Linear(sum in 16 bits)) with the product rounded to 16 bits first."""
    from clusten import _native
    gen = torch.Generator().manual_seed(41)
    for x_dtype in (torch.float32, dtype):
        for shape, c in (((3, 203), 64), ((2, 77), 128), ((5, 19), 256), ((1, 9), 512)):
            x = torch.randn(*shape, c, generator=gen).to(x_dtype).to(device)
            branch = torch.randn(*shape, c, generator=gen).to(dtype).to(device)
            w = (torch.randn(1, c, generator=gen) * c ** -0.5).to(dtype).to(device)
            b = torch.randn(1, generator=gen).to(dtype).to(device)
            for br in (branch, None):
                assert _native.add_row_score_supported(x, br, w)
                total, score = _native.add_row_score(x, br, w, b)
                want_total = x if br is None else x + br
                assert total.dtype == x.dtype and torch.equal(total, want_total)
                y = torch.nn.functional.linear(want_total.to(dtype).float(), w.float(), b.float()).to(dtype)
                want = torch.sigmoid(y.float())
                assert score.dtype == dtype and score.shape == tuple(shape) + (1,)
                assert oracle.rel_err(score.float().cpu(), want.cpu()) <= (2e-3 if dtype == torch.float16 else 1.6e-2)
    assert not _native.add_row_score_supported(x, None, w.float())
    assert not _native.add_row_score_supported(x[..., :96], None, w[:, :96])
    assert not _native.add_row_score_supported(x, branch.float(), w)
    with pytest.raises(RuntimeError):
        _native.add_row_score(x, None, w.float(), None)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("with_mask", [False, True])
def test_attention_glue_training_function_matches_autograd_through_the_expressions(device, dtype, with_mask):
    """Bias lookup, mask, blank token and softmax as one kernel forward and one backward (training): outputs and the
    gradients of the logits, the bias table and the blank logit against autograd through the tensor expressions."""
    from aff.model import _AttnSoftmax, default_ops
    ops = default_ops()
    gen = torch.Generator().manual_seed(47)
    b, h, n, m, rows = 2, 3, 50, 48, 211
    attn = torch.randn(b, h, n, m, generator=gen).to(dtype).to(device).requires_grad_()
    bias = torch.randn(rows, h, generator=gen).to(dtype).to(device).requires_grad_()
    blank = torch.randn(b, h, n, 1, generator=gen).to(device).requires_grad_()
    pe_idx = torch.randint(rows, (b, n, m), generator=gen).to(device)
    mask = (torch.rand(b, n, m, generator=gen) > 0.1).long().to(device) if with_mask else None
    g_p = torch.randn(b, h, n, m, generator=gen).to(device)
    g_b = torch.randn(b, h, n, 1, generator=gen).to(device)

    probs, blank_prob = _AttnSoftmax.apply(attn, bias, pe_idx, mask, blank, ops)
    ((probs * g_p).sum() + (blank_prob * g_b).sum()).backward()
    got = (probs.detach(), blank_prob.detach(), attn.grad.clone(), bias.grad.clone(), blank.grad.clone())
    attn.grad = bias.grad = blank.grad = None

    x = attn.float() + bias.float()[pe_idx].permute(0, 3, 1, 2)
    if mask is not None:
        x = x + (1 - mask.reshape(b, 1, n, m)) * (-100)
    p = torch.softmax(torch.cat([x, blank], dim=-1), dim=-1)
    ((p[..., :-1] * g_p).sum() + (p[..., -1:] * g_b).sum()).backward()
    want = (p[..., :-1].detach(), p[..., -1:].detach(), attn.grad, bias.grad, blank.grad)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for name, a, w in zip(("probs", "blank_prob", "d_attn", "d_bias", "d_blank"), got, want):
        assert a.shape == w.shape and a.dtype == w.dtype, name
        assert oracle.rel_err(a.float().cpu(), w.float().cpu()) <= tol, name


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_bias_table_grad_kernel_equals_the_scatter_add(device, dtype):
    """Gradient of the position-bias table: per-workgroup sums in LDS against index_add in fp64."""
    from clusten import _native
    gen = torch.Generator().manual_seed(43)
    for b, h, n, m, rows in ((3, 2, 200, 48, 12321), (2, 8, 49, 49, 12321), (1, 1, 5, 8, 7), (4, 16, 64, 48, 16000),
                             (2, 4, 96, 144, 36481), (1, 2, 33, 7, 40000), (2, 3, 64, 48, 100001)):
        g = torch.randn(b, h, n, m, generator=gen).to(dtype)
        # positions near the table's centre, as relative offsets of neighbours are, plus some anywhere (in a table of
        # more than 20 000 rows those mostly fall outside the rows the kernel sums in LDS)
        idx = (rows // 2 + torch.randint(-min(60, rows // 2), min(61, rows - rows // 2), (b, n, m), generator=gen))
        far = torch.rand(b, n, m, generator=gen) < (0.05 if rows <= 20000 else 0.3)
        idx[far] = torch.randint(rows, (int(far.sum()),), generator=gen)
        want = torch.zeros(rows, h, dtype=torch.float64)
        want.index_add_(0, idx.reshape(-1), g.double().permute(0, 2, 3, 1).reshape(-1, h))
        got = _native.bias_table_grad(g.to(device), idx.to(device), rows)
        assert got.dtype == torch.float32 and got.shape == (rows, h)
        assert oracle.rel_err(got.cpu().double(), want) <= 1e-5
    assert _native.bias_table_grad_supported(g.to(device), 40001) and not _native.bias_table_grad_supported(g.to(device), 0)
    assert not _native.bias_table_grad_supported(g, 100)
    with pytest.raises(RuntimeError):
        _native.bias_table_grad(g.to(device), idx.to(device)[:, :, :3], rows)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_bias_table_grad_on_offsets_between_neighbours_and_on_values_of_any_size(device, dtype):
    """The indices of a model are offsets between near tokens: a few hundred cells take every addition.  Tables of up
    to 20 000 rows are summed in 64-bit integer cells whose unit hangs on the largest magnitude of a workgroup's slice:
    values of very different sizes, zeros, subnormals, infinities and NaNs must come out as fp64 sums rounded once."""
    from clusten import _native
    gen = torch.Generator().manual_seed(47)
    b, h, n, m, rows = 6, 2, 784, 48, 12321
    dx, dy = torch.randint(-4, 5, (b, n, m), generator=gen), torch.randint(-4, 5, (b, n, m), generator=gen)
    idx = (dy + 55) * 111 + dx + 55                                   # 81 distinct cells
    big = {torch.float32: 1e30, torch.float16: 1e4, torch.bfloat16: 1e30}[dtype]   # (fp16: randn * 1e4 stays finite)
    tiny = {torch.float32: 1e-36, torch.float16: 6e-8, torch.bfloat16: 1e-36}[dtype]
    for scale_of_image in ((1.0,) * b, (big, 1.0, tiny, 1e-3, 0.0, 1e3)):
        g = torch.randn(b, h, n, m, generator=gen) * torch.tensor(scale_of_image).view(b, 1, 1, 1)
        g = g.to(dtype)
        want = torch.zeros(rows, h, dtype=torch.float64)
        want.index_add_(0, idx.reshape(-1), g.double().permute(0, 2, 3, 1).reshape(-1, h))
        got = _native.bias_table_grad(g.to(device), idx.to(device), rows).cpu().double()
        # fp64 sums of at most 6 * 784 * 48 values per cell, rounded to fp32 by at most a few hundred workgroups
        assert torch.isfinite(got).all()
        assert oracle.rel_err(got, want) <= 2e-6
        touched = want != 0
        assert (got[~touched] == 0).all()
    # values a slice can hold exactly: integers in fp16 sum without any rounding, whatever the order
    gi = torch.randint(-8, 9, (b, h, n, m), generator=gen).to(dtype)
    want = torch.zeros(rows, h, dtype=torch.float64)
    want.index_add_(0, idx.reshape(-1), gi.double().permute(0, 2, 3, 1).reshape(-1, h))
    got = _native.bias_table_grad(gi.to(device), idx.to(device), rows).cpu().double()
    assert torch.equal(got, want)
    # an infinity and a NaN reach their cells as they are and leave the others alone
    gs = torch.randn(b, h, n, m, generator=gen).to(dtype)
    gs[1, 0, 5, 7], gs[2, 1, 9, 3] = float("inf"), float("nan")
    got = _native.bias_table_grad(gs.to(device), idx.to(device), rows).cpu()
    assert torch.isinf(got[idx[1, 5, 7], 0]) and torch.isnan(got[idx[2, 9, 3], 1])
    clean = gs.clone()
    clean[1, 0, 5, 7], clean[2, 1, 9, 3] = 0.0, 0.0
    want = torch.zeros(rows, h, dtype=torch.float64)
    want.index_add_(0, idx.reshape(-1), clean.double().permute(0, 2, 3, 1).reshape(-1, h))
    keep = torch.ones(rows, h, dtype=torch.bool)
    keep[idx[1, 5, 7], 0], keep[idx[2, 9, 3], 1] = False, False
    assert oracle.rel_err(got.double()[keep], want[keep]) <= 2e-6


@pytest.mark.gpu
def test_merge_weights_kernel_equals_the_tensor_expressions(device):
    from clusten import _native
    gen = torch.Generator().manual_seed(19)
    b, n, n_out, m, rows = 3, 200, 50, 48, 321
    table_w = torch.randn(rows, 4, generator=gen).to(device)
    pe_idx = torch.randint(rows, (b, n_out, m), generator=gen).to(device)
    nbhd = torch.randint(n, (b, n_out, m), generator=gen).to(device)
    prob = torch.rand(b, n, 1, generator=gen).to(device)
    mask = (torch.rand(b, n_out, m, generator=gen) > 0.2).long().to(device)
    for p, mk in ((prob, mask), (prob, None), (None, mask), (None, None), (prob.half(), mask)):
        ref = table_w[pe_idx]
        if p is not None:
            ref = ref * p.gather(1, nbhd.reshape(b, -1, 1)).reshape(b, n_out, m, 1)
        if mk is not None:
            ref = ref * mk.unsqueeze(3)
        out = _native.merge_weights(table_w, pe_idx, nbhd, p, mk)
        assert out.dtype == torch.float32 and out.shape == (b, n_out, m, 4)
        assert torch.equal(out, ref.float())        # one fp32 product per factor, in the same order
    assert not _native.merge_weights_supported(table_w[:, :3])
    with pytest.raises(RuntimeError):
        _native.merge_weights(table_w, pe_idx.int(), nbhd, prob, mask)


@pytest.mark.gpu
def test_operator_dtypes_under_autocast(device):
    """fp16 autocast hands QK fp16 operands and AV / WF fp32 first operands, as in the reference model."""
    from aff.model import default_ops
    seen = {}
    real = default_ops()

    def spy(name, fn):
        def call(a, b, idx):
            seen.setdefault(name, (a.dtype, b.dtype, a.is_contiguous(), b.is_contiguous()))
            return fn(a, b, idx)
        return call
    ops = SimpleNamespace(qk=spy("qk", real.qk), av=spy("av", real.av), wf=spy("wf", real.wf))
    model = small_model(ops, img_size=128).to(device)
    x = torch.randn(2, 3, 128, 128, device=device)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        model(x)
    assert seen["qk"][:2] == (torch.float16, torch.float16)
    assert seen["av"][:2] == (torch.float32, torch.float16)
    assert seen["wf"][0] == torch.float32
    # q, key and v reach the operators as permuted views, not copies
    assert seen["qk"][2:] == (False, False) and seen["av"][3] is False


@pytest.mark.gpu
def test_aff_tiny_224_logits_equal_with_hip_operators_and_with_the_oracle(device):
    """The configuration the images/s figure is quoted on: every operator call of AFF-Tiny at 224x224 under fp16
    autocast (local and global attention in one kernel each, kNN kernel on the HIP side; tensor expressions
    on the other)."""
    from aff.model import default_ops
    ops = default_ops()
    calls = []
    one_kernel = ops.cluster_attention
    ops.cluster_attention = lambda *a, **kw: (calls.append(a[0].dtype), one_kernel(*a, **kw))[1]
    linear_calls = []
    linear_kernel = ops.linear
    ops.linear = lambda *a, **kw: (linear_calls.append(tuple(a[1].shape)), linear_kernel(*a, **kw))[1]
    dense_calls = []
    dense_kernel = ops.dense_attention
    ops.dense_attention = lambda *a, **kw: (dense_calls.append(a[0].shape[2]), dense_kernel(*a, **kw))[1]
    torch.manual_seed(0)
    hip = aff_tiny(ops=ops).to(device).eval()
    torch.manual_seed(0)
    ref = aff_tiny(ops=oracle_ops()).to(device).eval()
    ref.load_state_dict(hip.state_dict())
    x = torch.randn(2, 3, 224, 224, generator=torch.Generator().manual_seed(3)).to(device)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        y_hip, y_ref = hip(x), ref(x)
    assert y_hip.shape == (2, 1000) and torch.isfinite(y_hip).all()
    assert oracle.rel_err(y_hip.float(), y_ref.float()) < 2e-2
    # the 25 blocks of the three local-attention stages took the one-kernel path, on fp16 operands
    assert calls == [torch.float16] * 25
    # and the 5 blocks of the last stage (49 tokens, each attending to all) the dense one
    assert dense_calls == [49] * 5
    # the Linear layers keep the framework's kernels at this batch size (the library's takes 65536 rows and more)
    assert linear_calls == []
    # the same model with the three operators and the softmax kernel between them
    three = default_ops()
    del three.cluster_attention
    del three.dense_attention
    del three.linear
    del three.add_layer_norm
    del three.neighbour_lists
    del three.add_row_score
    del three.channel_affine_gelu
    hip3 = aff_tiny(ops=three).to(device).eval()
    hip3.load_state_dict(hip.state_dict())
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        y3 = hip3(x)
    assert oracle.rel_err(y_hip.float(), y3.float()) < 2e-2


@pytest.mark.gpu
def test_aff_tiny_224_small_linear_layers_through_the_library(device):
    """From 21 images on, the first stage has 65536 rows and more: its q / kv / proj / MLP layers take the library's
    Linear kernel; the logits agree with the framework's GEMMs."""
    from aff.model import default_ops
    ops = default_ops()
    shapes = []
    kernel = ops.linear
    ops.linear = lambda *a, **kw: (shapes.append((tuple(a[1].shape), bool(a[3]) if len(a) > 3 else False)),
                                   kernel(*a, **kw))[1]
    torch.manual_seed(0)
    hip = aff_tiny(ops=ops).to(device).eval()
    plain = default_ops()
    del plain.linear
    ref = aff_tiny(ops=plain).to(device).eval()
    ref.load_state_dict(hip.state_dict())
    x = torch.randn(24, 3, 224, 224, generator=torch.Generator().manual_seed(4)).to(device)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        y_hip, y_ref = hip(x), ref(x)
    assert torch.isfinite(y_hip).all()
    assert oracle.rel_err(y_hip.float(), y_ref.float()) < 1e-2
    per_block = [((64, 64), False), ((128, 64), False), ((64, 64), False), ((192, 64), True), ((64, 192), False)]
    assert shapes == per_block * 3        # the merge projection works on a quarter of the rows: below the threshold


@pytest.mark.gpu
def test_recorded_forward_replays_equal_the_eager_forward(device):
    """The forward recorded into a HIP graph: every replay, with eager forwards and synchronisations between
    them, gives the eager result bit for bit (the kernels are deterministic and the recording holds no memset)."""
    from aff.model import CapturedForward
    torch.manual_seed(0)
    net = aff_tiny().to(device).eval()
    gen = torch.Generator().manual_seed(5)
    xs = [torch.randn(2, 3, 224, 224, generator=gen).to(device) for _ in range(3)]

    def eager(x):
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
            return net(x)

    want = [eager(x).clone() for x in xs]
    recorded = CapturedForward(net, xs[0])
    for rep in range(3):
        for i, x in enumerate(xs):
            got = recorded(x).clone()
            torch.cuda.synchronize()
            assert torch.equal(got, want[i]), "replay %d of input %d" % (rep, i)
            assert torch.equal(eager(xs[(i + 1) % 3]), want[(i + 1) % 3])
    with pytest.raises(RuntimeError):
        recorded(xs[0][:1])
    with pytest.raises(RuntimeError):
        CapturedForward(net, xs[0].cpu())


@pytest.mark.gpu
def test_aff_tiny_224_at_the_benchmarked_batch_equals_the_small_batch(device):
    """The images/s figure is taken at batch 128, where the grid stage hands over one image's lists for the whole batch,
    the Linear layers of stage 1 go through the library's kernel and the forward is replayed from a HIP graph.  The
    logits of images 0 and 1 inside that batch equal those of a batch of just the two (itself checked against the
    oracle model above) within the mixed-precision tolerance, eager and replayed; the replay equals eager bit for bit."""
    from aff.model import CapturedForward
    torch.manual_seed(0)
    net = aff_tiny().to(device).eval()
    x = torch.randn(128, 3, 224, 224, generator=torch.Generator().manual_seed(6)).to(device)

    def eager(inp):
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
            return net(inp)

    small = eager(x[:2]).float()
    big = eager(x)
    assert big.shape == (128, 1000) and torch.isfinite(big).all()
    assert oracle.rel_err(big[:2].float(), small) < 2e-2
    recorded = CapturedForward(net, x)
    for _ in range(2):
        replayed = recorded(x).clone()
        torch.cuda.synchronize()
        assert torch.equal(replayed, big)
    assert oracle.rel_err(replayed[:2].float(), small) < 2e-2
    # every image of the batch is its own problem: a permutation of the batch permutes the logits
    perm = torch.randperm(128, generator=torch.Generator().manual_seed(7)).to(device)
    assert oracle.rel_err(eager(x[perm]).float(), big[perm].float()) < 2e-2
    del recorded


@pytest.mark.gpu
def test_aff_tiny_224_forward_and_gradients(device):
    model = aff_tiny().to(device)
    x = torch.randn(2, 3, 224, 224, device=device)
    model.eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        y = model(x)
    assert y.shape == (2, 1000) and torch.isfinite(y).all()
    model.train()
    model(x).square().mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())


@pytest.mark.gpu
def test_cached_16_bit_weights_follow_the_parameters(device):
    """Inference under autocast keeps 16-bit copies of the Linear weights between forwards; an in-place update, a
    load_state_dict and a move of the parameters must all be seen by the next forward."""
    from aff.model import default_ops
    model = small_model(default_ops(), img_size=128).to(device)
    x = torch.randn(2, 3, 128, 128, generator=torch.Generator().manual_seed(5)).to(device)

    def run(m):
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
            return m(x).float()

    y0 = run(model)
    assert torch.equal(run(model), y0)                      # second forward: from the cached copies
    state = {k: v.clone() for k, v in model.state_dict().items()}
    with torch.no_grad():                                   # in-place update of one projection and of the classifier
        model.layers[0].blocks[0].attn.proj.weight.mul_(1.5)
        model.head.bias.add_(1.0)
    y1 = run(model)
    fresh = small_model(default_ops(), img_size=128).to(device)
    fresh.load_state_dict(model.state_dict())
    assert torch.equal(y1, run(fresh)) and not torch.equal(y1, y0)
    model.load_state_dict(state)                            # back to the first weights
    assert torch.equal(run(model), y0)
    model.float()                                           # no-op conversion keeps working
    assert torch.equal(run(model), y0)
    # the position-bias table of an attention layer and the weight table of a merge are kept as well: functions of
    # their parameters and of the relative-position table only
    with torch.no_grad():
        model.layers[0].blocks[0].attn.pos_embed.weight.mul_(3.0)
        model.layers[0].downsample.weight_net[0].bias.add_(0.5)
    y2 = run(model)
    fresh = small_model(default_ops(), img_size=128).to(device)
    fresh.load_state_dict(model.state_dict())
    assert torch.equal(y2, run(fresh)) and not torch.equal(y2, y0)
    with torch.no_grad():                                   # without autocast: other tables, not the fp16 ones
        y_fp32 = model(x)
        assert torch.equal(y_fp32, fresh(x))
    assert torch.equal(run(model), y2)
    model.load_state_dict(state)
    assert torch.equal(run(model), y0)
    # training mode and grad mode do not use the cache
    model.train()
    with torch.autocast("cuda", dtype=torch.float16):
        model(x).float().sum().backward()
    assert model.head.weight.grad is not None


@pytest.mark.gpu
@pytest.mark.parametrize("img_size", [128, 120])
@pytest.mark.parametrize("amp", [True, False])
def test_training_with_the_one_kernel_attention_matches_the_operator_path(device, img_size, amp):
    """A training step (under fp16 autocast, or in fp32) with the local attention as one kernel forward and
    `cluster_attention_backward` plus its sums backward, against the same step through the three operators and the
    softmax kernels: same loss, parameter gradients within the noise of fp16 intermediates (fp32: within 1e-3 of the
    largest entry).  At 120 x 120 pixels the stages hold 900, 225 and 56 tokens: short last clusters, pad slots and
    masks in every local stage."""
    import contextlib
    from aff.model import default_ops
    mode = (lambda: torch.autocast("cuda", dtype=torch.float16)) if amp else contextlib.nullcontext
    fused_ops = default_ops()
    plain = dict(vars(default_ops()))
    plain.pop("cluster_attention_backward")
    plain_ops = SimpleNamespace(**plain)
    cfg = dict(embed_dim=(64, 128, 256, 512), num_heads=(2, 4, 8, 16), img_size=img_size)
    a = small_model(fused_ops, **cfg).to(device).train()
    b = small_model(plain_ops, **cfg).to(device).train()
    b.load_state_dict(a.state_dict())
    x = torch.randn(2, 3, img_size, img_size, generator=torch.Generator().manual_seed(5)).to(device)
    target = torch.tensor([3, 7], device=device)
    losses = []
    for m in (a, b):
        with mode():
            loss = torch.nn.functional.cross_entropy(m(x).float(), target)
        loss.backward()
        losses.append(float(loss.detach()))
    assert abs(losses[0] - losses[1]) <= (2e-2 if amp else 1e-5) * max(1.0, abs(losses[1]))
    # a gradient that is pure rounding noise (a bias in front of a batch norm) is measured against the largest gradient
    # of the model, not against itself
    biggest = max(float(p.grad.abs().max()) for p in b.parameters() if p.grad is not None)
    checked = 0
    for (name, pa), (_, pb) in zip(a.named_parameters(), b.named_parameters()):
        assert (pa.grad is None) == (pb.grad is None), name
        if pa.grad is None:
            continue
        scale = max(float(pb.grad.abs().max()), 1e-2 * biggest)
        err = float((pa.grad - pb.grad).abs().max()) / scale
        assert err <= (5e-2 if amp else 1e-3), "%s rel err %.3g" % (name, err)
        checked += 1
    assert checked > 50
    # the fused path was taken: its Function is in the graph of a fresh forward
    with mode():
        y = a(x)
    seen, stack = set(), [y.grad_fn]
    while stack:
        f = stack.pop()
        if f is None or f in seen:
            continue
        seen.add(f)
        stack.extend(nf for nf, _ in f.next_functions)
    assert any("_ClusterAttention" in type(f).__name__ for f in seen)
