"""The merge centres of the adaptive down-sampling as one kernel, against the tensor expressions of
`ClusterMerging.forward` (models/aff_transformer.py:296-346) written out here on the same device."""
import math

import pytest
import torch

from clusten import _native

pytestmark = pytest.mark.gpu


def _scores(pos, learned_prob, alpha, stride, reserve_on):
    """final_prob and the reserved mask as the reference builds them (aff_transformer.py:296-317)."""
    b, n, _ = pos.shape
    if stride == 2:
        prior = ((pos % stride).sum(-1) == 0).float()
        dist = None
    else:
        d2 = (pos[:, :, None, :] - pos[:, None, :, :]).pow(2).sum(-1)
        d2 = d2 + torch.eye(n, device=pos.device) * 1e9
        dist = d2.min(dim=2)[0].sqrt()
        spacing = 2 ** (dist.log2().ceil() + 1)
        prior = ((pos.long() % spacing.unsqueeze(2).long()).sum(-1) == 0).float()
    score = prior
    if learned_prob is not None:
        score = score + learned_prob.view(b, n) * alpha
    reserved = None
    if reserve_on:
        reserved = ((pos % (stride * 2)).sum(-1) == 0)
        score = score + reserved.float() * (-100)
    return score, reserved, dist


def _expected(score, reserved, sample_num, reserve_num):
    """The selection in the kernel's stated order, image by image."""
    rows = []
    for s, r in zip(score.cpu(), [None] * score.shape[0] if reserved is None else reserved.cpu()):
        kth = s.sort(descending=True)[0][sample_num - 1]
        above = (s > kth).nonzero()[:, 0]
        equal = (s == kth).nonzero()[:, 0][:sample_num - above.numel()]
        parts = [above, equal]
        if r is not None:
            parts.append(r.nonzero()[:, 0][:reserve_num])
        rows.append(torch.cat(parts))
    return torch.stack(rows)


def _grid(b, h, w, device):
    ys, xs = torch.meshgrid(torch.arange(h), torch.arange(w), indexing="ij")
    return torch.stack([xs.reshape(-1), ys.reshape(-1)], 1).float().expand(b, -1, -1).contiguous().to(device)


def _subset(b, h, w, n, seed, device):
    gen = torch.Generator().manual_seed(seed)
    full = _grid(1, h, w, "cpu")[0]
    return torch.stack([full[torch.randperm(h * w, generator=gen)[:n]] for _ in range(b)]).to(device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("reserve_on", [True, False])
def test_centres_on_the_full_grid(device, dtype, reserve_on):
    b, h, w, stride = 4, 56, 56, 2
    pos = _grid(b, h, w, device)
    n = h * w
    prob = torch.rand(b, n, 1, generator=torch.Generator().manual_seed(3)).to(device=device, dtype=dtype)
    keep = int(n * 0.25)
    reserve_num = math.ceil(h / (stride * 2)) * math.ceil(w / (stride * 2))
    sample = keep - reserve_num if reserve_on else keep
    got = _native.merge_centres(pos, None, prob, 4.0, stride, sample, reserve_num, reserve_on)
    score, reserved, _ = _scores(pos, prob, 4.0, stride, reserve_on)
    assert score.dtype == torch.float32
    assert torch.equal(got.cpu(), _expected(score, reserved, sample, reserve_num))
    # as a set, what topk selects (16-bit scores tie at the cut now and then: there any of the equal ones will do)
    top = score.topk(sample, dim=1, sorted=False)[1]
    s_got = score.gather(1, got[:, :sample]).sort(1)[0]
    assert torch.equal(s_got, score.gather(1, top).sort(1)[0])
    assert got.shape == (b, keep)
    assert all(row.unique().numel() == keep for row in got)


@pytest.mark.parametrize("n,stride", [(784, 4), (196, 8), (777, 4)])
def test_centres_on_an_adaptive_grid(device, n, stride):
    b, h, w = 3, 56, 56
    pos = _subset(b, h, w, n, 5 + n, device)
    prob = torch.rand(b, n, 1, generator=torch.Generator().manual_seed(n)).to(device)
    keep = int(n * 0.25)
    score, reserved, dist = _scores(pos, prob, 4.0, stride, True)
    reserve_num = int(reserved.sum(1).min())          # as many as every image has (the model's grids have the same)
    got = _native.merge_centres(pos, dist, prob, 4.0, stride, keep - reserve_num, reserve_num, True)
    assert torch.equal(got.cpu(), _expected(score, reserved, keep - reserve_num, reserve_num))
    # the library's own nearest-neighbour distances give the same centres
    from aff.points import knn
    dist2 = knn(pos, pos, 2, return_dist=True)[1][:, :, 1]
    assert torch.equal(dist2, dist)
    assert torch.equal(_native.merge_centres(pos, dist2, prob, 4.0, stride, keep - reserve_num, reserve_num, True), got)


def test_equal_scores_at_the_cut_go_to_the_lower_index(device):
    # no importance scores: the scores are 1, 0 and -99 only
    b, h, w = 2, 24, 40
    pos = _grid(b, h, w, device)
    n = h * w
    for sample in (1, 50, 240, 241, 600, n - 60):
        got = _native.merge_centres(pos, None, None, 4.0, 2, sample, 60, True)
        score, reserved, _ = _scores(pos, None, 4.0, 2, True)
        assert torch.equal(got.cpu(), _expected(score, reserved, sample, 60)), sample


def test_centres_of_the_first_stage_of_a_384_model(device):
    b, h, w = 2, 96, 96
    pos = _grid(b, h, w, device)
    n = h * w
    assert n <= _native.load().clusten_merge_centres_max_tokens()
    prob = torch.rand(b, n, 1, generator=torch.Generator().manual_seed(9)).to(device)
    keep, reserve_num = n // 4, 24 * 24
    got = _native.merge_centres(pos, None, prob, 4.0, 2, keep - reserve_num, reserve_num, True)
    score, reserved, _ = _scores(pos, prob, 4.0, 2, True)
    assert torch.equal(got.cpu(), _expected(score, reserved, keep - reserve_num, reserve_num))


def test_centres_of_a_sequence_past_48_kb_of_keys(device):
    b, h, w = 2, 128, 128                      # the first stage of a 512 x 512 image: 16 384 tokens, 64 KB of keys
    pos = _grid(b, h, w, device)
    n = h * w
    assert n <= _native.load().clusten_merge_centres_max_tokens()
    prob = torch.rand(b, n, 1, generator=torch.Generator().manual_seed(10)).to(device)
    keep, reserve_num = n // 4, 32 * 32
    got = _native.merge_centres(pos, None, prob, 4.0, 2, keep - reserve_num, reserve_num, True)
    score, reserved, _ = _scores(pos, prob, 4.0, 2, True)
    assert torch.equal(got.cpu(), _expected(score, reserved, keep - reserve_num, reserve_num))


def test_refusals(device):
    pos = _grid(1, 8, 8, device)
    with pytest.raises(RuntimeError):
        _native.merge_centres(pos, None, None, 4.0, 2, 0, 4, True)          # nothing to sample
    with pytest.raises(RuntimeError):
        _native.merge_centres(pos, None, None, 4.0, 2, 64, 4, True)         # more than there are tokens
    long = torch.zeros(1, _native.load().clusten_merge_centres_max_tokens() + 1, 2, device=device)
    assert not _native.merge_centres_supported(long)
    with pytest.raises(RuntimeError):
        _native.merge_centres(pos.cpu(), None, None, 4.0, 2, 4, 4, True)


def test_an_image_with_fewer_reserved_tokens_than_asked_for(device, monkeypatch):
    """The reference's reshape raises when an image does not hold reserve_num tokens on the coarse grid
    (aff_transformer.py:323).  The kernel fills the slots of the missing ones with -1 (nothing stays unwritten), the row
    gather reads row 0 for them, and under CLUSTEN_DEBUG_INDICES=1 the wrapper raises like the reference; a surplus of
    reserved tokens is cut to the first reserve_num."""
    pos = _grid(2, 8, 8, device)                       # 4 tokens of each image lie on the grid of spacing 4
    pos[1, 0] = torch.tensor([1.0, 1.0])               # ... but image 1 loses one: 3
    got = _native.merge_centres(pos, None, None, 4.0, 2, 8, 4, True)
    res = got[:, 8:].cpu()
    grid4 = ((pos.cpu() % 4).sum(-1) == 0)
    assert torch.equal(res[0], grid4[0].nonzero()[:, 0]) and res[0].tolist() == [0, 4, 32, 36]
    assert torch.equal(res[1, :3], grid4[1].nonzero()[:, 0]) and int(res[1, 3]) == -1
    assert int(got[:, :8].min()) >= 0
    rows = _native.merge_rows(got, pos)[0]
    assert torch.equal(rows[1, 8 + 3], pos[1, 0]) and torch.equal(rows[1, 8 + 2], pos[1, 36])
    few = _native.merge_centres(pos, None, None, 4.0, 2, 8, 2, True)           # more reserved tokens than slots
    assert torch.equal(few[:, 8:].cpu(), torch.stack([grid4[b].nonzero()[:2, 0] for b in range(2)]))
    monkeypatch.setenv("CLUSTEN_DEBUG_INDICES", "1")
    with pytest.raises(RuntimeError, match="fewer than reserve_num"):
        _native.merge_centres(pos, None, None, 4.0, 2, 8, 4, True)
    _native.merge_centres(pos, None, None, 4.0, 2, 8, 3, True)


@pytest.mark.parametrize("with_mask", [False, True])
def test_rows_at_the_centres(device, with_mask):
    gen = torch.Generator().manual_seed(11)
    b, n, m, n_out = 3, 500, 48, 125
    pos = torch.randint(0, 56, (b, n, 2), generator=gen).float().to(device)
    member = torch.randint(0, n, (b, n, m), generator=gen).to(device)
    pe = torch.randint(0, 111 * 111, (b, n, m), generator=gen).to(device)
    mask = (torch.rand(b, n, m, generator=gen) > 0.2).to(device=device, dtype=torch.float16)
    centre = torch.stack([torch.randperm(n, generator=gen)[:n_out] for _ in range(b)]).to(device)
    tensors = (pos, member, pe) + ((mask,) if with_mask else ())
    got = _native.merge_rows(centre, *tensors)
    assert len(got) == len(tensors)
    for g, t in zip(got, tensors):
        want = t.gather(1, centre.unsqueeze(2).expand(-1, -1, t.shape[2]))
        assert g.dtype == t.dtype and torch.equal(g, want)
    assert not _native.merge_rows_supported(mask[:, :, :3])                 # rows of 6 bytes
    with pytest.raises(RuntimeError):
        _native.merge_rows(centre, pos, member, pe, mask, pos)              # five tensors


def test_the_model_keeps_the_same_tokens_with_and_without_the_kernel(device):
    from aff.model import ClusterMerging, default_ops
    from types import SimpleNamespace
    ops = default_ops()
    plain = SimpleNamespace(**{k: v for k, v in vars(ops).items() if not k.startswith("merge_centres")})
    b, h, w = 2, 28, 28
    pos = _grid(b, h, w, device)
    prob = torch.rand(b, h * w, 1, generator=torch.Generator().manual_seed(2)).to(device)
    reserve_num = 49
    a = ClusterMerging(32, 64, ops=ops).to(device).select(pos, prob, 2, reserve_num)
    c = ClusterMerging(32, 64, ops=plain).to(device).select(pos, prob, 2, reserve_num)
    assert torch.equal(a.sort(1)[0], c.sort(1)[0])
    assert torch.equal(a[:, -reserve_num:], c[:, -reserve_num:])
    sub = _subset(b, 28, 28, 196, 4, device)
    prob = prob[:, :196]
    a = ClusterMerging(32, 64, ops=ops).to(device).select(sub, prob, 4, 10)
    c = ClusterMerging(32, 64, ops=plain).to(device).select(sub, prob, 4, 10)
    assert torch.equal(a[:, :-10].sort(1)[0], c[:, :-10].sort(1)[0])
