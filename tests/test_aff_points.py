"""Neighbourhood producer: balanced clustering against vectors taken from the reference, kNN against brute force."""
import os

import numpy as np
import pytest
import torch

from aff.points import knn, space_filling_cluster, _anchor_grid, _scanline_anchors, _scanline_ranking

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "space_filling_cluster.npz")
CASES = ["grid56", "grid14", "sub784", "sub196", "sub49", "ref_script", "wide", "grid96"]


def _load(name):
    z = np.load(GOLDEN)
    pos = torch.from_numpy(z[name + ".pos"].astype(np.int64))
    m, h, w = (int(v) for v in z[name + ".mhw"])
    return z, pos, m, h, w


def _ranking_key(pos, m, h, w):
    """The float key the tokens are sorted by, recomputed from the module's own pieces."""
    pos = pos.float()
    n = pos.shape[1]
    rank_of_cell, centres, cell, cols = _scanline_anchors(n, m, h, w, pos.device)
    cells = centres.shape[0]
    prev_c = torch.cat([(centres[0] - (centres[1] - centres[0]))[None], centres[:cells - 1]])
    next_c = torch.cat([centres[1:], (centres[-1] + (centres[-1] - centres[-2]))[None]])
    cxy = (pos / cell).floor()
    rank = rank_of_cell[(cxy[..., 0] + cxy[..., 1] * cols).long()]
    ratio = (pos - prev_c[rank]).pow(2).sum(-1) / ((pos - next_c[rank]).pow(2).sum(-1) + 1e-5)
    return rank * (ratio.max() + 1) + ratio


@pytest.mark.parametrize("name", CASES)
def test_ranking_matches_the_reference_up_to_the_order_of_equal_keys(name):
    z, pos, m, h, w = _load(name)
    new_pos, centres, member_idx, mask, ranking = space_filling_cluster(pos, m, h, w)
    mine = ranking.squeeze(2)
    gold = torch.from_numpy(z[name + ".ranking"].astype(np.int64))
    b, n = gold.shape
    # both are permutations
    assert torch.equal(mine.sort(1)[0], torch.arange(n).expand(b, -1))
    key = _ranking_key(pos, m, h, w)
    k_mine, k_gold = key.gather(1, mine), key.gather(1, gold)
    # the reference's order is sorted under this build's key, and the two orders differ only inside
    # groups of exactly equal keys (whose order the reference leaves to an unstable sort)
    assert bool((k_gold[:, 1:] >= k_gold[:, :-1]).all())
    assert torch.equal(k_mine, k_gold)
    differs = mine != gold
    if name == "sub49":
        assert not differs.any()
    # members and mask do not depend on the tie order
    assert np.array_equal(member_idx.numpy(), z[name + ".member_idx"])
    gm = z[name + ".mask"]
    assert (mask is None and gm.size == 0) or np.array_equal(mask.numpy(), gm)
    # clusters that no tie touches have the reference's centre exactly
    k = member_idx.shape[1]
    pad = k * m - n
    d = torch.cat([differs, differs.new_zeros(b, pad)], 1).reshape(b, k, m).any(2)
    same = ~d
    assert same.float().mean() > 0.5
    assert torch.equal(centres[same], torch.from_numpy(z[name + ".centres"])[same])
    assert torch.equal(new_pos[~differs], torch.from_numpy(z[name + ".new_pos"])[~differs])


@pytest.mark.parametrize("name", ["sub196", "wide"])
def test_no_reorder_returns_members_in_input_order(name):
    z, pos, m, h, w = _load(name)
    centres, member_idx, mask = space_filling_cluster(pos, m, h, w, no_reorder=True)
    _, centres_r, _, mask_r, ranking = space_filling_cluster(pos, m, h, w)
    b, n = pos.shape[:2]
    assert torch.equal(member_idx.reshape(b, -1)[:, :n], ranking.squeeze(2))
    assert torch.equal(centres, centres_r)
    assert (member_idx.reshape(b, -1)[:, n:] == 0).all()


def test_clusters_are_balanced_and_compact():
    torch.manual_seed(3)
    h = w = 56
    pos = torch.stack([torch.randperm(h * w)[:784] for _ in range(2)])
    pos = torch.stack([pos % w, pos // w], dim=2)
    new_pos, centres, member_idx, mask, ranking = space_filling_cluster(pos, 8, h, w)
    assert mask is None and centres.shape == (2, 98, 2)
    # members of cluster g are tokens 8g..8g+7 and the centre is their mean
    assert torch.equal(member_idx[0].reshape(-1), torch.arange(784))
    assert torch.allclose(centres, new_pos.reshape(2, 98, 8, 2).mean(2))
    # compact: a cluster's members are near its centre (the canvas diagonal is 79)
    spread = (new_pos.reshape(2, 98, 8, 2) - centres[:, :, None]).norm(dim=-1)
    assert spread.mean() < 4.0


def test_knn_against_brute_force_and_tie_order():
    torch.manual_seed(5)
    q = torch.randint(0, 20, (3, 37, 2)).float()
    x = torch.randint(0, 20, (3, 53, 2)).float()
    idx, dist = knn(q, x, 6, return_dist=True)
    for b in range(3):
        for i in range(37):
            d2 = [(float(((q[b, i] - x[b, j]) ** 2).sum()), j) for j in range(53)]
            d2.sort()
            assert [j for _, j in d2[:6]] == idx[b, i].tolist()
            assert np.allclose([v ** 0.5 for v, _ in d2[:6]], dist[b, i].numpy())
    # chunking over the batch does not change the result
    idx2 = knn(q, x, 6, chunk_elems=37 * 53)
    assert torch.equal(idx, idx2)
    # a token's nearest neighbour in its own set is itself when positions are distinct
    p = torch.stack([torch.randperm(400)[:100] for _ in range(2)])
    p = torch.stack([p % 20, p // 20], 2).float()
    self_idx, self_d = knn(p, p, 2, return_dist=True)
    assert torch.equal(self_idx[:, :, 0], torch.arange(100).expand(2, -1))
    assert (self_d[:, :, 0] == 0).all() and (self_d[:, :, 1] >= 1).all()


@pytest.mark.gpu
@pytest.mark.parametrize("k", [1, 2, 6, 8])
def test_knn_kernel_equals_the_tensor_formulation(device, k):
    from clusten import _native
    gen = torch.Generator().manual_seed(9)
    for nq, n in ((784, 98), (784, 784), (3136, 392), (37, 2500), (5, 8)):
        # integer and eighth-of-a-pixel positions: many exactly equal distances
        q = torch.randint(0, 56, (3, nq, 2), generator=gen).float()
        x = torch.randint(0, 56 * 8, (3, n, 2), generator=gen).float() / 8
        ref_idx, ref_dist = knn(q, x, k, return_dist=True)                 # CPU tensors: the tensor formulation
        idx, dist = _native.knn2d(q.to(device), x.to(device), k, return_dist=True)
        assert torch.equal(idx.cpu(), ref_idx)
        # squared distances are exact here; the two square roots may differ by an ulp
        assert torch.allclose(dist.cpu(), ref_dist, rtol=2.5e-7, atol=0)
        assert torch.equal(knn(q.to(device), x.to(device), k).cpu(), ref_idx)
    assert not _native.knn2d_supported(q.to(device), x.to(device), 9)
    with pytest.raises(RuntimeError):
        _native.knn2d(q, x, 2)


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_ranking_kernel_equals_the_tensor_formulation(device, name):
    """Bit-identical keys, hence the same order: the fixtures' positions and denser random ones."""
    from clusten import _native
    z, pos, m, h, w = _load(name)
    gen = torch.Generator().manual_seed(23)
    more = torch.stack([torch.randperm(h * w, generator=gen)[:pos.shape[1]] for _ in range(5)])
    more = torch.stack([more % w, more // w], dim=2)
    for p in (pos, more, more.float() + torch.rand(more.shape, generator=gen) * 0.99):
        p = p.float()
        ref = _scanline_ranking(p, m, h, w)                                  # CPU tensors: the tensor formulation
        rows, cols = _anchor_grid(p.shape[1], m, h, w)
        assert _native.scanline_rank_supported(p.to(device), rows, cols)
        got = _native.scanline_rank(p.to(device), rows, cols, w / cols, h / rows)
        assert got.dtype == torch.int64 and torch.equal(got.cpu(), ref)
        # and through the public function: same clusters on both devices (positions in cluster order and cluster
        # centres come from one kernel on the GPU; the centres of integer positions are exact on both)
        cpu = space_filling_cluster(p, m, h, w)
        gpu = space_filling_cluster(p.to(device), m, h, w)
        assert torch.equal(gpu[4].cpu(), cpu[4]) and torch.equal(gpu[0].cpu(), cpu[0])
        assert torch.allclose(gpu[1].cpu(), cpu[1], rtol=1e-6, atol=1e-6)
        if float((p - p.round()).abs().max()) == 0.0:
            assert torch.equal(gpu[1].cpu(), cpu[1])
        assert (gpu[3] is None) == (cpu[3] is None) and (cpu[3] is None or torch.equal(gpu[3].cpu(), cpu[3]))
    assert _native.load().clusten_scanline_rank_max_tokens() >= 16384
    assert not _native.scanline_rank_supported(torch.zeros(1, 40000, 2, device=device), 10, 10)
    with pytest.raises(RuntimeError):
        _native.scanline_rank(pos.float(), 4, 4, 1.0, 1.0)


@pytest.mark.gpu
def test_ranking_kernel_on_the_first_stage_of_a_384_model(device):
    """9216 tokens on a 96 x 96 grid, clusters of 24 (configs/aff_base_22kto1k_384.yaml:10): the sort of an image takes
    128 KB of LDS; same order as the tensor formulation, on the grid and on scattered fractional positions."""
    from clusten import _native
    gen = torch.Generator().manual_seed(24)
    ys, xs = torch.meshgrid(torch.arange(96), torch.arange(96), indexing="ij")
    grid = torch.stack([xs, ys], dim=2).reshape(1, -1, 2).float().expand(2, -1, -1).contiguous()
    scattered = torch.rand(2, 9216, 2, generator=gen) * 95.99
    for p in (grid, scattered):
        ref = _scanline_ranking(p, 24, 96, 96)
        rows, cols = _anchor_grid(9216, 24, 96, 96)
        assert _native.scanline_rank_supported(p.to(device), rows, cols)
        got = _native.scanline_rank(p.to(device), rows, cols, 96 / cols, 96 / rows)
        assert torch.equal(got.cpu(), ref)
        cpu = space_filling_cluster(p, 24, 96, 96)
        gpu = space_filling_cluster(p.to(device), 24, 96, 96)
        assert torch.equal(gpu[0].cpu(), cpu[0]) and torch.allclose(gpu[1].cpu(), cpu[1], rtol=1e-6, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_row_gather_kernel(device, dtype):
    from clusten import _native
    gen = torch.Generator().manual_seed(25)
    for b, n, c in ((3, 196, 256), (2, 784, 128), (1, 50, 8 if dtype == torch.float16 else 4)):
        x = torch.randn(b, n, c, generator=gen).to(dtype).to(device)
        order = torch.stack([torch.randperm(n, generator=gen) for _ in range(b)]).to(device)
        assert _native.gather_rows_supported(x)
        want = x.gather(1, order.unsqueeze(2).expand(-1, -1, c))
        assert torch.equal(_native.gather_rows(x, order), want)
        assert torch.equal(_native.gather_rows(x, order[0]), x[:, order[0]])
    assert not _native.gather_rows_supported(torch.zeros(1, 4, 3, device=device))
