"""The synthetic input generators produce what the benchmark configurations describe."""
import os

import torch

import workloads as wl


def test_windowed_lists_are_cluster_shared_distinct_and_local():
    gen = wl.generator(0)
    B, N, M = 3, 1024, 48
    idx = wl.windowed_cluster_lists(B, N, M, gen)
    assert idx.shape == (B, N, M) and idx.dtype == torch.int64
    assert idx.min() >= 0 and idx.max() < N
    g = idx.reshape(B, N // 8, 8, M)
    assert (g == g[:, :, :1]).all()                                    # the 8 tokens of a cluster share the list
    first = g[:, :, 0]
    assert (first.sort(dim=-1).values.diff(dim=-1) > 0).all()          # 48 distinct indices
    centre = (torch.arange(N // 8) * 8 + 4).reshape(1, -1, 1)
    assert ((first - centre).abs() <= 256).all()                       # inside the +-256 window
    assert not (first[0] == first[1]).all()                            # drawn independently per batch element


def test_windowed_lists_small_and_ragged_n():
    gen = wl.generator(1)
    for N in (49, 196, 197):
        idx = wl.windowed_cluster_lists(2, N, 48, gen)
        assert idx.shape == (2, N, 48) and idx.min() >= 0 and idx.max() < N
        assert (idx[:, :8] == idx[:, :1]).all()
        assert (idx[:, 0].sort(dim=-1).values.diff(dim=-1) > 0).all()


def test_generators_are_deterministic():
    a = wl.config0()
    b = wl.config0()
    assert torch.equal(a.query, b.query) and torch.equal(a.nbhd_idx, b.nbhd_idx)
    assert a.query.shape == (2, 2, 1024, 32) and a.nbhd_idx.shape == (2, 1024, 48)


def test_knn_lists_are_the_nearest_neighbours():
    gen = wl.generator(2)
    B, N, Nout, M = 2, 64, 16, 8
    state = gen.get_state()
    idx = wl.knn_lists(B, N, Nout, M, gen)
    gen.set_state(state)
    pos = torch.rand(B, N, 2, generator=gen)
    perm = torch.rand(B, N, generator=gen).argsort(dim=1)[:, :Nout]
    for b in range(B):
        for i in range(Nout):
            d = ((pos[b] - pos[b, perm[b, i]]) ** 2).sum(-1)
            assert set(idx[b, i].tolist()) == set(d.argsort()[:M].tolist())
            assert idx[b, i, 0] == perm[b, i]                          # a centre is its own nearest token


def test_wf_case_shapes_and_normalised_weights():
    c = wl.config2_wf(3, IC=4, B=2)
    assert c.weights.shape == (2, 49, 48, 4) and c.feat.shape == (2, 196, 256) and c.nbhd_idx.shape == (2, 49, 48)
    assert (c.weights >= 0).all()
    torch.testing.assert_close(c.weights.sum(dim=2), torch.ones(2, 49, 4))


def test_model_like_lists_are_six_aligned_runs_of_eight():
    idx = wl.model_like_lists(2, 784, wl.generator(3))
    assert idx.shape == (2, 784, 48)
    runs = idx.reshape(2, 784, 6, 8)
    assert (runs[..., 0] % 8 == 0).all()
    assert (runs == runs[..., :1] + torch.arange(8)).all()
    tiles = idx.reshape(2, 98, 8, 48)
    assert not (tiles == tiles[:, :, :1]).all(dim=-1).all(dim=-1).any()   # nearest-first order differs per token
    canon = wl.model_like_lists(2, 784, wl.generator(3), canonical=True)
    assert torch.equal(canon.sort(dim=-1).values, idx.sort(dim=-1).values)   # same sets, other order
    assert (canon.reshape(2, 784, 6, 8)[..., 0].diff(dim=-1) > 0).all()      # cluster ids ascending


def test_model_built_lists_are_whole_clusters_of_neighbouring_tokens():
    """Lists built by the balanced clustering itself: runs of whole clusters, the token's own cluster first, and
    neighbouring clusters of the sequence sharing their neighbours (what the strips of `model_like_lists` lack)."""
    for cluster, n in ((8, 784), (24, 600)):
        idx = wl.model_built_lists(2, n, wl.generator(4), cluster=cluster, nnc=6)
        assert idx.shape == (2, n, 6 * cluster) and int(idx.min()) >= 0 and int(idx.max()) < n
        runs = idx.reshape(2, n, 6, cluster)
        assert (runs[..., 0] % cluster == 0).all()
        assert (runs == runs[..., :1] + torch.arange(cluster)).all()
        own = torch.arange(n) // cluster
        assert ((runs[..., 0] // cluster == own.view(1, n, 1)).any(dim=-1)).float().mean() > 0.95   # a token lists its own cluster
        ids = runs[..., 0] // cluster                                      # (2, n, 6) cluster numbers
        per_tile = ids[:, :n // cluster * cluster].reshape(2, -1, cluster * 6)
        distinct = torch.tensor([[len(set(r.tolist())) for r in b] for b in per_tile]).float().mean()
        assert 6 < float(distinct) < 14                                    # the tokens of a cluster pick from the same dozen
    # a sequence that does not end on a cluster: pad slots hold row 0
    idx = wl.model_built_lists(1, 100, wl.generator(5), cluster=8, nnc=4)
    last = idx.reshape(1, 100, 4, 8)
    short = last[last[..., 0] == 96]
    assert short.numel() > 0 and (short[:, 4:] == 0).all() and (short[:, :4] == torch.arange(96, 100)).all()


def test_model_built_geometry_gives_the_lists_and_position_indices_of_the_models_own_layer():
    """The benchmark's attention legs take their lists and position indices from `model_built_geometry`: both equal
    what a layer of this build's model (`BasicLayer.neighbourhoods`, models/aff_transformer.py:454-487) computes for
    the same tokens, and the indices of a tile fall into a small part of the table."""
    import math
    from aff.model import BasicLayer
    for cluster, n in ((8, 784), (8, 100), (24, 600)):
        lists, pe, rows = wl.model_built_geometry(2, n, wl.generator(6), cluster=cluster, nnc=6)
        side = int(math.ceil(math.sqrt(n / 0.77)))
        assert rows == (2 * side - 1) ** 2 and lists.shape == pe.shape == (2, n, 6 * cluster)
        assert int(pe.min()) >= 0 and int(pe.max()) < rows
        assert torch.equal(lists, wl.model_built_lists(2, n, wl.generator(6), cluster=cluster, nnc=6))
        # the same canvas positions through the model's layer
        gen = wl.generator(6)
        ys, xs = torch.meshgrid(torch.arange(side), torch.arange(side), indexing="ij")
        canvas = torch.stack([xs.reshape(-1), ys.reshape(-1)], dim=1).float()
        pos = torch.stack([canvas[torch.randperm(side * side, generator=gen)[:n].sort().values] for _ in range(2)])
        layer = BasicLayer(8, 8, cluster, 6 * cluster, depth=0, num_heads=1, mlp_ratio=1.0, downsample=False)
        _, _, member_idx, _, pe_idx, _ = layer.neighbourhoods(pos, side, side, side - 1, 2 * side - 1)
        assert torch.equal(member_idx, lists) and torch.equal(pe_idx, pe)
        # offsets between near tokens: a tile of `cluster` tokens names a small share of the table's rows
        per_tile = pe[0, :n // cluster * cluster].reshape(-1, cluster * 6 * cluster)
        distinct = torch.tensor([len(set((r // (2 * side - 1)).tolist())) for r in per_tile]).float().mean()
        assert float(distinct) < 0.6 * (2 * side - 1)


def test_algorithmic_bytes_match_the_published_table():
    # AFF-Tiny stage 1, fp32: QK = AV = 513.8 MB, WF IC4 = 321.1 MB, IC1 = 186.3 MB
    assert round(wl.attn_bytes(128, 2, 3136, 32, 48, 4) / 1e6, 1) == 513.8
    assert round(wl.wf_bytes(128, 3136, 784, 64, 48, 4, 4) / 1e6, 1) == 321.1
    assert round(wl.wf_bytes(128, 3136, 784, 64, 48, 1, 4) / 1e6, 1) == 186.3
    assert round(wl.attn_bytes(64, 4, 9216, 32, 48, 2) / 1e6, 1) == 755.0
    assert wl.attn_flops(128, 2, 3136, 32, 48) == 2 * 128 * 2 * 3136 * 48 * 32


def test_bench_refuses_more_than_one_gpu_and_needs_one():
    import subprocess
    import sys as _sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([_sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)
