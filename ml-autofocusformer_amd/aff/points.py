"""Token geometry around the CLUSTEN operators: nearest neighbours and the balanced clustering that makes the
neighbourhood lists (`nbhd_idx`) the operators consume.

Counterparts of `knn_keops` (models/point_utils.py:27-58) and of the default path of `space_filling_cluster`
(models/point_utils.py:61-208: scan-line anchors, `sf_type=''`, `use_anchor=True`).  The Peano and Hilbert
orders and the anchor-free variant of the reference are not built: no shipped configuration selects them.
All results are integer index tensors or positions; nothing here is differentiated.
"""
import math

import torch


def knn(query, database, k, return_dist=False, chunk_elems=1 << 27):
    """The k database points nearest to each query point, nearest first.

    query (b, n_, d), database (b, n, d) -> indices (b, n_, k) int64 [, Euclidean distances (b, n_, k)].
    Closed form of `knn_keops` (point_utils.py:27-58): distance = sqrt(sum((q - x)^2)), k smallest, ascending.
    Equal distances are ordered by database index (the reference leaves that order to its library).
    The distance matrix is built from explicit differences, so integer positions give exact squared
    distances, and in batch chunks so that at most `chunk_elems` distances exist at a time.  This tensor
    formulation serves CPU tensors (and k > 8 or other than 2-D points on the GPU).
    """
    b, nq, _ = query.shape
    n = database.shape[1]
    query = query.detach().float()
    database = database.detach().float()
    if query.is_cuda:
        # on the GPU the search is one scan kernel of the HIP library (same distances, same tie rule)
        from clusten import _native
        if _native.knn2d_supported(query, database, k):
            return _native.knn2d(query, database, k, return_dist=return_dist)
    per_batch = max(1, nq * n)
    step = max(1, chunk_elems // per_batch)
    idx_parts, dist_parts = [], []
    for s in range(0, b, step):
        q = query[s:s + step]
        x = database[s:s + step]
        d2 = None
        for axis in range(q.shape[2]):
            diff = q[:, :, None, axis] - x[:, None, :, axis]
            d2 = diff * diff if d2 is None else d2 + diff * diff
        if k * 8 <= n:
            # few of many: the k smallest of the 64-bit keys (distance bits, index) — non-negative floats order
            # like their bit patterns, so this is the order of the full stable sort without sorting everything
            key = (d2.view(torch.int32).long() << 32) | torch.arange(n, device=d2.device)
            key = torch.topk(key, k, dim=2, largest=False, sorted=True)[0]
            idx = key & 0xFFFFFFFF
            dist = (key >> 32).int().view(torch.float32)
        else:
            dist, idx = torch.sort(d2, dim=2, stable=True)
            dist, idx = dist[:, :, :k], idx[:, :, :k]
        idx_parts.append(idx)
        if return_dist:
            dist_parts.append(dist.sqrt())
    idx = torch.cat(idx_parts) if len(idx_parts) > 1 else idx_parts[0]
    if return_dist:
        return idx, (torch.cat(dist_parts) if len(dist_parts) > 1 else dist_parts[0])
    return idx


def _anchor_grid(n, m, h, w):
    """(rows, cols) of the anchor grid: about one anchor per cluster of m of the n tokens (point_utils.py:91-101)."""
    k = int(math.ceil(n / m))
    side = (h * w / k) ** 0.5
    return int(round(h / side)), int(round(w / side))


def _scanline_anchors(n, m, h, w, device):
    """Anchor grid of the balanced clustering and its boustrophedon order.

    Returns (rank_of_cell (cells,), ordered anchor centres (cells, 2) as (x, y), cell size (2,) as (w, h),
    cells per row).  Follows point_utils.py:91-137: about one anchor per cluster, rows walked left to right
    and right to left alternately.
    """
    rows, cols = _anchor_grid(n, m, h, w)
    cell = torch.tensor([w / cols, h / rows], device=device)          # float32, as torch.Tensor([...]) gives
    ys, xs = torch.meshgrid(torch.arange(rows, device=device), torch.arange(cols, device=device), indexing="ij")
    # even rows ascend in x, odd rows descend; the row pitch of the key is the image width (point_utils.py:125-129)
    key = torch.where(ys % 2 == 0, xs, (w - 1) - xs) + ys * w
    order = key.reshape(-1).sort()[1]                                   # order[r] = cell at rank r
    rank_of_cell = torch.empty_like(order)
    rank_of_cell[order] = torch.arange(order.numel(), device=device)
    cells_xy = torch.stack([xs, ys], dim=2).reshape(-1, 2)[order]
    centres = cells_xy * cell + cell / 2 - 0.5
    return rank_of_cell, centres, cell, cols


def _scanline_ranking(pos, m, h, w):
    """(b, n) order of the tokens along the scan-line walk: the tensor formulation (point_utils.py:139-159)."""
    b, n, d = pos.shape
    rank_of_cell, centres, cell, cols = _scanline_anchors(n, m, h, w, pos.device)
    cells = centres.shape[0]

    # neighbours on the curve, extrapolated linearly past both ends
    prev_c = torch.empty_like(centres)
    next_c = torch.empty_like(centres)
    prev_c[1:] = centres[:cells - 1]
    prev_c[0] = centres[0] - (centres[1] - centres[0])
    next_c[:cells - 1] = centres[1:]
    next_c[cells - 1] = centres[cells - 1] + (centres[cells - 1] - centres[cells - 2])

    cell_xy = (pos / cell).floor()
    cell_id = (cell_xy[..., 0] + cell_xy[..., 1] * cols).long()    # (b, n)
    rank = rank_of_cell[cell_id]                                    # (b, n) position of the cell on the curve
    dist_prev = (pos - prev_c[rank]).pow(2).sum(-1)
    dist_next = (pos - next_c[rank]).pow(2).sum(-1)
    ratio = dist_prev / (dist_next + 1e-5)
    key = rank * (ratio.max() + 1) + ratio                          # one float key; max over the whole batch
    ranking = key.sort(dim=1, stable=True)[1]                       # (b, n)
    return ranking


def space_filling_cluster(pos, m, h, w, no_reorder=False):
    """Balanced clusters of `m` consecutive tokens along a scan-line space-filling order.

    pos (b, n, 2) token positions as (x, y) inside an h x w canvas.  Returns, as the reference does
    (point_utils.py:61-208):
      no_reorder=False: (pos reordered (b,n,2), cluster centres (b,k,2), member_idx (b,k,m), mask (b,k,m) or None,
                         ranking (b,n,1)) — token `ranking[b,i]` of the input is token i of the new order, cluster g
                         owns tokens g*m .. g*m+m-1, pad slots of the last cluster hold index 0 and mask 0;
      no_reorder=True:  (cluster centres, member_idx in the input's order, mask).
    Each token is assigned to the anchor cell it falls in; within a cell tokens are ordered by the ratio of
    their squared distances to the previous and the next anchor on the curve (point_utils.py:139-159).
    """
    with torch.no_grad():
        pos = pos.detach().float()
        b, n, d = pos.shape
        k = int(math.ceil(n / m))
        ranking = None
        if pos.is_cuda:
            # on the GPU the ranking is two kernels of the HIP library (same float operations, same order)
            from clusten import _native
            rows, cols = _anchor_grid(n, m, h, w)
            if _native.scanline_rank_supported(pos, rows, cols):
                ranking = _native.scanline_rank(pos, rows, cols, w / cols, h / rows)
        if ranking is None:
            ranking = _scanline_ranking(pos, m, h, w)

        if pos.is_cuda and d == 2:
            # the positions in cluster order and the cluster centres from one kernel of the HIP library
            from clusten import _native
            pos, cluster_centres = _native.cluster_centres(pos, ranking, m)
            mask = None
            if k * m != n:
                mask = (torch.arange(k * m, device=pos.device) < n).to(torch.int64).reshape(1, k, m).expand(b, -1, -1)
        else:
            pos = pos.gather(1, ranking.unsqueeze(2).expand(-1, -1, d))
            if k * m == n:
                mask = None
                cluster_centres = pos.reshape(b, k, m, d).mean(2)
            else:
                padded = pos.new_zeros(b, k * m, d)
                padded[:, :n] = pos
                mask = torch.zeros(b, k * m, dtype=torch.int64, device=pos.device)
                mask[:, :n] = 1
                mask = mask.reshape(b, k, m)
                cluster_centres = padded.reshape(b, k, m, d).sum(2) / mask.sum(2, keepdim=True)

        if no_reorder:
            member_idx = torch.zeros(b, k * m, dtype=torch.int64, device=pos.device)
            member_idx[:, :n] = ranking
            return cluster_centres, member_idx.reshape(b, k, m), mask
        member_idx = torch.arange(k * m, device=pos.device)
        member_idx[n:] = 0
        member_idx = member_idx.reshape(1, k, m).expand(b, -1, -1)
        return pos, cluster_centres, member_idx, mask, ranking.unsqueeze(2)
