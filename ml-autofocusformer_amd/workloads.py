"""Seeded synthetic inputs for the CLUSTEN benchmark and parity configurations.

Every tensor is generated on the CPU from `torch.Generator().manual_seed(1000 + config_id)` so
that the GPU kernels and the CPU oracle see identical bits; callers move them to the device.

Neighbour-list recipes
  * `windowed_cluster_lists` — tokens are grouped into consecutive clusters of 8; every cluster
    shares ONE list of M distinct indices drawn without replacement from a +-256-token window
    around the cluster centre, clipped to [0, N); drawn independently per batch element.
  * `knn_lists` — the M nearest tokens (Euclidean, ascending) of N' output centres among N tokens
    with positions uniform in [0,1]^2; the centres are the first N' entries of a random permutation.
    No sharing between tokens, no runs: the down-sampling (WF) case.
  * `model_like_lists` — what the model's token geometry produces (reference
    models/aff_transformer.py:476-480): per token, the members of its 6 nearest clusters, i.e. 6
    aligned runs of 8 consecutive indices; tokens of one cluster mostly, not always, agree.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

CLUSTER = 8          # tokens per cluster (reference configs/aff_tiny.yaml: CLUSTER_SIZE 8)
NBHD = 48            # neighbours per token (NBHD_SIZE 48)
WINDOW = 256         # half-width of the sampling window of windowed_cluster_lists


def generator(config_id: int) -> torch.Generator:
    return torch.Generator().manual_seed(1000 + config_id)


def windowed_cluster_lists(B: int, N: int, M: int, gen: torch.Generator, cluster: int = CLUSTER,
                           window: int = WINDOW) -> torch.Tensor:
    """(B,N,M) int64 lists shared by the tokens of each cluster of `cluster` consecutive tokens."""
    if N < M:
        raise ValueError("need at least M tokens to draw M distinct neighbours")
    G = (N + cluster - 1) // cluster
    centre = torch.arange(G) * cluster + cluster // 2
    lo = (centre - window).clamp_(min=0)
    hi = (centre + window).clamp_(max=N)
    # window shorter than M (only when N itself is barely above M): widen it to M tokens inside [0,N)
    short = (hi - lo) < M
    lo = torch.where(short, (hi - M).clamp_(min=0), lo)
    hi = torch.where(short, (lo + M).clamp_(max=N), hi)
    width = 2 * window
    offs = torch.arange(width)
    cand = lo[:, None] + offs[None, :]                      # (G, width) candidate token ids
    valid = cand < hi[:, None]
    out = torch.empty(B, G, M, dtype=torch.int64)
    for b in range(B):                                      # per batch element: bounded memory
        keys = torch.rand(G, width, generator=gen)
        keys.masked_fill_(~valid, 2.0)                      # invalid candidates sort last
        order = keys.argsort(dim=1)[:, :M]                  # random-key argsort = draw without replacement
        out[b] = cand.gather(1, order)
    lists = out.repeat_interleave(cluster, dim=1)[:, :N].contiguous()
    return lists


def knn_lists(B: int, N: int, Nout: int, M: int, gen: torch.Generator, chunk: int = 8) -> torch.Tensor:
    """(B,Nout,M) int64: the M nearest of N uniformly placed tokens for Nout randomly chosen centres."""
    if N < M:
        raise ValueError("need at least M tokens")
    out = torch.empty(B, Nout, M, dtype=torch.int64)
    for s in range(0, B, chunk):
        e = min(B, s + chunk)
        pos = torch.rand(e - s, N, 2, generator=gen)
        perm = torch.rand(e - s, N, generator=gen).argsort(dim=1)[:, :Nout]
        centres = pos.gather(1, perm[:, :, None].expand(-1, -1, 2))
        dist = torch.cdist(centres, pos)
        out[s:e] = dist.topk(M, dim=2, largest=False, sorted=True).indices
    return out


def model_like_lists(B: int, N: int, gen: torch.Generator, cluster: int = CLUSTER, nnc: int = 6,
                     canonical: bool = False) -> torch.Tensor:
    """(B,N,nnc*cluster) int64: per token the members of its `nnc` nearest clusters on a sqrt(N) grid
    whose tokens are ordered in scan-line clusters.  N must be a multiple of `cluster`.

    The clusters of a token come nearest first, as a k-nearest-neighbour search returns them, so two
    tokens with the same 6 clusters usually list them in different orders.  `canonical=True` sorts
    each token's clusters by id instead: attention does not depend on the slot order, and tokens
    with the same set of clusters then carry identical lists."""
    if N % cluster:
        raise ValueError("N must be a multiple of the cluster size")
    side = int(math.ceil(math.sqrt(N)))
    ids = torch.arange(N)
    pos = torch.stack([(ids // side).float(), (ids % side).float()], dim=1)          # (N,2)
    G = N // cluster
    out = torch.empty(B, N, nnc * cluster, dtype=torch.int64)
    member = torch.arange(N).reshape(G, cluster)
    for b in range(B):
        jitter = pos + 0.25 * torch.rand(N, 2, generator=gen)
        mean = jitter.reshape(G, cluster, 2).mean(dim=1)                              # cluster centres
        near = torch.cdist(jitter, mean).topk(nnc, dim=1, largest=False, sorted=True).indices  # (N,nnc)
        if canonical:
            near = near.sort(dim=1).values
        out[b] = member[near].reshape(N, nnc * cluster)
    return out


def model_built_geometry(B: int, N: int, gen: torch.Generator, cluster: int = CLUSTER, nnc: int = 6,
                         keep: float = 0.77):
    """((B,N,nnc*cluster) int64 lists, (B,N,nnc*cluster) int64 position indices, rows of the position table) built
    the way the reference model builds them for a stage of adaptively kept tokens (models/aff_transformer.py:454-487):
    per image N tokens at distinct integer positions of a square canvas (a random `keep` of its pixels), ordered and
    cut into clusters by the balanced clustering (`aff.points.space_filling_cluster`), each token listing the members
    of the `nnc` clusters whose centres are nearest, nearest first; the pad slots of a short last cluster hold row 0.
    The position index of (token, slot) is the offset between the two positions as a row of a (2 side - 1)^2 table
    (:483-485): neighbours are near, so a tile's indices fall into a few dozen adjacent rows of the table.
    Unlike `model_like_lists` (strips of a regular grid) neighbouring clusters here are neighbours in the plane, as
    in the model."""
    from aff.points import knn, space_filling_cluster
    side = int(math.ceil(math.sqrt(N / keep)))
    radius, width = side - 1, 2 * side - 1
    ys, xs = torch.meshgrid(torch.arange(side), torch.arange(side), indexing="ij")
    canvas = torch.stack([xs.reshape(-1), ys.reshape(-1)], dim=1).float()
    out = torch.empty(B, N, nnc * cluster, dtype=torch.int64)
    pe = torch.empty(B, N, nnc * cluster, dtype=torch.int64)
    for b in range(B):
        pos = canvas[torch.randperm(side * side, generator=gen)[:N].sort().values][None]
        pos, centres, _, _, _ = space_filling_cluster(pos, cluster, side, side)
        near = knn(pos, centres, nnc)[0]                                              # (N,nnc)
        rows = near.unsqueeze(2) * cluster + torch.arange(cluster)
        out[b] = torch.where(rows < N, rows, torch.zeros_like(rows)).reshape(N, nnc * cluster)
        rel = pos[0][out[b]] - (pos[0][:, None, :] - radius)                          # (N,M,2), every entry in [0, width)
        pe[b] = (rel[..., 1] * width + rel[..., 0]).long()
    return out, pe, width * width


def model_built_lists(B: int, N: int, gen: torch.Generator, cluster: int = CLUSTER, nnc: int = 6,
                      keep: float = 0.77) -> torch.Tensor:
    """The lists of `model_built_geometry` alone."""
    return model_built_geometry(B, N, gen, cluster, nnc, keep)[0]


@dataclass
class AttnCase:
    """Inputs of one QK / AV problem."""
    name: str
    query: torch.Tensor      # (B,H,N,C)
    key: torch.Tensor        # (B,H,N,C)
    value: torch.Tensor      # (B,H,N,C)
    nbhd_idx: torch.Tensor   # (B,N,M)

    def to(self, device):
        return AttnCase(self.name, self.query.to(device), self.key.to(device), self.value.to(device),
                        self.nbhd_idx.to(device))


@dataclass
class WfCase:
    """Inputs of one WF problem."""
    name: str
    weights: torch.Tensor    # (B,Nout,M,IC)
    feat: torch.Tensor       # (B,N,C)
    nbhd_idx: torch.Tensor   # (B,Nout,M)

    def to(self, device):
        return WfCase(self.name, self.weights.to(device), self.feat.to(device), self.nbhd_idx.to(device))


def run_lists(B: int, N: int, M: int, gen, kind: str = "clusters", spread: int = 12) -> torch.Tensor:
    """Lists made of runs of 8 slots, the shape the model's neighbourhoods have, with the irregularities real
    sequences show.  Token i draws its M/8 runs from the `spread` clusters around its own.

      clusters   every run is the 8 members 8g..8g+7 of a cluster, clusters distinct per token
      unaligned  runs of 8 consecutive rows starting anywhere
      padded     as clusters, but a last cluster of N % 8 (or 4) members whose other slots hold index 0
      scattered  every token draws from the whole sequence: few runs are common to the tokens of a tile
      repeated   as clusters, and every token's second run repeats its first
    """
    R = M // 8
    assert M % 8 == 0 and N >= 8 * R
    G = (N + 7) // 8 if kind == "padded" else N // 8   # clusters to draw from (whole ones unless padded)
    own = (torch.arange(N) // 8).clamp(max=G - 1)
    lo = (own - spread // 2).clamp(min=0, max=max(G - spread, 0))
    width = min(spread, G) if kind != "scattered" else G
    if kind == "scattered":
        lo = torch.zeros_like(lo)
    keys = torch.rand(B, N, width, generator=gen)
    pick = keys.argsort(dim=2)[:, :, :R] + lo.view(1, N, 1)            # (B, N, R) distinct clusters
    if kind == "repeated" and R > 1:
        pick[:, :, 1] = pick[:, :, 0]
    base = pick * 8
    if kind == "unaligned":
        base = (base + torch.randint(0, 8, base.shape, generator=gen)).clamp(max=N - 8)
    idx = (base.unsqueeze(3) + torch.arange(8).view(1, 1, 1, 8)).reshape(B, N, M)
    if kind == "padded":
        tail = N % 8 if N % 8 else 4              # members of the short last cluster
        last = (N - 1) // 8 * 8
        run = torch.arange(last, last + 8)
        run[tail:] = 0
        hit = (idx.reshape(B, N, R, 8)[..., 0] == last)
        idx = torch.where(hit.unsqueeze(3), run.view(1, 1, 1, 8), idx.reshape(B, N, R, 8)).reshape(B, N, M)
    return idx.contiguous()


def attn_case(name: str, config_id: int, B: int, H: int, N: int, C: int, M: int = NBHD, dtype=torch.float32,
              scale_q: bool = True, lists: str = "windowed") -> AttnCase:
    gen = generator(config_id)
    q = torch.randn(B, H, N, C, generator=gen)
    k = torch.randn(B, H, N, C, generator=gen)
    v = torch.randn(B, H, N, C, generator=gen)
    if scale_q:
        q = q * (C ** -0.5)
    if lists == "windowed":
        idx = windowed_cluster_lists(B, N, M, gen)
    elif lists == "model":
        idx = model_like_lists(B, N, gen)
    elif lists == "model_built":
        idx = model_built_lists(B, N, gen)
    elif lists == "model_canonical":
        idx = model_like_lists(B, N, gen, canonical=True)
    elif lists == "random":
        idx = torch.randint(N, (B, N, M), generator=gen)
    elif lists.startswith("runs:"):
        idx = run_lists(B, N, M, gen, kind=lists[5:])
    else:
        raise ValueError(lists)
    return AttnCase(name, q.to(dtype), k.to(dtype), v.to(dtype), idx)


def wf_case(name: str, config_id: int, B: int, N: int, C: int, IC: int = 4, M: int = NBHD, dtype=torch.float32,
            Nout: int | None = None) -> WfCase:
    gen = generator(config_id)
    Nout = N // 4 if Nout is None else Nout
    feat = torch.randn(B, N, C, generator=gen)
    w = torch.rand(B, Nout, M, IC, generator=gen)
    w = w / w.sum(dim=2, keepdim=True)
    idx = knn_lists(B, N, Nout, M, gen)
    return WfCase(name, w.to(dtype), feat.to(dtype), idx)


# ---- the BASELINE configurations ------------------------------------------------------------------

# (embedding dim, heads, tokens) of the four AFF-Tiny stages at 224x224 (reference configs/aff_tiny.yaml)
AFF_TINY_STAGES = ((64, 2, 3136), (128, 4, 784), (256, 8, 196), (512, 16, 49))


def config0() -> AttnCase:
    """CPU plumbing case: B2 H2 N1024 C32 M48 fp32, Q and K ~ N(0,1) (no scaling)."""
    return attn_case("cfg0", 0, B=2, H=2, N=1024, C=32, scale_q=False)


def config1(dtype=torch.float32, B: int = 256) -> AttnCase:
    """AFF-Mini stage 1: B256 H2 N3136 C16 M48."""
    return attn_case("cfg1", 1, B=B, H=2, N=3136, C=16, dtype=dtype)


def config2_attn(stage: int, B: int = 128) -> AttnCase:
    """AFF-Tiny stage `stage` (1-based) QK/AV inputs, fp32."""
    dim, heads, n = AFF_TINY_STAGES[stage - 1]
    return attn_case("cfg2_s%d" % stage, 2 * 10 + stage, B=B, H=heads, N=n, C=dim // heads)


def config2_wf(stage: int, IC: int = 4, B: int = 128) -> WfCase:
    """AFF-Tiny stage `stage` (1-based) WF inputs: N -> N/4 tokens, C = embedding dim, fp32."""
    dim, _, n = AFF_TINY_STAGES[stage - 1]
    return wf_case("cfg2_s%d_wf_ic%d" % (stage, IC), 2 * 10 + 4 + stage, B=B, N=n, C=dim, IC=IC)


def config3_attn(dtype=torch.bfloat16, B: int = 64) -> AttnCase:
    """AFF-Base 384x384 stage 1: B64 H4 N9216 C32 M48."""
    return attn_case("cfg3", 3, B=B, H=4, N=9216, C=32, dtype=dtype)


def config3_wf(dtype=torch.bfloat16, IC: int = 4, B: int = 64) -> WfCase:
    """AFF-Base 384x384 stage 1 WF: 9216 -> 2304 tokens, C = 128."""
    return wf_case("cfg3_wf_ic%d" % IC, 34, B=B, N=9216, C=128, IC=IC, dtype=dtype)


# ---- algorithmic bytes and flops (each input read once, each output written once) -----------------

def attn_bytes(B, H, N, C, M, elem_size) -> int:
    """QK forward = AV forward: two (B,H,N,C) tensors, one (B,H,N,M) tensor, int64 lists."""
    return 2 * B * H * N * C * elem_size + B * N * M * 8 + B * H * N * M * elem_size


def wf_bytes(B, N, Nout, C, M, IC, elem_size) -> int:
    return (B * Nout * M * IC + B * N * C + B * Nout * IC * C) * elem_size + B * Nout * M * 8


def attn_flops(B, H, N, C, M) -> int:
    return 2 * B * H * N * M * C


def wf_flops(B, Nout, C, M, IC) -> int:
    return 2 * B * Nout * M * IC * C
