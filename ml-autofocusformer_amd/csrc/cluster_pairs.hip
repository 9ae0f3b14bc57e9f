// cluster_pairs: the pair lists the cluster-by-cluster scatters read (scatter_by_cluster.hip, wf_dfeat_by_cluster.hip),
// built on the device from the neighbour lists themselves — nothing is read back by the host, so the backward entry
// points never synchronise and take the same kernels on every call.
//
// Lists made of whole clusters: nbhd_idx[b,i,8r+t] = 8 c(b,i,r) + t for every run r of 8 slots (the lists of
// models/aff_transformer.py:476-480; the short last cluster of a sequence whose length is not a multiple of 8 is
// followed by pad slots that hold row 0, models/point_utils.py:203-206).  For such lists
//   keys[(b*N + i)*R + r] = c(b,i,r)                                       (cluster_keys_kernel; R = M/8)
//   pairs[starts[b*K+g] .. ends[b*K+g]) = the entries i*8 + r with c(b,i,r) = g, ascending   (cluster_sort_kernel)
// Any other run sets *not_whole, which the consumers read on the device: the cluster-by-cluster kernels return at
// once when it is set, the atomic kernels when it is clear.
//
// The sort is a stable counting sort per image, one workgroup each: per-wave histograms in LDS over the image's K
// clusters, a scan over (cluster, wave), and a second walk in which every wave places its contiguous share of the
// entries in order (lanes that hold the same key in one step are ranked with a ballot).  The order inside a cluster's
// list is therefore fixed — ascending (i, r) — and so is the order of the sums that read it.
// A pair that names the short last cluster feeds row 0 with its pad slots: it is listed a second time, flagged
// (kPadEntry), after the regular pairs of cluster 0 of its image.
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kPadEntry = 1 << 30;
constexpr int kSortLdsBytes = 60000;

__global__ __launch_bounds__(64) void clear_flag_kernel(int32_t* flag) {
    if (threadIdx.x == 0) *flag = 0;
}

// One thread per run: 64 bytes of the list.  Workgroups that start after the flag is up have nothing left to find.
__global__ __launch_bounds__(256) void cluster_keys_kernel(const int64_t* __restrict__ idx, int32_t* __restrict__ keys,
                                                           int32_t* not_whole, int D, int64_t runs) {
    if (*static_cast<volatile int32_t*>(not_whole) != 0) return;
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= runs) return;
    const int64_t* run = idx + e * 8;
    const int64_t head = run[0];
    // a whole cluster, or the short last one (D % 8 rows) followed by pad slots that hold row 0
    const int own = (head == D - (D & 7)) ? (D & 7) : 8;
    bool ok = (head & 7) == 0 && head >= 0 && head < D;
#pragma unroll
    for (int t = 1; t < 8; ++t) ok = ok && run[t] == (t < own ? head + t : 0);
    keys[e] = ok ? (int32_t)(head >> 3) : 0;
    if (!ok) atomicOr(not_whole, 1);
}

// Exclusive scan of one value per thread over the workgroup; `scratch` holds one int per wave.  Returns the sum of
// the values of the threads before this one; *total receives the sum over the workgroup.
__device__ __forceinline__ int block_exclusive_scan(int v, int* scratch, int* total) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, W = blockDim.x >> 6;
    int inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(inc, d);
        if (lane >= d) inc += up;
    }
    if (lane == 63) scratch[w] = inc;
    __syncthreads();
    int before = 0, all = 0;
    for (int k = 0; k < W; ++k) {
        const int t = scratch[k];
        if (k < w) before += t;
        all += t;
    }
    __syncthreads();
    *total = all;
    return before + inc - v;
}

// One workgroup per image.  E entries (i, r) of the image in the order e = i*R + r; K clusters; `cap` entries of
// `pairs` per image (2E when the sequence ends in a short cluster, else E).
__global__ __launch_bounds__(1024) void cluster_sort_kernel(const int32_t* __restrict__ keys,
                                                            const int32_t* __restrict__ not_whole,
                                                            int32_t* __restrict__ pairs, int32_t* __restrict__ starts,
                                                            int32_t* __restrict__ ends, int E, int R, int K, int cap,
                                                            int pad) {
    if (*not_whole != 0) return;
    extern __shared__ int32_t lds[];
    const int W = blockDim.x >> 6, w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int* hist = lds;              // [W][K]: count, then the start inside the key's list, of wave w's entries of key k
    int* base = lds + W * K;      // [K]: the key's total, then the start of its list inside the image
    int* scratch = base + K;      // [W]
    const int b = blockIdx.x;
    const int32_t* my_keys = keys + (int64_t)b * E;
    const int share = (((E + W - 1) / W + 63) / 64) * 64;   // entries per wave, in whole steps of 64
    const int lo = min(E, w * share), hi = min(E, lo + share);

    for (int z = threadIdx.x; z < W * K; z += blockDim.x) hist[z] = 0;
    __syncthreads();
    for (int e = lo + lane; e < hi; e += 64) atomicAdd(&hist[w * K + my_keys[e]], 1);
    __syncthreads();
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        int run = 0;
        for (int v = 0; v < W; ++v) {
            const int c = hist[v * K + k];
            hist[v * K + k] = run;
            run += c;
        }
        base[k] = run;
    }
    __syncthreads();
    const int regular0 = base[0];
    const int extra = pad ? base[K - 1] : 0;   // pairs of the short last cluster, listed again under cluster 0
    __syncthreads();
    // every thread scans a contiguous range of clusters
    const int per = (K + blockDim.x - 1) / blockDim.x;
    const int k_lo = min(K, (int)threadIdx.x * per), k_hi = min(K, k_lo + per);
    int mine = 0;
    for (int k = k_lo; k < k_hi; ++k) mine += base[k] + (k == 0 ? extra : 0);
    int total;
    int at = block_exclusive_scan(mine, scratch, &total);
    for (int k = k_lo; k < k_hi; ++k) {
        const int n = base[k] + (k == 0 ? extra : 0);
        base[k] = at;
        starts[(int64_t)b * K + k] = b * cap + at;
        ends[(int64_t)b * K + k] = b * cap + at + n;
        at += n;
    }
    __syncthreads();
    int32_t* out = pairs + (int64_t)b * cap;
    const int again_at = base[0] + regular0;       // where the flagged copies go
    for (int e0 = lo; e0 < hi; e0 += 64) {
        const int e = e0 + lane;
        const bool valid = e < hi;
        const int k = valid ? my_keys[e] : -1;
        const int entry = (e / R) * 8 + e % R;
        uint64_t remaining = __ballot(valid);
        while (remaining != 0) {
            const int sl = __builtin_ctzll(remaining);
            const int ks = __builtin_amdgcn_readlane(k, sl);
            const bool hit = k == ks;
            const uint64_t match = __ballot(hit);
            const int rank = __popcll(match & ((1ull << lane) - 1));
            const int cur = hist[w * K + ks];
            if (hit) {
                out[base[ks] + cur + rank] = entry;
                if (pad && ks == K - 1) out[again_at + cur + rank] = entry | kPadEntry;
            }
            lds_sync();
            if (lane == sl) hist[w * K + ks] = cur + __popcll(match);
            lds_sync();
            remaining &= ~match;
        }
    }
}

}  // namespace

bool cluster_pairs_supported(int B, int rows, int M, int D) {
    if (B <= 0 || rows <= 0 || M <= 0 || M % 8 != 0 || M > 64 || D < 8) return false;
    const int64_t R = M / 8, K = (D + 7) / 8;
    const int64_t E = (int64_t)rows * R;
    if (rows >= (1 << 26) || 2 * E * B >= ((int64_t)1 << 31) || K * B >= ((int64_t)1 << 30)) return false;
    return (2 * K + 16) * 4 + 64 <= kSortLdsBytes;   // at least one wave's histogram fits
}

ClusterPairsLayout cluster_pairs_layout(int B, int rows, int M, int D) {
    ClusterPairsLayout l;
    const size_t R = M / 8, K = (D + 7) / 8, E = (size_t)rows * R;
    const size_t cap = (D % 8) ? 2 * E : E;
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    l.flag = 0;
    l.keys = 256;
    l.pairs = l.keys + up((size_t)B * E * 4);
    l.starts = l.pairs + up((size_t)B * cap * 4);
    l.ends = l.starts + up((size_t)B * K * 4);
    l.bytes = l.ends + up((size_t)B * K * 4);
    return l;
}

int launch_cluster_pairs(const int64_t* idx, int32_t* keys, int32_t* not_whole, int32_t* pairs, int32_t* starts,
                         int32_t* ends, int B, int rows, int M, int D, hipStream_t stream) {
    const int R = M / 8, K = (D + 7) / 8;
    const int64_t E = (int64_t)rows * R;
    const int64_t runs = (int64_t)B * E;
    const int cap = (int)((D % 8) ? 2 * E : E);
    hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(64), 0, stream, not_whole);
    hipLaunchKernelGGL(cluster_keys_kernel, dim3((unsigned)((runs + 255) / 256)), dim3(256), 0, stream, idx, keys, not_whole,
                       D, runs);
    int waves = (kSortLdsBytes / 4 - 16) / K - 1;    // (waves + 1) * K + waves ints of LDS
    waves = waves > 16 ? 16 : waves;
    const int64_t steps = (E + 63) / 64;
    if (waves > steps) waves = (int)steps;
    if (waves < 1) waves = 1;
    const size_t lds = ((size_t)(waves + 1) * K + 16) * 4;
    hipLaunchKernelGGL(cluster_sort_kernel, dim3(B), dim3(64 * waves), lds, stream, keys, not_whole, pairs, starts, ends,
                       (int)E, R, K, cap, (D % 8) ? 1 : 0);
    return launch_status();
}

}  // namespace clusten
