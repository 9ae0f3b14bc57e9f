// cluster_pairs: the pair lists the cluster-by-cluster scatters read (scatter_by_cluster.hip, wf_dfeat_by_cluster.hip),
// built on the device from the neighbour lists themselves — nothing is read back by the host, so the backward entry
// points never synchronise and take the same kernels on every call.
//
// Lists made of whole clusters: nbhd_idx[b,i,8r+t] = 8 c(b,i,r) + t for every run r of 8 slots (the lists of
// models/aff_transformer.py:476-480; the short last cluster of a sequence whose length is not a multiple of 8 is
// followed by pad slots that hold row 0, models/point_utils.py:203-206).  For such lists
//   keys[(b*N + i)*R + r] = c(b,i,r)                                       (cluster_keys_kernel; R = M/8)
//   pairs[starts[b*K+g] .. ends[b*K+g]) = the entries i*32 + r with c(b,i,r) = g, ascending  (cluster_sort_kernel)
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

// Four lanes per run of 8 entries, 16 bytes (two entries) each, so that a wave reads 1 KiB of the lists per access;
// every thread takes kKeysPerThread such pieces, all requested before the first is looked at.
// Every workgroup reports what it found in a word of its own (`wg_bad`), and the sort kernel that follows adds the
// words up: one flag for all would be one address, served by one channel of the L2, and waves that polled it in order
// to leave early, raised it with an atomic each or even just stored to it spent their time queueing at that channel
// (250 us instead of 45 on lists that are not whole clusters).
constexpr int kKeysBlock = 256;
constexpr int kKeysPerThread = 4;
__global__ __launch_bounds__(kKeysBlock) void cluster_keys_kernel(const int64_t* __restrict__ idx,
                                                                  int32_t* __restrict__ keys,
                                                                  int32_t* __restrict__ wg_bad, int D, int64_t runs) {
    typedef long long I64x2 __attribute__((ext_vector_type(2)));
    const int lane = threadIdx.x & 63;
    const int64_t first = (int64_t)blockIdx.x * (kKeysBlock * kKeysPerThread) + threadIdx.x;
    I64x2 two[kKeysPerThread];
#pragma unroll
    for (int u = 0; u < kKeysPerThread; ++u) {
        const int64_t piece = first + u * kKeysBlock;                // two entries
        two[u] = (piece >> 2) < runs ? *reinterpret_cast<const I64x2*>(idx + piece * 2) : I64x2{0, 0};
    }
    bool any_bad = false;
#pragma unroll
    for (int u = 0; u < kKeysPerThread; ++u) {
        const int64_t piece = first + u * kKeysBlock;
        const int64_t e = piece >> 2;                                // the run
        const int q = (int)(piece & 3);                              // which quarter of it
        const bool live = e < runs;
        // the run's first entry, from the first lane of the quad (64-bit shuffle as two halves)
        const int lo = __shfl((int)(two[u][0] & 0xffffffffll), lane & ~3);
        const int hi = __shfl((int)(two[u][0] >> 32), lane & ~3);
        const int64_t head = ((int64_t)hi << 32) | (uint32_t)lo;
        // a whole cluster, or the short last one (D % 8 rows) followed by pad slots that hold row 0
        const int own = (head == D - (D & 7)) ? (D & 7) : 8;
        bool ok = (head & 7) == 0 && head >= 0 && head < D;
        ok = ok && two[u][0] == (2 * q < own ? head + 2 * q : 0) && two[u][1] == (2 * q + 1 < own ? head + 2 * q + 1 : 0);
        const uint64_t bad = __ballot(live && !ok);
        const bool run_ok = ((bad >> (lane & ~3)) & 0xf) == 0;
        if (live && q == 0) keys[e] = run_ok ? (int32_t)(head >> 3) : 0;
        any_bad = any_bad || bad != 0;
    }
    const int found = __syncthreads_or(any_bad);
    if (threadIdx.x == 0) wg_bad[blockIdx.x] = found ? 1 : 0;
}

// The same table of keys from cluster numbers (the lists given as (B,rows,R) int32, R numbers of clusters of 8 rows per
// token): the numbers are the keys; a number outside [0, K) raises the flag.
__global__ __launch_bounds__(kKeysBlock) void cluster_number_keys_kernel(const int32_t* __restrict__ numbers,
                                                                         int32_t* __restrict__ keys,
                                                                         int32_t* __restrict__ wg_bad, int K, int64_t runs) {
    const int64_t first = (int64_t)blockIdx.x * (kKeysBlock * kKeysPerThread) + threadIdx.x;
    bool any_bad = false;
#pragma unroll
    for (int u = 0; u < kKeysPerThread; ++u) {
        const int64_t e = first + u * kKeysBlock;
        if (e < runs) {
            const int c = numbers[e];
            const bool ok = (unsigned)c < (unsigned)K;
            keys[e] = ok ? c : 0;
            any_bad = any_bad || !ok;
        }
    }
    const int found = __syncthreads_or(any_bad);
    if (threadIdx.x == 0) wg_bad[blockIdx.x] = found ? 1 : 0;
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

// The stable counting sort of one image by one workgroup.  E entries in the order e = 0 .. E-1, K keys; the sorted
// entries go to `pairs` (cap per image), the bounds of every key's list to starts / ends.
//   ROWS = false: keys[e] = cluster number of run e = i*R + r, entry = i*32 + r; `pad`: the pairs of the short last
//                 cluster are listed again, flagged, under cluster 0;
//   ROWS = true:  keys64[e] = destination row of list entry e (any row: entries outside [0, K) are left out),
//                 entry = e.
template <bool ROWS>
__device__ __forceinline__ void sort_image(const void* __restrict__ keys_any, int32_t* __restrict__ pairs,
                                           int32_t* __restrict__ starts, int32_t* __restrict__ ends, int E, int R, int K,
                                           int cap, int pad, int key_bits) {
    extern __shared__ int32_t lds[];
    const int W = blockDim.x >> 6, w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int* hist = lds;              // [W][K]: count, then the start inside the key's list, of wave w's entries of key k
    int* base = lds + W * K;      // [K]: the key's total, then the start of its list inside the image
    int* scratch = base + K;      // [W]
    const int b = blockIdx.x;
    const int32_t* keys32 = static_cast<const int32_t*>(keys_any) + (int64_t)b * E;
    const int64_t* keys64 = static_cast<const int64_t*>(keys_any) + (int64_t)b * E;
    auto key_of = [&](int e) -> int {
        if constexpr (ROWS) {
            const int64_t row = keys64[e];
            return (row >= 0 && row < K) ? (int)row : -1;
        } else {
            return keys32[e];
        }
    };
    const int share = (((E + W - 1) / W + 63) / 64) * 64;   // entries per wave, in whole steps of 64
    const int lo = min(E, w * share), hi = min(E, lo + share);

    for (int z = threadIdx.x; z < W * K; z += blockDim.x) hist[z] = 0;
    __syncthreads();
    for (int e0 = lo; e0 < hi; e0 += 4 * 64) {
        int k4[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) k4[u] = e0 + 64 * u + lane < hi ? key_of(e0 + 64 * u + lane) : -1;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (k4[u] >= 0) atomicAdd(&hist[w * K + k4[u]], 1);
        }
    }
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
    for (int e00 = lo; e00 < hi; e00 += 4 * 64) {
        int k4[4];    // four steps' keys requested together
#pragma unroll
        for (int u = 0; u < 4; ++u) k4[u] = e00 + 64 * u + lane < hi ? key_of(e00 + 64 * u + lane) : -1;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = e00 + 64 * u + lane;
            const int k = k4[u];
            const bool valid = k >= 0;
            const int entry = ROWS ? e : ((e / R) << kPairRunBits) + e % R;
            // the lanes of this step that hold the lane's key: one ballot per bit of the key
            uint64_t same = __ballot(valid);
            for (int bit = 0; bit < key_bits; ++bit) {
                const bool one = (k >> bit) & 1;
                const uint64_t ones = __ballot(one);
                same &= one ? ones : ~ones;
            }
            const int rank = __popcll(same & ((1ull << lane) - 1));
            const int group = __popcll(same);
            const int leader = valid ? __builtin_ctzll(same) : lane;
            // the first lane of every group moves its key's cursor (distinct keys: distinct addresses) and tells the others
            int cur = 0;
            if (valid && rank == 0) cur = atomicAdd(&hist[w * K + k], group);
            cur = __shfl(cur, leader);
            if (valid) {
                out[base[k] + cur + rank] = entry;
                if (pad && k == K - 1) out[again_at + cur + rank] = entry | kPadEntry;
            }
        }
    }
}

// One workgroup per image: the pair lists of lists made of whole clusters.
__global__ __launch_bounds__(1024) void cluster_sort_kernel(const int32_t* __restrict__ keys,
                                                            const int32_t* __restrict__ wg_bad, int n_wg_bad,
                                                            int32_t* __restrict__ not_whole,
                                                            int32_t* __restrict__ pairs, int32_t* __restrict__ starts,
                                                            int32_t* __restrict__ ends, int E, int R, int K, int cap,
                                                            int pad, int key_bits) {
    {
        // what the workgroups of the keys kernel found, added up by every workgroup here for itself; the first one
        // writes the flag the later kernels read
        int bad = 0;
        for (int z = threadIdx.x; z < n_wg_bad; z += blockDim.x) bad |= wg_bad[z];
        bad = __syncthreads_or(bad);
        if (blockIdx.x == 0 && threadIdx.x == 0) *not_whole = bad ? 1 : 0;
        if (bad) return;
    }
    sort_image<false>(keys, pairs, starts, ends, E, R, K, cap, pad, key_bits);
}

// One workgroup per image: the entries (i, j) of any list tensor by destination row, for the lists that are not made
// of whole clusters (`only_if`, may be null: a device flag; nothing happens when it points to zero).
__global__ __launch_bounds__(1024) void row_sort_kernel(const int64_t* __restrict__ idx, const int32_t* __restrict__ only_if,
                                                        int32_t* __restrict__ entries, int32_t* __restrict__ starts,
                                                        int32_t* __restrict__ ends, int E, int K, int key_bits) {
    if (only_if != nullptr && *only_if == 0) return;
    sort_image<true>(idx, entries, starts, ends, E, 1, K, E, 0, key_bits);
}

}  // namespace

namespace {
inline size_t keys_workgroups(int64_t runs) {
    const int64_t per = (int64_t)kKeysBlock * kKeysPerThread;
    return (size_t)((4 * runs + per - 1) / per);
}
}  // namespace

bool cluster_pairs_supported(int B, int rows, int M, int D) {
    if (B <= 0 || rows <= 0 || M <= 0 || M % 8 != 0 || M > kPairMaxSlots || D < 8) return false;
    const int64_t R = M / 8, K = (D + 7) / 8;
    const int64_t E = (int64_t)rows * R;
    if (rows >= (1 << (30 - kPairRunBits)) || 2 * E * B >= ((int64_t)1 << 31) || K * B >= ((int64_t)1 << 30)) return false;
    return (2 * K + 16) * 4 + 64 <= kSortLdsBytes;   // at least one wave's histogram fits
}

ClusterPairsLayout cluster_pairs_layout(int B, int rows, int M, int D) {
    ClusterPairsLayout l;
    const size_t R = M / 8, K = (D + 7) / 8, E = (size_t)rows * R;
    const size_t cap = (D % 8) ? 2 * E : E;
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    l.flag = 0;
    l.wg_bad = 256;
    l.keys = l.wg_bad + up(keys_workgroups((int64_t)B * (int64_t)E) * 4);
    l.pairs = l.keys + up((size_t)B * E * 4);
    l.starts = l.pairs + up((size_t)B * cap * 4);
    l.ends = l.starts + up((size_t)B * K * 4);
    l.bytes = l.ends + up((size_t)B * K * 4);
    return l;
}

int launch_cluster_pairs(const int64_t* idx, int32_t* keys, int32_t* wg_bad, int32_t* not_whole, int32_t* pairs,
                         int32_t* starts, int32_t* ends, int B, int rows, int M, int D, hipStream_t stream,
                         const int32_t* numbers) {
    const int R = M / 8, K = (D + 7) / 8;
    const int64_t E = (int64_t)rows * R;
    const int64_t runs = (int64_t)B * E;
    const int cap = (int)((D % 8) ? 2 * E : E);
    const int n_wg = (int)keys_workgroups(runs);   // (sized for the lists: four threads per run; the numbers use fewer)
    if (numbers != nullptr) {
        hipLaunchKernelGGL(cluster_number_keys_kernel, dim3((unsigned)n_wg), dim3(kKeysBlock), 0, stream, numbers, keys,
                           wg_bad, K, runs);
    } else {
        hipLaunchKernelGGL(cluster_keys_kernel, dim3((unsigned)n_wg), dim3(kKeysBlock), 0, stream, idx, keys, wg_bad, D, runs);
    }
    int waves = (kSortLdsBytes / 4 - 16) / K - 1;    // (waves + 1) * K + waves ints of LDS
    waves = waves > 16 ? 16 : waves;
    const int64_t steps = (E + 63) / 64;
    if (waves > steps) waves = (int)steps;
    if (waves < 1) waves = 1;
    const size_t lds = ((size_t)(waves + 1) * K + 16) * 4;
    int key_bits = 0;
    while ((1 << key_bits) < K) ++key_bits;
    hipLaunchKernelGGL(cluster_sort_kernel, dim3(B), dim3(64 * waves), lds, stream, keys, wg_bad, n_wg, not_whole, pairs,
                       starts, ends, (int)E, R, K, cap, (D % 8) ? 1 : 0, key_bits);
    return launch_status();
}

// ---- entries of any list tensor by destination row ---------------------------------------------------------------

namespace {
constexpr int kRowSortLdsBytes = 150 * 1024;   // of the 160 KB of a compute unit
inline int row_sort_waves(int K, int64_t E) {
    int waves = (kRowSortLdsBytes / 4 - 16) / K - 1;
    waves = waves > 16 ? 16 : waves;
    const int64_t steps = (E + 63) / 64;
    if (waves > steps) waves = (int)steps;
    return waves;
}
}  // namespace

bool row_entries_supported(int B, int rows, int M, int D) {
    if (B <= 0 || rows <= 0 || M <= 0 || D <= 0) return false;
    const int64_t E = (int64_t)rows * M;
    if (E >= ((int64_t)1 << 30) || E * B >= ((int64_t)1 << 31) || (int64_t)B * D >= ((int64_t)1 << 30)) return false;
    return row_sort_waves(D, E) >= 1;
}

RowEntriesLayout row_entries_layout(int B, int rows, int M, int D) {
    RowEntriesLayout l;
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    l.entries = 0;
    l.starts = up((size_t)B * rows * M * 4);
    l.ends = l.starts + up((size_t)B * D * 4);
    l.bytes = l.ends + up((size_t)B * D * 4);
    return l;
}

int launch_row_entries(const int64_t* idx, const int32_t* only_if, int32_t* entries, int32_t* starts, int32_t* ends, int B,
                       int rows, int M, int D, hipStream_t stream) {
    const int64_t E = (int64_t)rows * M;
    const int waves = row_sort_waves(D, E);
    const size_t lds = ((size_t)(waves + 1) * D + 16) * 4;
    int key_bits = 0;
    while ((1 << key_bits) < D) ++key_bits;
    if (lds > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(row_sort_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess) {
            (void)hipGetLastError();
            return CLUSTEN_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(row_sort_kernel, dim3(B), dim3(64 * waves), lds, stream, idx, only_if, entries, starts, ends, (int)E, D,
                       key_bits);
    return launch_status();
}

}  // namespace clusten
