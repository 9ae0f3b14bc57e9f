// Shared by the one-kernel attention of 16-bit data (cluster_attention.hip) and of fp32 data
// (cluster_attention_f32.hip): the shape they serve, the per-tile plan and the reductions over a token's 8 lanes.
#pragma once

#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace ca {

constexpr int kC = 32;            // head dim
constexpr int kR = 6;             // clusters per token
constexpr int kM = 8 * kR;        // neighbours per token

// A tile's plan: what the kernel works out from the index tensors before its first head — the distinct clusters of
// the tile, and per lane the bias-table rows (sign bit: masked slot), the distinct-cluster number of each run of its
// token and the runs that repeat an earlier one.  The lists of a stage serve all its layers, so the plan is built once
// per stage (cluster_attention_plan_kernel) and read back by every layer in two 16-byte loads per lane:
//   [0, 16)            U, the number of distinct clusters
//   [16, 16 + 192)     their cluster numbers
//   [256, 256 + 2048)  per lane: pe[6] (24 bytes), us[6] (6 bytes), repeats (1 byte), 1 byte unused
constexpr int kPlanLane = 256;
constexpr int kPlanBytes = kPlanLane + kWave * 32;

// Reductions over the 8 lanes of a token (lanes 8t .. 8t+7) with data-parallel-primitive moves: neighbours in a
// quad, the other pair of the quad, then the mirrored lane of the other quad.  Every lane ends with the same value.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float oct_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    return fmaxf(v, dpp_move<0x141>(v));  // row_half_mirror
}
__device__ __forceinline__ float oct_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    return v + dpp_move<0x141>(v);
}

// What a tile works out from the index tensors: `tok` = row of the lane's token (lane / 8) in them, `list_b` their
// batch element.  Lane (t, i) = member i of the runs of token t.
__device__ __forceinline__ void tile_setup(const int32_t* __restrict__ cluster_idx, const int64_t* __restrict__ pe_idx,
                                           const int64_t* __restrict__ mask, int64_t list_b, int N, int i0, int nt,
                                           int64_t tok, int (&pe)[kR], int (&us)[kR], int& repeats, int& U, int* ulist) {
    const int lane = threadIdx.x;
    const int t = lane >> 3, i = lane & 7;
    // cluster numbers: lane rho < 48 owns run rho = token * 6 + run of the tile
    const int rho = min(lane, kTileTokens * kR - 1);
    const int cid = cluster_idx[(list_b * N + i0 + min(rho / kR, nt - 1)) * kR + rho % kR];
    {
        int64_t wide[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) wide[r] = pe_idx[tok * kM + 8 * r + i];
#pragma unroll
        for (int r = 0; r < kR; ++r) pe[r] = (int)wide[r] & 0x7fffffff;
        if (mask) {
#pragma unroll
            for (int r = 0; r < kR; ++r) wide[r] = mask[tok * kM + 8 * r + i];
#pragma unroll
            for (int r = 0; r < kR; ++r) pe[r] |= wide[r] == 0 ? (int)0x80000000 : 0;
        }
    }
    // number the distinct cluster numbers in order of first appearance
    uint64_t remaining = (1ull << (kTileTokens * kR)) - 1;
    int uslot = 0;
    bool first = false;
    U = 0;
    while (remaining != 0) {
        const int s = __builtin_ctzll(remaining);
        const int cs = __builtin_amdgcn_readlane(cid, s);
        const bool hit = cid == cs;
        const uint64_t match = __ballot(hit) & remaining;
        if (hit) uslot = U;
        first = first || lane == s;
        remaining &= ~match;
        ++U;
    }
    if (first) ulist[uslot] = cid;
#pragma unroll
    for (int r = 0; r < kR; ++r) us[r] = __shfl(uslot, t * kR + r);
    // does a token of the tile list a cluster twice?  Bit r: run r repeats an earlier run of the token; its
    // probability is then added to that run's before the probabilities are laid out by distinct cluster.
    repeats = 0;
#pragma unroll
    for (int r = 1; r < kR; ++r) {
#pragma unroll
        for (int r2 = 0; r2 < r; ++r2) repeats |= us[r] == us[r2] ? 1 << r : 0;
    }
}

}  // namespace ca
}  // namespace clusten
