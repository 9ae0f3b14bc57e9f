// Shared by the one-kernel attention of 16-bit data (cluster_attention.hip) and of fp32 data
// (cluster_attention_f32.hip): the shape they serve, the per-tile plan and the reductions over a token's 8 lanes.
#pragma once

#include "dpp.hpp"
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace ca {

constexpr int kC = 32;            // head dim
constexpr int kNnc = 6;           // clusters per token

// Shape of the lists for clusters of CS tokens (8 in the 224 x 224 models, 24 in the 384 x 384 ones): a token lists the
// CS members of its 6 nearest clusters, i.e. kR runs of 8 slots, run r = rows CS * cluster(r / kSub) + 8 * (r % kSub) ...
template <int CS>
struct Geo {
    static_assert(CS % 8 == 0 && CS >= 8 && CS <= 32, "clusters of whole runs of 8 tokens");
    static constexpr int kSub = CS / 8;          // runs of 8 per cluster
    static constexpr int kR = kNnc * kSub;       // runs of 8 per token
    static constexpr int kM = 8 * kR;            // neighbours per token
    // per lane of the plan: pe[kR] (4 bytes each), the distinct-cluster number of each of the token's 6 clusters
    // (1 byte each), repeats (1 byte), padded to whole 16-byte pieces
    static constexpr int kPlanLaneBytes = (4 * kR + 8 + 15) / 16 * 16;
    static constexpr int kPlanBytes = 256 + kWave * kPlanLaneBytes;
};
constexpr int kR = Geo<8>::kR;    // clusters of 8: runs = clusters per token
constexpr int kM = Geo<8>::kM;

// A tile's plan: what the kernel works out from the index tensors before its first head — the distinct clusters of
// the tile, and per lane the bias-table rows (sign bit: masked slot), the distinct-cluster number of each cluster of
// its token and the clusters that repeat an earlier one.  The lists of a stage serve all its layers, so the plan is
// built once per stage (cluster_attention_plan_kernel) and read back by every layer in a few 16-byte loads per lane:
//   [0, 16)            U, the number of distinct clusters
//   [16, 16 + 192)     their cluster numbers
//   [256, ...)         per lane (Geo<CS>::kPlanLaneBytes): pe[kR], us[6] (6 bytes), repeats (1 byte), padding
// For clusters of 8 that is 32 bytes per lane: pe[6] (24 bytes), us[6], repeats, 1 byte unused.
constexpr int kPlanLane = 256;
constexpr int kPlanBytes = Geo<8>::kPlanBytes;

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
// batch element.  Lane (t, i) = member i of the runs of 8 of token t; us[k] = distinct-cluster number of the token's
// cluster k, ulist[u] = cluster number of distinct cluster u.
template <int CS = 8>
__device__ __forceinline__ void tile_setup(const int32_t* __restrict__ cluster_idx, const int64_t* __restrict__ pe_idx,
                                           const int64_t* __restrict__ mask, int64_t list_b, int N, int i0, int nt,
                                           int64_t tok, int (&pe)[Geo<CS>::kR], int (&us)[kNnc], int& repeats, int& U,
                                           int* ulist) {
    constexpr int kRuns = Geo<CS>::kR, kSlots = Geo<CS>::kM;
    const int lane = threadIdx.x & 63;   // (the callers are one wave per tile; some have several waves a workgroup)
    const int t = lane >> 3, i = lane & 7;
    // cluster numbers: lane rho < 48 owns entry rho = token * 6 + cluster of the tile
    const int rho = min(lane, kTileTokens * kNnc - 1);
    const int cid = cluster_idx[(list_b * N + i0 + min(rho / kNnc, nt - 1)) * kNnc + rho % kNnc];
    {
        constexpr int kBatch = 6;   // index loads in flight at a time
#pragma unroll
        for (int r0 = 0; r0 < kRuns; r0 += kBatch) {
            int64_t wide[kBatch];
#pragma unroll
            for (int r = 0; r < kBatch; ++r) wide[r] = pe_idx[tok * kSlots + 8 * (r0 + r) + i];
#pragma unroll
            for (int r = 0; r < kBatch; ++r) pe[r0 + r] = (int)wide[r] & 0x7fffffff;
            if (mask) {
#pragma unroll
                for (int r = 0; r < kBatch; ++r) wide[r] = mask[tok * kSlots + 8 * (r0 + r) + i];
#pragma unroll
                for (int r = 0; r < kBatch; ++r) pe[r0 + r] |= wide[r] == 0 ? (int)0x80000000 : 0;
            }
        }
    }
    // number the distinct cluster numbers in order of first appearance
    uint64_t remaining = (1ull << (kTileTokens * kNnc)) - 1;
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
    for (int r = 0; r < kNnc; ++r) us[r] = __shfl(uslot, t * kNnc + r);
    // does a token of the tile list a cluster twice?  Bit r: cluster r repeats an earlier cluster of the token; its
    // probabilities are then added to that one's before the probabilities are laid out by distinct cluster.
    repeats = 0;
#pragma unroll
    for (int r = 1; r < kNnc; ++r) {
#pragma unroll
        for (int r2 = 0; r2 < r; ++r2) repeats |= us[r] == us[r2] ? 1 << r : 0;
    }
}

}  // namespace ca
}  // namespace clusten
