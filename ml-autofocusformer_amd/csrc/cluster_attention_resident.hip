// cluster_attention for short sequences: the one-kernel local attention of cluster_attention.hip (same inputs, same
// plan, same arithmetic in the same order, same results) with the K and V rows of a whole (image, head) resident in LDS.
//
// The kernel of cluster_attention.hip gathers, per tile of 8 tokens and head, the rows of the tile's 7-12 distinct
// clusters from the L2: 12 KB per tile and head, 1.3 GB a launch at 196 tokens x 8 heads x 128 images, and that launch
// takes what 1.3 GB of L2 hits take on this device (52 us at ~25 TB/s).  A sequence of at most 256 tokens has 16 KB of K
// rows and 16 KB of V rows per head: here a workgroup of several waves loads them once (25 KB at 196 tokens: what the
// old kernel gathered for two tiles), and its waves take the sequence's tiles in turn, reading their matrix operands
// from those rows in place - row 8 c + m of the sequence is row 8 c + m of the LDS copy, so a tile's distinct clusters
// need no staging at all, only their numbers (models/aff_transformer.py:120-155; the 196-token stage of the 224 x 224
// models holds 18 of their 25 attention layers).
//
// Per tile a wave does what a wave of cluster_attention.hip does per head: plan (or the tile's own numbering), scores
// of the tile's distinct clusters on six 16x16x32 matrix instructions a pass, each token's slots picked from the score
// matrix in LDS, softmax across the 8 lanes of a token, probabilities re-indexed by distinct cluster, weighted sum of
// the V rows through `ds_read_b64_tr_b16`, one output chunk.  16-bit data, head dim 32, clusters of 8 (M = 48).
#include <cstdlib>

#include "cluster_attention_plan.hpp"

namespace clusten {
namespace {

using namespace ca;

constexpr int kRB = kC * 2;                // bytes per row
constexpr int kPassRuns = 12;              // distinct clusters per pass
constexpr int kPassRows = 8 * kPassRuns;
constexpr int kBlocks = kPassRows / 16;    // 16-row blocks of the score product
constexpr int kSteps = kPassRows / 32;     // 32-row steps of the value product
constexpr int kSRow = kPassRows + 4;       // floats per token row of the score matrix
constexpr int kPRow = kPassRows + 8;       // 16-bit elements per token row of the re-indexed probabilities

constexpr int kResWaves = 8;               // waves of a workgroup: two per SIMD
constexpr int kResMaxRows = 256;           // tokens of a sequence this kernel takes

// LDS: the sequence's K rows, its V rows (whole 16-row accesses each), then one private area per wave.
constexpr int Q_OFF = 0;                                   // q rows of two tiles (slot = turn % 2): LDS-direct loads
constexpr int Q_SLOT = kTileTokens * kRB;
constexpr int S_OFF = Q_OFF + 2 * Q_SLOT;                  // scores; later the probabilities of a pass
constexpr int S_BYTES = kTileTokens * kSRow * 4;
constexpr int P_BYTES = kTileTokens * kPRow * 2;
constexpr int O_OFF = S_OFF + S_BYTES;                     // output chunk
constexpr int UL_OFF = O_OFF + kTileTokens * kRB;          // cluster number of each distinct cluster
constexpr int PB_OFF = UL_OFF + kTileTokens * kNnc * 4;    // blank-token probability per token
constexpr int W_BYTES = (PB_OFF + kTileTokens * 4 + 1023) / 1024 * 1024;
static_assert(P_BYTES <= S_BYTES && P_BYTES > 1024 && P_BYTES <= 2048, "the probabilities fit the score area");
// rows of the sequence padded to whole 16-row accesses (the pad rows hold copies of row 0, as the pad slots of a short
// last cluster name row 0), then one more access of copies of row 0: the rows of a cluster number outside the sequence
inline int resident_rows_bytes(int N) { return ((N + 15) / 16 * 16 + 16) * kRB; }
inline int resident_lds_bytes(int N) { return 2 * resident_rows_bytes(N) + kResWaves * W_BYTES; }

template <typename T>
__global__ __launch_bounds__(kResWaves* kWave) void cluster_attention_resident_kernel(
    const T* __restrict__ q, clusten_strides qs, const T* __restrict__ k, clusten_strides ks, const T* __restrict__ v,
    clusten_strides vs, const int32_t* __restrict__ cluster_idx, const T* __restrict__ table,
    const int64_t* __restrict__ pe_idx, const int64_t* __restrict__ mask, const float* __restrict__ blank_k,
    const float* __restrict__ blank_v, T* __restrict__ out, clusten_strides os, int H_all, int N, float scale,
    int tiles_per_batch, int total_units, int lists_shared, const char* __restrict__ plan, float* __restrict__ lse) {
    typedef short S4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) S4* LdsS4;

    extern __shared__ __attribute__((aligned(1024))) char stage[];
    const int KF_BASE = 0;
    const int n_pad = (N + 15) / 16 * 16;
    const int VF_BASE = (n_pad + 16) * kRB;
    const int W_BASE = 2 * VF_BASE;
    const int clusters = (N + 7) / 8;           // clusters of the sequence; number `clusters` and beyond: rows of row 0
    const int zero_cluster_bytes = n_pad * kRB;

    // unit -> (image, head): the heads of an image are neighbours in the grid (they read the same plan and lists)
    const int unit = xcd_tile(blockIdx.x, total_units);
    if (unit < 0) return;
    const int b = unit / H_all;
    const int h = unit - b * H_all;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15;     // matrix side: row of A / column of B
    const int kq = lane >> 4;      // matrix side: k group
    const int g_sub = lane >> 2;   // load side: row of a 16-row access
    const int g_pos = lane & 3;    //            16-byte piece of the row
    const int t = lane >> 3;       // softmax side: token of the tile
    const int i = lane & 7;        //               member of each cluster
    const int64_t list_b = lists_shared ? 0 : b;

    // ---- the head's K and V rows, all of them, once ---------------------------------------------------------------
    {
        const char* k_bh = reinterpret_cast<const char*>(k + (int64_t)b * ks.b + (int64_t)h * ks.h);
        const char* v_bh = reinterpret_cast<const char*>(v + (int64_t)b * vs.b + (int64_t)h * vs.h);
        for (int a = wave; a * 16 < n_pad + 16; a += kResWaves) {
            const int r = a * 16 + g_sub;
            const uint32_t row = (uint32_t)(r < N ? r : 0);
            CLUSTEN_LDS_DMA16(k_bh + lane_offset(row * (uint32_t)ks.n * 2 + (uint32_t)g_pos * 16), stage + KF_BASE + a * 1024);
            CLUSTEN_LDS_DMA16(v_bh + lane_offset(row * (uint32_t)vs.n * 2 + (uint32_t)g_pos * 16), stage + VF_BASE + a * 1024);
        }
    }
    char* mine = stage + W_BASE + wave * W_BYTES;
    int* ulist = reinterpret_cast<int*>(mine + UL_OFF);
    const char* q_bh = reinterpret_cast<const char*>(q + (int64_t)b * qs.b + (int64_t)h * qs.h);
    auto fetch_q = [&](int tile, int slot) {
        if (lane < 32) {
            const int i0 = tile * kTileTokens;
            const uint32_t row = (uint32_t)min(i0 + g_sub, N - 1);
            CLUSTEN_LDS_DMA16(q_bh + lane_offset(row * (uint32_t)qs.n * 2 + (uint32_t)g_pos * 16), mine + Q_OFF + slot * Q_SLOT);
        }
    };
    // byte offset of a cluster's 8 rows in the LDS copies (the copies of row 0 for a number outside the sequence)
    auto cluster_bytes = [&](int c) -> int {
        return (unsigned)c < (unsigned)clusters ? c * (8 * kRB) : zero_cluster_bytes;
    };
    // a tile's plan as it is loaded: two 16-byte pieces per lane, the number of distinct clusters, one cluster number
    struct PlanRegs {
        Piece lo, hi;
        int U, cluster;
    };
    auto load_plan = [&](int tile) -> PlanRegs {
        const char* pl = plan + (list_b * tiles_per_batch + tile) * (int64_t)kPlanBytes;
        PlanRegs r;
        r.lo = *reinterpret_cast<const Piece*>(pl + kPlanLane + lane * 32);
        r.hi = *reinterpret_cast<const Piece*>(pl + kPlanLane + lane * 32 + 16);
        r.U = *reinterpret_cast<const int*>(pl);
        r.cluster = *reinterpret_cast<const int*>(pl + 16 + min(lane, kTileTokens * kNnc - 1) * 4);
        return r;
    };
    // the wave's first tile: q rows and plan requested along with the K and V rows
    PlanRegs ahead = PlanRegs{Piece{0u, 0u, 0u, 0u}, Piece{0u, 0u, 0u, 0u}, 0, 0};
    if (wave < tiles_per_batch) {
        fetch_q(wave, 0);
        if (plan != nullptr) ahead = load_plan(wave);
    }
    // per-head constants
    const float4 bk = *reinterpret_cast<const float4*>(blank_k + h * kC + 4 * i);
    const float bv[2] = {blank_v[h * kC + r16], blank_v[h * kC + 16 + r16]};
    __syncthreads();   // (waits for every load above: the rows are in LDS for all waves)

    int turn = 0;
    for (int tile = wave; tile < tiles_per_batch; tile += kResWaves, ++turn) {
        const int i0 = tile * kTileTokens;
        const int nt = min(kTileTokens, N - i0);
        const int64_t tok = list_b * N + i0 + min(t, nt - 1);
        const char* q_lds = mine + Q_OFF + (turn & 1) * Q_SLOT;
        const bool more = tile + kResWaves < tiles_per_batch;

        int pe[kR];      // per-slot inputs: row of the bias table; the sign bit marks a masked slot
        int usc[kNnc];   // distinct-cluster number of each of this lane's token's clusters
        int repeats = 0; // bit c: cluster c repeats an earlier one of the token
        int U = 0;       // distinct clusters of the tile
        lds_sync();      // the tile before has read its cluster offsets
        if (plan != nullptr) {
            const PlanRegs now = ahead;
            U = now.U;
            // `ulist` holds where each distinct cluster's rows lie in the LDS copies
            if (lane < kTileTokens * kNnc) ulist[lane] = cluster_bytes(now.cluster);
            pe[0] = (int)now.lo[0]; pe[1] = (int)now.lo[1]; pe[2] = (int)now.lo[2]; pe[3] = (int)now.lo[3];
            pe[4] = (int)now.hi[0]; pe[5] = (int)now.hi[1];
            usc[0] = now.hi[2] & 0xff; usc[1] = (now.hi[2] >> 8) & 0xff; usc[2] = (now.hi[2] >> 16) & 0xff;
            usc[3] = now.hi[2] >> 24;
            usc[4] = now.hi[3] & 0xff; usc[5] = (now.hi[3] >> 8) & 0xff;
            repeats = (now.hi[3] >> 16) & 0xff;
        } else {
            tile_setup<8>(cluster_idx, pe_idx, mask, list_b, N, i0, nt, tok, pe, usc, repeats, U, ulist);
            lds_sync();
            if (lane < kTileTokens * kNnc) ulist[lane] = cluster_bytes(ulist[lane]);   // cluster numbers -> offsets
        }
        const bool twice = __any(repeats) != 0;
        // the bias of the lane's slots, then the next tile's plan and q rows: requested before the wait for this tile's
        float bias[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t cell = lane_offset(((uint32_t)(pe[r] & 0x7fffffff) * (uint32_t)H_all + (uint32_t)h) * 2);
            bias[r] = to_acc(*reinterpret_cast<const T*>(reinterpret_cast<const char*>(table) + cell)) +
                      (pe[r] < 0 ? -100.f : 0.f);
        }
        if (more) {
            if (plan != nullptr) ahead = load_plan(tile + kResWaves);
            fetch_q(tile + kResWaves, (turn + 1) & 1);
            // this tile's q rows were requested a tile ago: before the loads above, which may stay in flight
            lds_sync_vm<5>();
        } else {
            lds_sync_vm<0>();
        }

        const int passes = (U + kPassRuns - 1) / kPassRuns;
        const int total_rows = 8 * U;

        // ---- scores ----------------------------------------------------------------------------------------------
        float logit[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) logit[r] = 0.f;
        const Piece qraw = *reinterpret_cast<const Piece*>(q_lds + (r16 & 7) * kRB + kq * 16);
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
            // the lane's row of each 16-row block: member r16 % 8 of distinct cluster 2 blk + r16 / 8 of the pass
            // (clusters past the last one repeat it, so that every row of a block holds data)
            int kaddr[kBlocks];
#pragma unroll
            for (int blk = 0; blk < kBlocks; ++blk) {
                kaddr[blk] = ulist[min(pass * kPassRuns + 2 * blk + (r16 >> 3), U - 1)] + (r16 & 7) * kRB + kq * 16;
            }
            if (pass > 0) lds_sync();   // the scores of the pass before have been picked
#pragma unroll
            for (int blk = 0; blk < kBlocks; ++blk) {
                if (blk * 16 < rows_here) {
                    const Piece kraw = *reinterpret_cast<const Piece*>(stage + KF_BASE + kaddr[blk]);
                    const F32x4 d = tile_mfma<T>(kraw, qraw, F32x4{0.f, 0.f, 0.f, 0.f});
                    // lane (r16, kq): pass rows 16*blk + 4*kq .. +3 of token r16
                    if (r16 < kTileTokens) {
                        *reinterpret_cast<F32x4*>(mine + S_OFF + (r16 * kSRow + 16 * blk + 4 * kq) * 4) = d;
                    }
                }
            }
            lds_sync();
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const unsigned u = (unsigned)(usc[r] - pass * kPassRuns);
                const float sc = *reinterpret_cast<const float*>(
                    mine + S_OFF + (t * kSRow + (int)min(u, (unsigned)kPassRuns - 1) * 8 + i) * 4);
                logit[r] = u < (unsigned)kPassRuns ? sc : logit[r];
            }
        }

        // ---- softmax over the neighbours and the blank token ---------------------------------------------------
        float x[kR];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            x[r] = logit[r] * scale + bias[r];
            mx = fmaxf(mx, x[r]);
        }
        float part = 0.f;
        {
            const T* qrow = reinterpret_cast<const T*>(q_lds + t * kRB) + 4 * i;
            part = to_acc(qrow[0]) * bk.x + to_acc(qrow[1]) * bk.y + to_acc(qrow[2]) * bk.z + to_acc(qrow[3]) * bk.w;
        }
        const float bl = oct_sum(part) * scale;
        mx = fmaxf(oct_max(mx), bl);
        float p[kR];
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            p[r] = __expf(x[r] - mx);
            sum += p[r];
        }
        const float eb = __expf(bl - mx);
        const float total = oct_sum(sum) + eb;
        const float inv = 1.f / total;
        if (lse != nullptr && i == 0 && t < nt) lse[((int64_t)b * H_all + h) * N + i0 + t] = mx + __logf(total);
#pragma unroll
        for (int r = 0; r < kR; ++r) p[r] *= inv;
        if (i == 0) *reinterpret_cast<float*>(mine + PB_OFF + t * 4) = eb * inv;
        if (twice) {
#pragma unroll
            for (int c = kNnc - 1; c >= 1; --c) {
#pragma unroll
                for (int c2 = 0; c2 < c; ++c2) {
                    // the first listing of a cluster collects the probabilities of its repeats
                    const bool firstmatch = usc[c] == usc[c2] && ((repeats >> c) & 1) && !((repeats >> c2) & 1);
                    p[c2] += firstmatch ? p[c] : 0.f;
                }
            }
        }

        // ---- weighted sum of the V rows --------------------------------------------------------------------------
        F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
            // the lane's rows of each 32-row step: members r16 / 4 and r16 / 4 + 4 of distinct cluster 4 s + kq
            int vaddr[kSteps];
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                vaddr[s] = ulist[min(pass * kPassRuns + 4 * s + kq, U - 1)] + (r16 >> 2) * kRB + (r16 & 3) * 8;
            }
            lds_sync();  // the scores have been picked (the probabilities of the pass before have been read)
            // probabilities of this pass, re-indexed by distinct cluster: zero, then each lane puts in its own
            *reinterpret_cast<Piece*>(mine + S_OFF + lane * 16) = Piece{0u, 0u, 0u, 0u};
            if (lane < (P_BYTES - 1024) / 16) {
                *reinterpret_cast<Piece*>(mine + S_OFF + 1024 + lane * 16) = Piece{0u, 0u, 0u, 0u};
            }
            lds_sync();
            T* prow = reinterpret_cast<T*>(mine + S_OFF) + t * kPRow + i;
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                // clusters of other passes, and repeats (already added to their first listing), go to the spare cells
                const unsigned u = ((repeats >> r) & 1) ? ~0u : (unsigned)(usc[r] - pass * kPassRuns);
                prow[min(u, (unsigned)kPassRuns) * 8] = from_acc<T>(p[r]);
            }
            lds_sync();
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                if (s * 32 < rows_here) {
                    const Piece a = *reinterpret_cast<const Piece*>(mine + S_OFF + ((r16 & 7) * kPRow + 32 * s + 8 * kq) * 2);
                    const char* lo_row = stage + VF_BASE + vaddr[s];
                    const char* hi_row = lo_row + 4 * kRB;
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        // rows 0-3 and 4-7 of the lane's cluster, transposed to channel 16*cb + r16
                        const S4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(lo_row + cb * 32));
                        const S4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(hi_row + cb * 32));
                        const U32x2 lo = __builtin_bit_cast(U32x2, b0), hi = __builtin_bit_cast(U32x2, b1);
                        acc[cb] = tile_mfma<T>(a, Piece{lo[0], lo[1], hi[0], hi[1]}, acc[cb]);
                    }
                }
            }
        }

        // ---- blank token, output chunk (8 tokens x 32 channels, row-major) -----------------------------------------------
        if (kq < 2) {
            const F32x4 pb = *reinterpret_cast<const F32x4*>(mine + PB_OFF + 16 * kq);
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    reinterpret_cast<T*>(mine + O_OFF)[(4 * kq + e) * kC + 16 * cb + r16] =
                        from_acc<T>(acc[cb][e] + pb[e] * bv[cb]);
                }
            }
        }
        lds_sync();
        if (lane < 32 && g_sub < nt) {
            const Piece o = *reinterpret_cast<const Piece*>(mine + O_OFF + lane * 16);
            char* dst = reinterpret_cast<char*>(out + (int64_t)b * os.b + (int64_t)h * os.h + (int64_t)(i0 + g_sub) * os.n);
            *reinterpret_cast<Piece*>(dst + g_pos * 16) = o;   // plain: the output projection reads it next
        }
    }
}

template <typename T>
int launch_typed(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v, clusten_strides vs,
                 const int32_t* cluster_idx, const void* table, const int64_t* pe_idx, const int64_t* mask,
                 const float* blank_k, const float* blank_v, void* out, clusten_strides os, float scale, int lists_shared,
                 const void* plan, float* lse, const clusten_attn_shape& s, hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * s.H;
    // more LDS than a workgroup gets without asking (two workgroups share a CU's 160 KB)
    const int lds = resident_lds_bytes(s.N);
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(cluster_attention_resident_kernel<T>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, resident_lds_bytes(kResMaxRows)) != hipSuccess) {
        (void)hipGetLastError();
        return CLUSTEN_ERR_LAUNCH;
    }
    hipLaunchKernelGGL((cluster_attention_resident_kernel<T>), dim3(xcd_grid(total)), dim3(kResWaves * kWave), lds, stream,
                       static_cast<const T*>(q), qs, static_cast<const T*>(k), ks, static_cast<const T*>(v), vs,
                       cluster_idx, static_cast<const T*>(table), pe_idx, mask, blank_k, blank_v, static_cast<T*>(out), os,
                       s.H, s.N, scale, tiles_per_batch, total, lists_shared, static_cast<const char*>(plan), lse);
    return launch_status();
}

}  // namespace

// True when the resident kernel takes the shape: clusters of 8, a sequence that fits its LDS copy, and enough (image,
// head) pairs to fill the device (below that the kernel with one workgroup per tile has more waves to offer).
// CLUSTEN_ATTENTION_RESIDENT in the environment overrides the last two conditions: 0 = never, 1 = whenever the sequence
// fits (read once; for tests and measurements).
bool cluster_attention_resident_takes(const clusten_attn_shape& s, int dtype) {
    static const int forced = [] {
        const char* e = getenv("CLUSTEN_ATTENTION_RESIDENT");
        return e == nullptr ? -1 : atoi(e);
    }();
    const bool fits = (dtype == CLUSTEN_F16 || dtype == CLUSTEN_BF16) && s.M == kM && s.C == kC && s.N <= kResMaxRows;
    if (forced == 0 || !fits) return false;
    if (forced > 0) return true;
    return s.N >= 2 * kResWaves * kTileTokens && (int64_t)s.B * s.H >= 512;
}

int launch_cluster_attention_resident(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                      clusten_strides vs, const int32_t* cluster_idx, const void* table,
                                      const int64_t* pe_idx, const int64_t* mask, const float* blank_k,
                                      const float* blank_v, void* out, clusten_strides os, float scale, int lists_shared,
                                      const void* plan, float* lse, const clusten_attn_shape& s, int dtype,
                                      hipStream_t stream) {
    if (dtype == CLUSTEN_F16) {
        return launch_typed<f16_t>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os, scale,
                                   lists_shared, plan, lse, s, stream);
    }
    return launch_typed<bf16_t>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os, scale,
                                lists_shared, plan, lse, s, stream);
}

}  // namespace clusten
