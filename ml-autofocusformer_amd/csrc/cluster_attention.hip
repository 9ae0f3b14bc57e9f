// cluster_attention: local attention of a cluster-ordered token sequence in one kernel (inference).
//
//   logit[b,h,i,j] = scale * sum_c q[b,h,i,c] * k[b,h,row(i,j),c] + table[pe_idx[b,i,j], h] - 100 * (1 - mask[b,i,j])
//   blank[b,h,i]   = scale * sum_c q[b,h,i,c] * blank_k[h,c]
//   p[b,h,i,:], p_blank[b,h,i] = softmax over the M neighbours and the blank token
//   out[b,h,i,c]   = sum_j p[b,h,i,j] * v[b,h,row(i,j),c] + p_blank[b,h,i] * blank_v[h,c]
//   row(i,j)       = CS * cluster_idx[b,i,j/CS] + j%CS   (row 0 where that is not in [0,N)); CS = cluster size
//
// This is CLUSTENQKFunction, the tensor expressions between the two operators and CLUSTENAVFunction of the
// reference model (models/aff_transformer.py:120-155; kernels clusten/src/clustenqk_cuda_kernel.cu:18-49 and
// clusten/src/clustenav_cuda_kernel.cu:18-49) with the (B,H,N,M) logits and probabilities never leaving the
// chip.  16-bit data (fp16 / bf16), head dim 32, six clusters per token: M = 48 for clusters of 8 (every attention
// layer of the shipped 224 x 224 models under mixed precision), M = 144 for clusters of 24 (the 384 x 384 models,
// configs/aff_base_22kto1k_384.yaml:10-11), which the kernel treats as three runs of 8 rows each: a tile of 8 tokens
// then names some 8 distinct clusters = 24 runs and a head takes two or three passes.
//
// One wave owns 8 consecutive tokens (one cluster) and walks the heads.  The tile's 48 cluster numbers are
// numbered by distinct value (`U` of them; 7-12 in the shipped models: neighbouring tokens choose among the same
// clusters); per head the rows of up to 12 distinct clusters at a time (a pass: 96 rows) travel to LDS by
// LDS-direct loads, and
//   QK  S[row][token] = K_pass (96 x 32) * q^T (32 x 8): six 16x16x32 matrix instructions; each token picks its own
//       slots from the score matrix in LDS;
//   softmax: lane (t = lane / 8, i = lane % 8) holds slots 8*r + i, r < 6, of token t; maxima and sums go across the
//       8 lanes of a token;
//   AV  out (8 x 32) = P_pass (8 x 96) * V_pass (96 x 32): the probabilities are written to LDS re-indexed by
//       distinct cluster (zero where a token does not hold the cluster; a cluster held twice adds up), rounded to
//       the storage type; the V operand needs consecutive rows of one channel per lane, which
//       `ds_read_b64_tr_b16` delivers from the row-major rows.
// The first K and V rows of the next head are requested during the last AV pass of the current one, ahead of its
// output store, so that a head whose clusters fit one pass never waits for rows.  Tiles with more distinct
// clusters (up to 48: lists with nothing in common) take further passes.
//
// A token whose probabilities are zero for a cluster still multiplies that cluster's V rows by zero: non-finite
// values in rows a token does not list reach its output as NaN (the unfused operators share this on their
// union path).
#include "cluster_attention_plan.hpp"

namespace clusten {

int launch_cluster_attention_f32(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                 clusten_strides vs, const int32_t* cluster_idx, const void* table, const int64_t* pe_idx,
                                 const int64_t* mask, const float* blank_k, const float* blank_v, void* out,
                                 clusten_strides os, float scale, int lists_shared, const void* plan, float* lse,
                                 const clusten_attn_shape& s, hipStream_t stream);   // cluster_attention_f32.hip
// cluster_attention_resident.hip: short sequences, the K and V rows of an (image, head) resident in LDS
bool cluster_attention_resident_takes(const clusten_attn_shape& s, int dtype);
int launch_cluster_attention_resident(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                      clusten_strides vs, const int32_t* cluster_idx, const void* table,
                                      const int64_t* pe_idx, const int64_t* mask, const float* blank_k,
                                      const float* blank_v, void* out, clusten_strides os, float scale, int lists_shared,
                                      const void* plan, float* lse, const clusten_attn_shape& s, int dtype,
                                      hipStream_t stream);

namespace {

using namespace ca;

constexpr int kRB = kC * 2;       // bytes per row
constexpr int kPassRuns = 12;     // distinct clusters per pass
constexpr int kPassRows = 8 * kPassRuns;
constexpr int kBlocks = kPassRows / 16;   // 16-row blocks of the score product
constexpr int kSteps = kPassRows / 32;    // 32-row steps of the value product
constexpr int kAccesses = kPassRows / 16; // wave accesses (16 rows of 64 bytes) per pass
constexpr int kSRow = kPassRows + 4;   // floats per token row of the score matrix
constexpr int kPRow = kPassRows + 8;   // 16-bit elements per token row of the re-indexed probabilities; the last 8
                                       // are never read: cells for the writes of runs outside the pass

// LDS: two row areas and small tables.
//   [K_BASE, +6144)  K rows of a pass; once they are in registers the score matrix; during the AV passes the
//                    probabilities of a pass (the next head's K rows are requested only once those are in registers)
//   [V_BASE, +6144)  V rows of a pass
constexpr int K_BASE = 0;
constexpr int S_BASE = K_BASE;
constexpr int P_BASE = K_BASE;
constexpr int P_BYTES = kTileTokens * kPRow * 2;
constexpr int V_BASE = K_BASE + kPassRows * kRB;
constexpr int O_BASE = V_BASE + kPassRows * kRB;           // output chunk of a head
constexpr int Q_BASE = O_BASE + kTileTokens * kRB;         // q rows of two heads (slot h % 2)
constexpr int Q_SLOT = kTileTokens * kRB;
constexpr int UL_BASE = Q_BASE + 2 * Q_SLOT;               // cluster number of each distinct cluster
constexpr int PB_BASE = UL_BASE + kTileTokens * kNnc * 4;  // blank-token probability per token
constexpr int LDS_BYTES = PB_BASE + kTileTokens * 4;
static_assert(P_BYTES % 16 == 0 && P_BYTES <= kPassRows * kRB, "the probabilities fit the K area");
static_assert(kTileTokens * kSRow * 4 <= kPassRows * kRB, "the scores fit the K area");
static_assert(kPassRows % 32 == 0 && Q_BASE % 16 == 0, "whole 32-row steps");

// One wave per tile: the plan of every tile of the index tensors (B_lists batch elements).
template <int CS>
__global__ __launch_bounds__(kWave) void cluster_attention_plan_kernel(const int32_t* __restrict__ cluster_idx,
                                                                       const int64_t* __restrict__ pe_idx,
                                                                       const int64_t* __restrict__ mask,
                                                                       char* __restrict__ plan, int N, int tiles_per_batch,
                                                                       int total_tiles) {
    typedef Geo<CS> G;
    __shared__ int ulist[kTileTokens * kNnc];
    const int tile = blockIdx.x;
    if (tile >= total_tiles) return;
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTileTokens;
    const int nt = min(kTileTokens, N - i0);
    const int lane = threadIdx.x;
    const int64_t tok = (int64_t)b * N + i0 + min(lane >> 3, nt - 1);
    int pe[G::kR], us[kNnc], repeats, U;
    tile_setup<CS>(cluster_idx, pe_idx, mask, b, N, i0, nt, tok, pe, us, repeats, U, ulist);
    lds_sync();
    char* mine = plan + (int64_t)tile * G::kPlanBytes;
    if (lane == 0) *reinterpret_cast<int*>(mine) = U;
    if (lane < kTileTokens * kNnc) *reinterpret_cast<int*>(mine + 16 + lane * 4) = lane < U ? ulist[lane] : 0;
    // the lane's record: pe[kR], then the six distinct-cluster numbers and the repeat bits, one byte each
    uint32_t words[G::kPlanLaneBytes / 4];
#pragma unroll
    for (int w = 0; w < G::kPlanLaneBytes / 4; ++w) words[w] = 0u;
#pragma unroll
    for (int r = 0; r < G::kR; ++r) words[r] = (uint32_t)pe[r];
    words[G::kR] = (uint32_t)us[0] | ((uint32_t)us[1] << 8) | ((uint32_t)us[2] << 16) | ((uint32_t)us[3] << 24);
    words[G::kR + 1] = (uint32_t)us[4] | ((uint32_t)us[5] << 8) | ((uint32_t)repeats << 16);
#pragma unroll
    for (int q = 0; q < G::kPlanLaneBytes / 16; ++q) {
        *reinterpret_cast<Piece*>(mine + kPlanLane + lane * G::kPlanLaneBytes + q * 16) =
            Piece{words[4 * q], words[4 * q + 1], words[4 * q + 2], words[4 * q + 3]};
    }
}

template <typename T, int CS>
__global__ __launch_bounds__(kWave) void cluster_attention_kernel(
    const T* __restrict__ q, clusten_strides qs, const T* __restrict__ k, clusten_strides ks, const T* __restrict__ v,
    clusten_strides vs, const int32_t* __restrict__ cluster_idx, const T* __restrict__ table,
    const int64_t* __restrict__ pe_idx, const int64_t* __restrict__ mask, const float* __restrict__ blank_k,
    const float* __restrict__ blank_v, T* __restrict__ out, clusten_strides os, int H_all, int N, float scale,
    int tiles_per_batch, int total_tiles, int lists_shared, int head_groups, const char* __restrict__ plan,
    float* __restrict__ lse) {
    typedef short S4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) S4* LdsS4;
    typedef Geo<CS> G;
    constexpr int kRuns = G::kR;     // runs of 8 slots per token
    constexpr int kSub = G::kSub;    // runs per cluster

    __shared__ __attribute__((aligned(1024))) char stage[LDS_BYTES];

    // a workgroup serves the heads [h0, h0 + H) of its tile (see head_groups_for())
    const int unit = xcd_tile(blockIdx.x, total_tiles * head_groups);
    if (unit < 0) return;
    const int tile = unit / head_groups;
    const int heads_per_group = (H_all + head_groups - 1) / head_groups;
    const int h0 = (unit - tile * head_groups) * heads_per_group;
    const int H = min(heads_per_group, H_all - h0);
    if (H <= 0) return;
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTileTokens;
    const int nt = min(kTileTokens, N - i0);
    const int lane = threadIdx.x;
    const int r16 = lane & 15;     // matrix side: row of A / column of B
    const int kq = lane >> 4;      // matrix side: k group
    const int g_sub = lane >> 2;   // gather side: row of a 16-row access
    const int g_pos = lane & 3;    //              16-byte piece of the row
    const int t = lane >> 3;       // softmax side: token of the tile (tokens past a partial tile repeat its last one)
    const int i = lane & 7;        //               member of each cluster
    // the token's row in the index tensors: those of batch element 0 serve every image when the lists are shared
    // (the tokens of a regular grid have the same neighbourhoods in every image)
    const int64_t list_b = lists_shared ? 0 : b;
    const int64_t tok = list_b * N + i0 + min(t, nt - 1);

    // q rows of head h -> slot h % 2 (lanes 0..31: token lane / 4, piece lane % 4)
    const char* q_tile = reinterpret_cast<const char*>(q + (int64_t)b * qs.b + (int64_t)h0 * qs.h + (int64_t)i0 * qs.n);
    const uint32_t q_off = (uint32_t)min(g_sub, nt - 1) * (uint32_t)qs.n * 2 + (uint32_t)g_pos * 16;
    auto fetch_q = [&](int h) {
        if (lane < 32) {
            CLUSTEN_LDS_DMA16(q_tile + (int64_t)h * qs.h * 2 + lane_offset(q_off), stage + Q_BASE + (h & 1) * Q_SLOT);
        }
    };
    fetch_q(0);
    if (H > 1) fetch_q(1);

    int pe[kRuns];   // per-slot inputs the heads share: row of the bias table; the sign bit marks a masked slot
    int usc[kNnc];   // distinct-cluster number of each of this lane's token's clusters
    int repeats = 0; // bit k: cluster k repeats an earlier one of the token; its probabilities are added to that one's
    int U = 0;       // distinct clusters of the tile
    int* ulist = reinterpret_cast<int*>(stage + UL_BASE);
    if (plan != nullptr) {
        // the tile's plan, built once for all layers that use these lists
        const char* mine = plan + (list_b * tiles_per_batch + (tile - b * tiles_per_batch)) * (int64_t)G::kPlanBytes;
        uint32_t words[G::kPlanLaneBytes / 4];
#pragma unroll
        for (int q = 0; q < G::kPlanLaneBytes / 16; ++q) {
            const Piece w4 = *reinterpret_cast<const Piece*>(mine + kPlanLane + lane * G::kPlanLaneBytes + q * 16);
            words[4 * q] = w4[0]; words[4 * q + 1] = w4[1]; words[4 * q + 2] = w4[2]; words[4 * q + 3] = w4[3];
        }
        U = *reinterpret_cast<const int*>(mine);
        if (lane < kTileTokens * kNnc) ulist[lane] = *reinterpret_cast<const int*>(mine + 16 + lane * 4);
#pragma unroll
        for (int r = 0; r < kRuns; ++r) pe[r] = (int)words[r];
        const uint32_t w2 = words[kRuns], w3 = words[kRuns + 1];
        usc[0] = w2 & 0xff; usc[1] = (w2 >> 8) & 0xff; usc[2] = (w2 >> 16) & 0xff; usc[3] = w2 >> 24;
        usc[4] = w3 & 0xff; usc[5] = (w3 >> 8) & 0xff;
        repeats = (w3 >> 16) & 0xff;
    } else {
        tile_setup<CS>(cluster_idx, pe_idx, mask, list_b, N, i0, nt, tok, pe, usc, repeats, U, ulist);
    }
    const bool twice = __any(repeats) != 0;
    lds_sync();
    // in units of runs of 8 rows: distinct cluster u holds the units kSub * u .. kSub * u + kSub - 1
    int ub[kNnc];
#pragma unroll
    for (int c = 0; c < kNnc; ++c) ub[c] = usc[c] * kSub;
    auto unit_of = [&](auto ri) -> int {   // the unit of the token's run r (a compile-time number)
        constexpr int r = decltype(ri)::value;
        return ub[r / kSub] + r % kSub;
    };
    const int units = U * kSub;

    const int total_rows = 8 * units;
    const int passes = (units + kPassRuns - 1) / kPassRuns;
    const uint32_t k_pitch = (uint32_t)ks.n * 2, v_pitch = (uint32_t)vs.n * 2;
    const char* k_b = reinterpret_cast<const char*>(k + (int64_t)b * ks.b + (int64_t)h0 * ks.h);
    const char* v_b = reinterpret_cast<const char*>(v + (int64_t)b * vs.b + (int64_t)h0 * vs.h);

    // rows of the units 12*pass .. 12*pass+11, as this lane gathers them: access a moves row 16*a + g_sub of the
    // pass; units past the last one repeat it so that every row of a 32-row step holds data
    auto pass_rows = [&](int pass, uint32_t (&rr)[kAccesses]) {
#pragma unroll
        for (int a = 0; a < kAccesses; ++a) {
            const int urow = a * 16 + g_sub;
            const int unit = min(pass * kPassRuns + (urow >> 3), units - 1);
            const int row = ulist[unit / kSub] * CS + (unit % kSub) * 8 + (urow & 7);
            rr[a] = (unsigned)row < (unsigned)N ? (uint32_t)row : 0u;
        }
    };
    auto gather = [&](const char* rows_bh, uint32_t pitch, const uint32_t (&rr)[kAccesses], int rows_here, int lds_base) {
#pragma unroll
        for (int a = 0; a < kAccesses; ++a) {
            if ((a & ~1) * 16 < rows_here) {
                CLUSTEN_LDS_DMA16(rows_bh + lane_offset(rr[a] * pitch + (uint32_t)g_pos * 16), stage + lds_base + a * 1024);
            }
        }
    };
    // K and V rows of the same pass together, access by access: when k and v are the two halves of one projection output
    // (a model hands them over so) a K row and its V row share a 128-byte line, and the V access finds in the L1 what
    // the K access just asked for
    auto gather_both = [&](const char* k_bh, const char* v_bh, const uint32_t (&rr)[kAccesses], int rows_here) {
#pragma unroll
        for (int a = 0; a < kAccesses; ++a) {
            if ((a & ~1) * 16 < rows_here) {
                CLUSTEN_LDS_DMA16(k_bh + lane_offset(rr[a] * k_pitch + (uint32_t)g_pos * 16), stage + K_BASE + a * 1024);
                CLUSTEN_LDS_DMA16(v_bh + lane_offset(rr[a] * v_pitch + (uint32_t)g_pos * 16), stage + V_BASE + a * 1024);
            }
        }
    };
    uint32_t rr0[kAccesses];  // pass 0: used by every head
    pass_rows(0, rr0);
    const int rows0 = min(kPassRows, total_rows);
    gather_both(k_b, v_b, rr0, rows0);

    for (int h = 0; h < H; ++h) {
        const char* k_bh = k_b + (int64_t)h * ks.h * 2;
        const char* v_bh = v_b + (int64_t)h * vs.h * 2;
        const char* q_lds = stage + Q_BASE + (h & 1) * Q_SLOT;

        // The first K and V rows of this head were requested during the previous head (or above); the only
        // vector-memory operation issued after them is that head's output store, which may stay in flight.
        if (h == 0) {
            lds_sync_vm<0>();
        } else {
            lds_sync_vm<1>();
        }

        // small per-head operands: their latency passes under the score computation
        float bias[kRuns];
#pragma unroll
        for (int r = 0; r < kRuns; ++r) {
            const uint32_t cell = lane_offset(((uint32_t)(pe[r] & 0x7fffffff) * (uint32_t)H_all + (uint32_t)(h0 + h)) * 2);
            bias[r] = to_acc(*reinterpret_cast<const T*>(reinterpret_cast<const char*>(table) + cell)) +
                      (pe[r] < 0 ? -100.f : 0.f);
        }
        const float4 bk = *reinterpret_cast<const float4*>(blank_k + (h0 + h) * kC + 4 * i);
        const float bv[2] = {blank_v[(h0 + h) * kC + r16], blank_v[(h0 + h) * kC + 16 + r16]};

        // ---- scores -------------------------------------------------------------------------------------
        float logit[kRuns];
#pragma unroll
        for (int r = 0; r < kRuns; ++r) logit[r] = 0.f;
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
            if (pass > 0) lds_sync_vm<0>();  // the K rows of this pass are in LDS
            const Piece qraw = *reinterpret_cast<const Piece*>(q_lds + (r16 & 7) * kRB + kq * 16);
            Piece kraw[kBlocks];
#pragma unroll
            for (int blk = 0; blk < kBlocks; ++blk) {
                if (blk * 16 < rows_here) {
                    kraw[blk] = *reinterpret_cast<const Piece*>(stage + K_BASE + (blk * 16 + r16) * kRB + kq * 16);
                }
            }
            lds_sync();  // the K rows are in registers: their area takes the scores
#pragma unroll
            for (int blk = 0; blk < kBlocks; ++blk) {
                if (blk * 16 < rows_here) {
                    const F32x4 d = tile_mfma<T>(kraw[blk], qraw, F32x4{0.f, 0.f, 0.f, 0.f});
                    // lane (r16, kq): pass rows 16*blk + 4*kq .. +3 of token r16
                    if (r16 < kTileTokens) {
                        *reinterpret_cast<F32x4*>(stage + S_BASE + (r16 * kSRow + 16 * blk + 4 * kq) * 4) = d;
                    }
                }
            }
            lds_sync();
            static_for<0, kRuns>([&](auto ri) {
                constexpr int r = decltype(ri)::value;
                const unsigned u = (unsigned)(unit_of(ri) - pass * kPassRuns);
                const float sc = *reinterpret_cast<const float*>(
                    stage + S_BASE + (t * kSRow + (int)min(u, (unsigned)kPassRuns - 1) * 8 + i) * 4);
                logit[r] = u < (unsigned)kPassRuns ? sc : logit[r];
            });
            if (pass + 1 < passes) {
                lds_sync();  // the scores are picked: the area takes the next K rows
                uint32_t rr[kAccesses];
                pass_rows(pass + 1, rr);
                gather(k_bh, k_pitch, rr, min(kPassRows, total_rows - (pass + 1) * kPassRows), K_BASE);
            }
        }

        // ---- softmax over the neighbours and the blank token ---------------------------------------------------
        float x[kRuns];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < kRuns; ++r) {
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
        float p[kRuns];
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < kRuns; ++r) {
            p[r] = __expf(x[r] - mx);
            sum += p[r];
        }
        const float eb = __expf(bl - mx);
        const float total = oct_sum(sum) + eb;
        const float inv = 1.f / total;
        // for a backward pass that recomputes the probabilities: the logarithm of the softmax's denominator
        if (lse != nullptr && i == 0 && t < nt) lse[((int64_t)b * H_all + h0 + h) * N + i0 + t] = mx + __logf(total);
#pragma unroll
        for (int r = 0; r < kRuns; ++r) p[r] *= inv;
        if (i == 0) *reinterpret_cast<float*>(stage + PB_BASE + t * 4) = eb * inv;
        if (twice) {
#pragma unroll
            for (int c = kNnc - 1; c >= 1; --c) {
#pragma unroll
                for (int c2 = 0; c2 < c; ++c2) {
                    // the first listing of a cluster collects the probabilities of its repeats
                    const bool firstmatch = usc[c] == usc[c2] && ((repeats >> c) & 1) && !((repeats >> c2) & 1);
#pragma unroll
                    for (int q = 0; q < kSub; ++q) p[c2 * kSub + q] += firstmatch ? p[c * kSub + q] : 0.f;
                }
            }
        }

        // ---- weighted sum of the V rows --------------------------------------------------------------------------
        F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
            lds_sync();  // the previous reads of the probability area (K area) are complete
            // probabilities of this pass, re-indexed by distinct cluster: zero, then each lane puts in its own
            *reinterpret_cast<Piece*>(stage + P_BASE + lane * 16) = Piece{0u, 0u, 0u, 0u};
            static_assert(P_BYTES > 1024 && P_BYTES <= 2048, "two accesses clear the probabilities");
            if (lane < (P_BYTES - 1024) / 16) {
                *reinterpret_cast<Piece*>(stage + P_BASE + 1024 + lane * 16) = Piece{0u, 0u, 0u, 0u};
            }
            lds_sync();
            T* prow = reinterpret_cast<T*>(stage + P_BASE) + t * kPRow + i;
            static_for<0, kRuns>([&](auto ri) {
                constexpr int r = decltype(ri)::value;
                // runs of other passes, and repeats (already added to their first listing), go to the spare cells
                const unsigned u = ((repeats >> (r / kSub)) & 1) ? ~0u : (unsigned)(unit_of(ri) - pass * kPassRuns);
                prow[min(u, (unsigned)kPassRuns) * 8] = from_acc<T>(p[r]);
            });
            if (pass > 0) {
                lds_sync_vm<0>();  // the V rows of this pass are in LDS, the probabilities are written
            } else {
                lds_sync();
            }
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                if (s * 32 < rows_here) {
                    const Piece a = *reinterpret_cast<const Piece*>(stage + P_BASE + ((r16 & 7) * kPRow + 32 * s + 8 * kq) * 2);
                    const char* col = stage + V_BASE + (32 * s + 8 * kq + (r16 >> 2)) * kRB + (r16 & 3) * 8;
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        // rows 0-3 and 4-7 of the lane's 8, transposed to channel 16*cb + r16
                        const S4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32));
                        const S4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32 + 4 * kRB));
                        const U32x2 lo = __builtin_bit_cast(U32x2, b0), hi = __builtin_bit_cast(U32x2, b1);
                        acc[cb] = tile_mfma<T>(a, Piece{lo[0], lo[1], hi[0], hi[1]}, acc[cb]);
                    }
                }
            }
            lds_sync();  // the operands have been read: the V area and the probability area are free
            if (pass + 1 < passes) {
                uint32_t rr[kAccesses];
                pass_rows(pass + 1, rr);
                gather(v_bh, v_pitch, rr, min(kPassRows, total_rows - (pass + 1) * kPassRows), V_BASE);
            } else if (h + 1 < H) {
                gather_both(k_b + (int64_t)(h + 1) * ks.h * 2, v_b + (int64_t)(h + 1) * vs.h * 2, rr0, rows0);
                if (h + 2 < H) fetch_q(h + 2);
            }
        }

        // ---- blank token, output chunk (8 tokens x 32 channels, row-major) -----------------------------------------------
        if (kq < 2) {
            const F32x4 pb = *reinterpret_cast<const F32x4*>(stage + PB_BASE + 16 * kq);
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    reinterpret_cast<T*>(stage + O_BASE)[(4 * kq + e) * kC + 16 * cb + r16] =
                        from_acc<T>(acc[cb][e] + pb[e] * bv[cb]);
                }
            }
        }
        lds_sync();
        // the head's only store, and the last vector-memory operation it issues (see the wait at the top of the loop)
        if (lane < 32 && g_sub < nt) {
            const Piece o = *reinterpret_cast<const Piece*>(stage + O_BASE + lane * 16);
            char* dst = reinterpret_cast<char*>(out + (int64_t)b * os.b + (int64_t)(h0 + h) * os.h + (int64_t)(i0 + g_sub) * os.n);
            *reinterpret_cast<Piece*>(dst + g_pos * 16) = o;   // plain: the output projection reads it next
        }
    }
}

template <typename T, int CS>
int launch_typed(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                 clusten_strides vs, const int32_t* cluster_idx, const void* table, const int64_t* pe_idx,
                 const int64_t* mask, const float* blank_k, const float* blank_v, void* out, clusten_strides os,
                 float scale, int lists_shared, const void* plan, float* lse, const clusten_attn_shape& s,
                 hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int groups = head_groups_for(total, s.H);  // 196 tokens x 8 heads, B = 128: 69.6 -> 63.9 us
    hipLaunchKernelGGL((cluster_attention_kernel<T, CS>), dim3(xcd_grid(total * groups)), dim3(kWave), 0, stream,
                       static_cast<const T*>(q), qs, static_cast<const T*>(k), ks, static_cast<const T*>(v), vs,
                       cluster_idx, static_cast<const T*>(table), pe_idx, mask, blank_k, blank_v, static_cast<T*>(out),
                       os, s.H, s.N, scale, tiles_per_batch, total, lists_shared, groups, static_cast<const char*>(plan), lse);
    return launch_status();
}

}  // namespace

size_t cluster_attention_plan_bytes(int B, int N, int M) {
    const size_t per_tile = M == Geo<24>::kM ? Geo<24>::kPlanBytes : (M == Geo<8>::kM ? Geo<8>::kPlanBytes : 0);
    return (size_t)B * ((N + kTileTokens - 1) / kTileTokens) * per_tile;
}

int launch_cluster_attention_plan(const int32_t* cluster_idx, const int64_t* pe_idx, const int64_t* mask, void* plan,
                                  int B, int N, int M, hipStream_t stream) {
    const int tiles_per_batch = (N + kTileTokens - 1) / kTileTokens;
    const int64_t total = (int64_t)B * tiles_per_batch;
    if (total <= 0 || total >= ((int64_t)1 << 30)) return CLUSTEN_ERR_BAD_DIMS;
    const int cluster_size = M / kNnc;
    if (M % kNnc != 0) return CLUSTEN_ERR_BAD_DIMS;
    if (cluster_size == 8) {
        hipLaunchKernelGGL(cluster_attention_plan_kernel<8>, dim3((unsigned)total), dim3(kWave), 0, stream, cluster_idx,
                           pe_idx, mask, static_cast<char*>(plan), N, tiles_per_batch, (int)total);
    } else if (cluster_size == 24) {
        hipLaunchKernelGGL(cluster_attention_plan_kernel<24>, dim3((unsigned)total), dim3(kWave), 0, stream, cluster_idx,
                           pe_idx, mask, static_cast<char*>(plan), N, tiles_per_batch, (int)total);
    } else {
        return CLUSTEN_ERR_BAD_DIMS;
    }
    return launch_status();
}

int launch_cluster_attention(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                             clusten_strides vs, const int32_t* cluster_idx, const void* table, const int64_t* pe_idx,
                             const int64_t* mask, const float* blank_k, const float* blank_v, void* out,
                             clusten_strides os, float scale, int lists_shared, const void* plan, float* lse,
                             clusten_attn_shape s, int dtype, hipStream_t stream) {
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16 && dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    // six clusters per token: 48 neighbours = clusters of 8, 144 = clusters of 24
    if (s.C != kC || (s.M != Geo<8>::kM && s.M != Geo<24>::kM)) return CLUSTEN_ERR_BAD_DIMS;
    const int cluster_size = s.M / kNnc;
    if (cluster_size == 24 && dtype == CLUSTEN_F32) return CLUSTEN_ERR_BAD_DIMS;   // clusters of 24: 16-bit data only
    const size_t eb = dtype_size(dtype);
    const bool ok = rows_aligned16(q, qs, eb) && rows_aligned16(k, ks, eb) && rows_aligned16(v, vs, eb) &&
                    rows_aligned16(out, os, eb) && aligned16(blank_k) && slice_fits_int32(ks, s.H, s.N, s.C) &&
                    slice_fits_int32(vs, s.H, s.N, s.C) && slice_fits_int32(qs, s.H, s.N, s.C);
    if (!ok) return CLUSTEN_ERR_UNALIGNED;
    if (dtype == CLUSTEN_F32) {
        return launch_cluster_attention_f32(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os,
                                            scale, lists_shared, plan, lse, s, stream);
    }
    if (cluster_size == 24) {
        if (dtype == CLUSTEN_F16) {
            return launch_typed<f16_t, 24>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os,
                                           scale, lists_shared, plan, lse, s, stream);
        }
        return launch_typed<bf16_t, 24>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os,
                                        scale, lists_shared, plan, lse, s, stream);
    }
    if (cluster_attention_resident_takes(s, dtype)) {
        return launch_cluster_attention_resident(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out,
                                                 os, scale, lists_shared, plan, lse, s, dtype, stream);
    }
    if (dtype == CLUSTEN_F16) {
        return launch_typed<f16_t, 8>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os, scale,
                                      lists_shared, plan, lse, s, stream);
    }
    return launch_typed<bf16_t, 8>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os, scale,
                                   lists_shared, plan, lse, s, stream);
}

}  // namespace clusten
