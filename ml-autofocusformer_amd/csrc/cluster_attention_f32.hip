// cluster_attention for fp32 data: the one-kernel local attention of cluster_attention.hip (same inputs, same plan,
// same result layout; models/aff_transformer.py:120-155 with clusten/src/clustenqk_cuda_kernel.cu:18-49 and
// clusten/src/clustenav_cuda_kernel.cu:18-49 between the tensor expressions) with every sum and product in fp32.
//
// What differs from the 16-bit kernel is the matrix side.  Rows are 128 bytes, so a pass holds the rows of 6 distinct
// clusters (48 rows, 6 KB each for K and V: the same LDS per wave) and most tiles take two passes per head.  The
// products are `v_mfma_f32_16x16x4_f32`; a sum over k may take its terms in any order as long as both operands agree,
// which lets every operand be read as 16-byte pieces:
//   QK  S[row][token] = K_pass (48 x 32) * q^T: lane (r16, kq) reads pieces 2 kq and 2 kq + 1 of its K row and of its
//       token's q row - k-step (j, e) is channel 8 kq + 4 j + e for both;
//   AV  out (8 x 32) = P_pass (8 x 48) * V_pass: lane (r16, kq) reads probabilities 16 j + 4 kq .. + 3 of its token as
//       one piece - k-step (j, e) is pass row 16 j + 4 kq + e - and channel 16 cb + r16 of those V rows one float at a
//       time.
// Rows travel to LDS by LDS-direct loads, one cluster (8 rows of 8 pieces) per wave access; piece P of row R lands at
// position P ^ (R & 7) of the row, so that the 16 rows a matrix operand reads at once fall into different banks.
#include "cluster_attention_plan.hpp"

namespace clusten {
namespace {

using namespace ca;

constexpr int fRB = kC * 4;            // bytes per row
constexpr int fPassRuns = 6;           // distinct clusters per pass (8 or 12, with the LDS they take, are no faster)
constexpr int fPassRows = 8 * fPassRuns;
constexpr int fBlocks = fPassRows / 16;    // 16-row blocks of the score product and of the value product's k range
constexpr int fAccesses = fPassRuns;       // wave accesses (one cluster: 8 rows of 128 bytes) per pass
constexpr int fSRow = fPassRows + 4;       // floats per token row of the score matrix
constexpr int fPRow = fPassRows + 8;       // floats per token row of the re-indexed probabilities; the last 8 are never
                                           // read: cells for the writes of runs outside the pass

// LDS: two row areas and small tables (the layout of the 16-bit kernel).
constexpr int K_BASE = 0;
constexpr int S_BASE = K_BASE;
constexpr int P_BASE = K_BASE;
constexpr int P_BYTES = kTileTokens * fPRow * 4;
constexpr int V_BASE = K_BASE + fPassRows * fRB;
constexpr int O_BASE = V_BASE + fPassRows * fRB;           // output chunk of a head
constexpr int Q_BASE = O_BASE + kTileTokens * fRB;         // q rows of two heads (slot h % 2)
constexpr int Q_SLOT = kTileTokens * fRB;
constexpr int UL_BASE = Q_BASE + 2 * Q_SLOT;               // cluster number of each distinct cluster
constexpr int PB_BASE = UL_BASE + kTileTokens * kR * 4;    // blank-token probability per token
constexpr int LDS_BYTES = PB_BASE + kTileTokens * 4;
static_assert(P_BYTES % 16 == 0 && P_BYTES <= fPassRows * fRB, "the probabilities fit the K area");
static_assert(kTileTokens * fSRow * 4 <= fPassRows * fRB, "the scores fit the K area");

__global__ __launch_bounds__(kWave) void cluster_attention_f32_kernel(
    const float* __restrict__ q, clusten_strides qs, const float* __restrict__ k, clusten_strides ks,
    const float* __restrict__ v, clusten_strides vs, const int32_t* __restrict__ cluster_idx,
    const float* __restrict__ table, const int64_t* __restrict__ pe_idx, const int64_t* __restrict__ mask,
    const float* __restrict__ blank_k, const float* __restrict__ blank_v, float* __restrict__ out, clusten_strides os,
    int H_all, int N, float scale, int tiles_per_batch, int total_tiles, int lists_shared, int head_groups,
    const char* __restrict__ plan, float* __restrict__ lse) {
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
    const int g_sub = lane >> 3;   // gather side: row of an 8-row access
    const int g_pos = lane & 7;    //              position of the 16-byte piece in the row
    const int t = lane >> 3;       // softmax side: token of the tile (tokens past a partial tile repeat its last one)
    const int i = lane & 7;        //               member of each cluster
    const int64_t list_b = lists_shared ? 0 : b;
    const int64_t tok = list_b * N + i0 + min(t, nt - 1);

    // q rows of head h -> slot h % 2: lane (token, position) fetches piece position ^ token
    const char* q_tile = reinterpret_cast<const char*>(q + (int64_t)b * qs.b + (int64_t)h0 * qs.h + (int64_t)i0 * qs.n);
    const uint32_t q_off = (uint32_t)min(g_sub, nt - 1) * (uint32_t)qs.n * 4 + (uint32_t)(g_pos ^ g_sub) * 16;
    auto fetch_q = [&](int h) {
        CLUSTEN_LDS_DMA16(q_tile + (int64_t)h * qs.h * 4 + lane_offset(q_off), stage + Q_BASE + (h & 1) * Q_SLOT);
    };
    fetch_q(0);
    if (H > 1) fetch_q(1);

    int pe[kR];      // per-slot inputs the heads share: row of the bias table; the sign bit marks a masked slot
    int us[kR];      // distinct-cluster number of this lane's token's runs
    int repeats = 0; // bit r: run r repeats an earlier run of the token; its probability is added to that run's
    int U = 0;
    int* ulist = reinterpret_cast<int*>(stage + UL_BASE);
    if (plan != nullptr) {
        // the tile's plan, built once for all layers that use these lists
        const char* mine = plan + (list_b * tiles_per_batch + (tile - b * tiles_per_batch)) * (int64_t)kPlanBytes;
        const Piece lo = *reinterpret_cast<const Piece*>(mine + kPlanLane + lane * 32);
        const Piece hi = *reinterpret_cast<const Piece*>(mine + kPlanLane + lane * 32 + 16);
        U = *reinterpret_cast<const int*>(mine);
        if (lane < kTileTokens * kR) ulist[lane] = *reinterpret_cast<const int*>(mine + 16 + lane * 4);
        pe[0] = (int)lo[0]; pe[1] = (int)lo[1]; pe[2] = (int)lo[2]; pe[3] = (int)lo[3];
        pe[4] = (int)hi[0]; pe[5] = (int)hi[1];
        us[0] = hi[2] & 0xff; us[1] = (hi[2] >> 8) & 0xff; us[2] = (hi[2] >> 16) & 0xff; us[3] = hi[2] >> 24;
        us[4] = hi[3] & 0xff; us[5] = (hi[3] >> 8) & 0xff;
        repeats = (hi[3] >> 16) & 0xff;
    } else {
        tile_setup(cluster_idx, pe_idx, mask, list_b, N, i0, nt, tok, pe, us, repeats, U, ulist);
    }
    const bool twice = __any(repeats) != 0;
    lds_sync();

    const int total_rows = 8 * U;
    const int passes = (U + fPassRuns - 1) / fPassRuns;
    const uint32_t k_pitch = (uint32_t)ks.n * 4, v_pitch = (uint32_t)vs.n * 4;
    const char* k_b = reinterpret_cast<const char*>(k + (int64_t)b * ks.b + (int64_t)h0 * ks.h);
    const char* v_b = reinterpret_cast<const char*>(v + (int64_t)b * vs.b + (int64_t)h0 * vs.h);

    // rows of the distinct clusters 6*pass .. 6*pass+5, as this lane gathers them: access a moves the 8 rows of cluster
    // a of the pass; clusters past the last one repeat it so that every row of a 16-row block holds data
    auto pass_rows = [&](int pass, uint32_t (&rr)[fAccesses]) {
#pragma unroll
        for (int a = 0; a < fAccesses; ++a) {
            const int c = ulist[min(pass * fPassRuns + a, U - 1)];
            const int row = c * 8 + g_sub;
            rr[a] = (unsigned)row < (unsigned)N ? (uint32_t)row : 0u;
        }
    };
    auto gather = [&](const char* rows_bh, uint32_t pitch, const uint32_t (&rr)[fAccesses], int rows_here, int lds_base) {
#pragma unroll
        for (int a = 0; a < fAccesses; ++a) {
            if ((a & ~1) * 8 < rows_here) {
                CLUSTEN_LDS_DMA16(rows_bh + lane_offset(rr[a] * pitch + (uint32_t)(g_pos ^ g_sub) * 16), stage + lds_base + a * 1024);
            }
        }
    };
    uint32_t rr0[fAccesses];  // pass 0: used by every head
    pass_rows(0, rr0);
    const int rows0 = min(fPassRows, total_rows);
    gather(k_b, k_pitch, rr0, rows0, K_BASE);
    gather(v_b, v_pitch, rr0, rows0, V_BASE);

    for (int h = 0; h < H; ++h) {
        const char* k_bh = k_b + (int64_t)h * ks.h * 4;
        const char* v_bh = v_b + (int64_t)h * vs.h * 4;
        const char* q_lds = stage + Q_BASE + (h & 1) * Q_SLOT;

        // The first K and V rows of this head were requested during the previous head (or above); the only
        // vector-memory operation issued after them is that head's output store, which may stay in flight.
        if (h == 0) {
            lds_sync_vm<0>();
        } else {
            lds_sync_vm<1>();
        }

        // small per-head operands: their latency passes under the score computation
        float bias[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t cell = lane_offset(((uint32_t)(pe[r] & 0x7fffffff) * (uint32_t)H_all + (uint32_t)(h0 + h)) * 4);
            bias[r] = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(table) + cell) + (pe[r] < 0 ? -100.f : 0.f);
        }
        const float4 bk = *reinterpret_cast<const float4*>(blank_k + (h0 + h) * kC + 4 * i);
        const float bv[2] = {blank_v[(h0 + h) * kC + r16], blank_v[(h0 + h) * kC + 16 + r16]};

        // ---- scores -------------------------------------------------------------------------------------
        float logit[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) logit[r] = 0.f;
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(fPassRows, total_rows - pass * fPassRows);
            if (pass > 0) lds_sync_vm<0>();  // the K rows of this pass are in LDS
            // pieces 2 kq + j of the lane's q row and K rows: position (2 kq + j) ^ (row & 7)
            F32x4 qv[2];
            F32x4 kv[fBlocks][2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int pos = ((2 * kq + j) ^ (r16 & 7)) * 16;
                qv[j] = *reinterpret_cast<const F32x4*>(q_lds + (r16 & 7) * fRB + pos);
#pragma unroll
                for (int blk = 0; blk < fBlocks; ++blk) {
                    if (blk * 16 < rows_here) {
                        kv[blk][j] = *reinterpret_cast<const F32x4*>(stage + K_BASE + (blk * 16 + r16) * fRB + pos);
                    }
                }
            }
            lds_sync();  // the K rows are in registers: their area takes the scores
#pragma unroll
            for (int blk = 0; blk < fBlocks; ++blk) {
                if (blk * 16 < rows_here) {
                    F32x4 d = F32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) d = mfma_16x16x4(kv[blk][j][e], qv[j][e], d);
                    }
                    // lane (r16, kq): pass rows 16*blk + 4*kq .. +3 of token r16
                    if (r16 < kTileTokens) {
                        *reinterpret_cast<F32x4*>(stage + S_BASE + (r16 * fSRow + 16 * blk + 4 * kq) * 4) = d;
                    }
                }
            }
            lds_sync();
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const unsigned u = (unsigned)(us[r] - pass * fPassRuns);
                const float sc = *reinterpret_cast<const float*>(
                    stage + S_BASE + (t * fSRow + (int)min(u, (unsigned)fPassRuns - 1) * 8 + i) * 4);
                logit[r] = u < (unsigned)fPassRuns ? sc : logit[r];
            }
            if (pass + 1 < passes) {
                lds_sync();  // the scores are picked: the area takes the next K rows
                uint32_t rr[fAccesses];
                pass_rows(pass + 1, rr);
                gather(k_bh, k_pitch, rr, min(fPassRows, total_rows - (pass + 1) * fPassRows), K_BASE);
            }
        }

        // ---- softmax over the 48 neighbours and the blank token ----------------------------------------------
        float x[kR];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            x[r] = logit[r] * scale + bias[r];
            mx = fmaxf(mx, x[r]);
        }
        float part = 0.f;
        {
            // channels 4 i .. 4 i + 3 of the token's q row: piece i, at position i ^ token
            const F32x4 qr = *reinterpret_cast<const F32x4*>(q_lds + t * fRB + ((i ^ t) * 16));
            part = qr[0] * bk.x + qr[1] * bk.y + qr[2] * bk.z + qr[3] * bk.w;
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
        if (lse != nullptr && i == 0 && t < nt) lse[((int64_t)b * H_all + h0 + h) * N + i0 + t] = mx + __logf(total);
#pragma unroll
        for (int r = 0; r < kR; ++r) p[r] *= inv;
        if (i == 0) *reinterpret_cast<float*>(stage + PB_BASE + t * 4) = eb * inv;
        if (twice) {
#pragma unroll
            for (int r = kR - 1; r >= 1; --r) {
#pragma unroll
                for (int r2 = 0; r2 < r; ++r2) {
                    // the first run with the same cluster collects the probabilities of its repeats
                    bool firstmatch = us[r] == us[r2] && ((repeats >> r) & 1) && !((repeats >> r2) & 1);
                    p[r2] += firstmatch ? p[r] : 0.f;
                }
            }
        }

        // ---- weighted sum of the V rows --------------------------------------------------------------------------
        F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(fPassRows, total_rows - pass * fPassRows);
            lds_sync();  // the previous reads of the probability area (K area) are complete
            // probabilities of this pass, re-indexed by distinct cluster: zero, then each lane puts in its own
#pragma unroll
            for (int z = 0; z < P_BYTES; z += 1024) {
                if (z + 1024 <= P_BYTES || lane < (P_BYTES - z) / 16) {
                    *reinterpret_cast<Piece*>(stage + P_BASE + z + lane * 16) = Piece{0u, 0u, 0u, 0u};
                }
            }
            lds_sync();
            float* prow = reinterpret_cast<float*>(stage + P_BASE) + t * fPRow + i;
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                // runs of other passes, and repeats (already added to their first run), go to the spare cells
                const unsigned u = ((repeats >> r) & 1) ? ~0u : (unsigned)(us[r] - pass * fPassRuns);
                prow[min(u, (unsigned)fPassRuns) * 8] = p[r];
            }
            if (pass > 0) {
                lds_sync_vm<0>();  // the V rows of this pass are in LDS, the probabilities are written
            } else {
                lds_sync();
            }
#pragma unroll
            for (int j = 0; j < fBlocks; ++j) {
                if (j * 16 < rows_here) {
                    // k-step (j, e): pass row 16 j + 4 kq + e
                    const F32x4 a = *reinterpret_cast<const F32x4*>(stage + P_BASE + ((r16 & 7) * fPRow + 16 * j + 4 * kq) * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = 16 * j + 4 * kq + e;
                        const char* vrow = stage + V_BASE + row * fRB + (r16 & 3) * 4;
#pragma unroll
                        for (int cb = 0; cb < 2; ++cb) {
                            const float bval = *reinterpret_cast<const float*>(vrow + (((4 * cb + (r16 >> 2)) ^ (row & 7)) * 16));
                            acc[cb] = mfma_16x16x4(a[e], bval, acc[cb]);
                        }
                    }
                }
            }
            lds_sync();  // the operands have been read: the V area and the probability area are free
            if (pass + 1 < passes) {
                uint32_t rr[fAccesses];
                pass_rows(pass + 1, rr);
                gather(v_bh, v_pitch, rr, min(fPassRows, total_rows - (pass + 1) * fPassRows), V_BASE);
            } else if (h + 1 < H) {
                gather(k_b + (int64_t)(h + 1) * ks.h * 4, k_pitch, rr0, rows0, K_BASE);
                gather(v_b + (int64_t)(h + 1) * vs.h * 4, v_pitch, rr0, rows0, V_BASE);
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
                    reinterpret_cast<float*>(stage + O_BASE)[(4 * kq + e) * kC + 16 * cb + r16] = acc[cb][e] + pb[e] * bv[cb];
                }
            }
        }
        lds_sync();
        // the head's only store, and the last vector-memory operation it issues (see the wait at the top of the loop)
        if (g_sub < nt) {
            const Piece o = *reinterpret_cast<const Piece*>(stage + O_BASE + lane * 16);
            char* dst = reinterpret_cast<char*>(out + (int64_t)b * os.b + (int64_t)(h0 + h) * os.h + (int64_t)(i0 + g_sub) * os.n);
            *reinterpret_cast<Piece*>(dst + g_pos * 16) = o;   // plain: the output projection reads it next
        }
    }
}

}  // namespace

int launch_cluster_attention_f32(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                 clusten_strides vs, const int32_t* cluster_idx, const void* table, const int64_t* pe_idx,
                                 const int64_t* mask, const float* blank_k, const float* blank_v, void* out,
                                 clusten_strides os, float scale, int lists_shared, const void* plan, float* lse,
                                 const clusten_attn_shape& s, hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int groups = head_groups_for(total, s.H);
    hipLaunchKernelGGL(cluster_attention_f32_kernel, dim3(xcd_grid(total * groups)), dim3(kWave), 0, stream,
                       static_cast<const float*>(q), qs, static_cast<const float*>(k), ks, static_cast<const float*>(v), vs,
                       cluster_idx, static_cast<const float*>(table), pe_idx, mask, blank_k, blank_v,
                       static_cast<float*>(out), os, s.H, s.N, scale, tiles_per_batch, total, lists_shared, groups,
                       static_cast<const char*>(plan), lse);
    return launch_status();
}

}  // namespace clusten
