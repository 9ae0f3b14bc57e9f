// cluster_attention_backward for fp32 data: the query-side half of the backward of the one-kernel local attention
// (cluster_attention_bwd.hip: same inputs, same plan, same results and layouts; the backward of
// models/aff_transformer.py:120-155 with clusten/src/clustenqk_cuda_kernel.cu:51-132 and
// clusten/src/clustenav_cuda_kernel.cu:51-127 between the tensor expressions) with every sum and product in fp32.
//
//   p = exp(x - lse),  dP[t,j] = d_out[t] . v[row(t,j)],  delta[t] = d_out[t] . out[t],
//   dS = p * (dP - delta),  d_q[t] = scale * (sum_j dS[t,j] * k[row(t,j)] + dS_b[t] * blank_k)
//
// The matrix side is that of cluster_attention_f32.hip: rows of 128 bytes, the rows of 6 distinct clusters a pass (48
// rows of K and 48 of V), `v_mfma_f32_16x16x4_f32` on operands read as 16-byte pieces, piece P of row R at position
// P ^ (R & 7) of its row in LDS.  Per pass S = K q^T and dP = V d_out^T (24 instructions each), every lane picks the
// scores and dP of its own slots and forms p and dS, and dS re-indexed by distinct cluster times the K rows of the
// pass is added to the query gradient.  `out` is fp32 here, so delta is taken from it directly and most tiles, which
// need two passes, still sweep their rows once.
#include "cluster_attention_plan.hpp"

namespace clusten {
namespace {

using namespace ca;

constexpr int fRB = kC * 4;            // bytes per row
constexpr int fPassRuns = 6;           // distinct clusters per pass
constexpr int fPassRows = 8 * fPassRuns;
constexpr int fBlocks = fPassRows / 16;
constexpr int fAccesses = fPassRuns;   // wave accesses (one cluster: 8 rows of 128 bytes) per pass
constexpr int fSRow = fPassRows + 4;   // floats per token row of a score matrix
constexpr int fPRow = fPassRows + 8;   // floats per token row of the re-indexed logit gradients; the last 8 take the
                                       // writes of runs outside the pass and are never read

constexpr int K_BASE = 0;
constexpr int V_BASE = K_BASE + fPassRows * fRB;
constexpr int Q_BASE = V_BASE + fPassRows * fRB;           // q rows of two heads (slot h % 2)
constexpr int Q_SLOT = kTileTokens * fRB;
constexpr int G_BASE = Q_BASE + 2 * Q_SLOT;                // d_out rows of two heads
constexpr int O_BASE = G_BASE + 2 * Q_SLOT;                // d_q chunk of a head
constexpr int S_BASE = O_BASE + kTileTokens * fRB;         // scores; later the re-indexed logit gradients
constexpr int D_BASE = S_BASE;
constexpr int D_BYTES = kTileTokens * fPRow * 4;
constexpr int S_BYTES = D_BYTES;
constexpr int S2_BASE = S_BASE + S_BYTES;                  // dP; after the passes the blank token's logit gradients
constexpr int PW_BASE = S2_BASE + S_BYTES;                 // p rows of a head (8 x 48), then its dS rows
constexpr int PW_BYTES = kTileTokens * kM * 4;
constexpr int UL_BASE = PW_BASE + 2 * PW_BYTES;
constexpr int LDS_BYTES = UL_BASE + kTileTokens * kR * 4;
static_assert(kTileTokens * fSRow * 4 <= S_BYTES, "the scores fit their area");
static_assert(D_BYTES > 1024 && D_BYTES <= 2048, "the logit gradients are cleared in two wave stores");
static_assert(S_BASE % 16 == 0 && S2_BASE % 16 == 0 && Q_BASE % 1024 == 0 && PW_BASE % 16 == 0, "aligned areas");

__global__ __launch_bounds__(kWave) void cluster_attention_bwd_f32_kernel(
    const float* __restrict__ q, clusten_strides qs, const float* __restrict__ k, clusten_strides ks,
    const float* __restrict__ v, clusten_strides vs, const float* __restrict__ d_out, clusten_strides gs,
    const float* __restrict__ out, clusten_strides os, const float* __restrict__ lse,
    const int32_t* __restrict__ cluster_idx, const float* __restrict__ table, const int64_t* __restrict__ pe_idx,
    const int64_t* __restrict__ mask, const float* __restrict__ blank_k, const float* __restrict__ blank_v,
    float* __restrict__ d_q, clusten_strides dqs, float* __restrict__ probs, float* __restrict__ d_logit,
    float* __restrict__ p_blank, float* __restrict__ ds_blank, int H_all, int N, float scale, int tiles_per_batch,
    int total_tiles, int lists_shared, int head_groups, const char* __restrict__ plan) {
    __shared__ __attribute__((aligned(1024))) char stage[LDS_BYTES];

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
    const int r16 = lane & 15, kq = lane >> 4;     // matrix side
    const int g_sub = lane >> 3, g_pos = lane & 7; // gather side: row of an 8-row access, position of the 16-byte piece
    const int t = lane >> 3, i = lane & 7;         // softmax side: token of the tile, member of each cluster
    const int tc = min(t, nt - 1);
    const int64_t list_b = lists_shared ? 0 : b;
    const int64_t tok = list_b * N + i0 + tc;

    // q and d_out rows of head h -> slot h % 2: lane (token, position) fetches piece position ^ token
    const char* q_tile = reinterpret_cast<const char*>(q + (int64_t)b * qs.b + (int64_t)h0 * qs.h + (int64_t)i0 * qs.n);
    const char* g_tile = reinterpret_cast<const char*>(d_out + (int64_t)b * gs.b + (int64_t)h0 * gs.h + (int64_t)i0 * gs.n);
    const uint32_t q_off = (uint32_t)tc * (uint32_t)qs.n * 4 + (uint32_t)(g_pos ^ g_sub) * 16;
    const uint32_t g_off = (uint32_t)tc * (uint32_t)gs.n * 4 + (uint32_t)(g_pos ^ g_sub) * 16;
    auto fetch_rows = [&](int h) {
        CLUSTEN_LDS_DMA16(q_tile + (int64_t)h * qs.h * 4 + lane_offset(q_off), stage + Q_BASE + (h & 1) * Q_SLOT);
        CLUSTEN_LDS_DMA16(g_tile + (int64_t)h * gs.h * 4 + lane_offset(g_off), stage + G_BASE + (h & 1) * Q_SLOT);
    };
    fetch_rows(0);
    if (H > 1) fetch_rows(1);

    int pe[kR], us[kR];
    int repeats = 0, U = 0;
    int* ulist = reinterpret_cast<int*>(stage + UL_BASE);
    if (plan != nullptr) {
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
    uint32_t rr0[fAccesses];
    pass_rows(0, rr0);
    const int rows0 = min(fPassRows, total_rows);
    gather(k_b, k_pitch, rr0, rows0, K_BASE);
    gather(v_b, v_pitch, rr0, rows0, V_BASE);

    for (int h = 0; h < H; ++h) {
        const int hh = h0 + h;
        const char* k_bh = k_b + (int64_t)h * ks.h * 4;
        const char* v_bh = v_b + (int64_t)h * vs.h * 4;
        const char* q_lds = stage + Q_BASE + (h & 1) * Q_SLOT;
        const char* g_lds = stage + G_BASE + (h & 1) * Q_SLOT;

        // small per-head operands of the lane's token, requested before the wait for the rows
        float bias[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t cell = lane_offset(((uint32_t)(pe[r] & 0x7fffffff) * (uint32_t)H_all + (uint32_t)hh) * 4);
            bias[r] = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(table) + cell) + (pe[r] < 0 ? -100.f : 0.f);
        }
        const float4 bk = *reinterpret_cast<const float4*>(blank_k + hh * kC + 4 * i);
        const float4 bv4 = *reinterpret_cast<const float4*>(blank_v + hh * kC + 4 * i);
        const float lse_t = lse[((int64_t)b * H_all + hh) * N + i0 + tc];
        const float4 o4 = *reinterpret_cast<const float4*>(out + (int64_t)b * os.b + (int64_t)hh * os.h +
                                                           (int64_t)(i0 + tc) * os.n + 4 * i);

        lds_sync_vm<0>();   // the rows of this head's first pass, its q and d_out rows, the operands above

        // per token: delta = d_out . out, the blank token's probability and logit gradient
        float delta, p_b, ds_b;
        {
            // channels 4 i .. 4 i + 3 of the token's rows: piece i, at position i ^ token
            const F32x4 g4 = *reinterpret_cast<const F32x4*>(g_lds + t * fRB + ((i ^ t) * 16));
            const F32x4 q4 = *reinterpret_cast<const F32x4*>(q_lds + t * fRB + ((i ^ t) * 16));
            delta = oct_sum(g4[0] * o4.x + g4[1] * o4.y + g4[2] * o4.z + g4[3] * o4.w);
            const float dpb = oct_sum(g4[0] * bv4.x + g4[1] * bv4.y + g4[2] * bv4.z + g4[3] * bv4.w);
            const float bl = oct_sum(q4[0] * bk.x + q4[1] * bk.y + q4[2] * bk.z + q4[3] * bk.w) * scale;
            p_b = __expf(bl - lse_t);
            ds_b = p_b * (dpb - delta);
        }
        // pieces 2 kq + j of the lane's token's q and d_out rows (B operands of both score products)
        F32x4 qv[2], gv[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int pos = ((2 * kq + j) ^ (r16 & 7)) * 16;
            qv[j] = *reinterpret_cast<const F32x4*>(q_lds + (r16 & 7) * fRB + pos);
            gv[j] = *reinterpret_cast<const F32x4*>(g_lds + (r16 & 7) * fRB + pos);
        }

        float p_all[kR], ds_all[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) p_all[r] = ds_all[r] = 0.f;
        F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(fPassRows, total_rows - pass * fPassRows);
            if (pass > 0) lds_sync_vm<0>();  // the K and V rows of this pass are in LDS
            // ---- S = K q^T and dP = V d_out^T --------------------------------------------------------------
#pragma unroll
            for (int blk = 0; blk < fBlocks; ++blk) {
                if (blk * 16 < rows_here) {
                    F32x4 s = F32x4{0.f, 0.f, 0.f, 0.f}, d = F32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const int pos = ((2 * kq + j) ^ (r16 & 7)) * 16;
                        const F32x4 kv = *reinterpret_cast<const F32x4*>(stage + K_BASE + (blk * 16 + r16) * fRB + pos);
                        const F32x4 vv = *reinterpret_cast<const F32x4*>(stage + V_BASE + (blk * 16 + r16) * fRB + pos);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            s = mfma_16x16x4(kv[e], qv[j][e], s);
                            d = mfma_16x16x4(vv[e], gv[j][e], d);
                        }
                    }
                    // lane (r16, kq): pass rows 16*blk + 4*kq .. +3 of token r16
                    if (r16 < kTileTokens) {
                        *reinterpret_cast<F32x4*>(stage + S_BASE + (r16 * fSRow + 16 * blk + 4 * kq) * 4) = s;
                        *reinterpret_cast<F32x4*>(stage + S2_BASE + (r16 * fSRow + 16 * blk + 4 * kq) * 4) = d;
                    }
                }
            }
            lds_sync();
            // ---- the lane's own slots: p and dS ---------------------------------------------------------------
            float ds_pass[kR];
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const unsigned u = (unsigned)(us[r] - pass * fPassRuns);
                const bool in = u < (unsigned)fPassRuns;
                const int cell = (t * fSRow + (int)min(u, (unsigned)fPassRuns - 1) * 8 + i) * 4;
                const float sc = *reinterpret_cast<const float*>(stage + S_BASE + cell);
                const float dp = *reinterpret_cast<const float*>(stage + S2_BASE + cell);
                const float pr = __expf(sc * scale + bias[r] - lse_t);
                const float ds = pr * (dp - delta);
                p_all[r] = in ? pr : p_all[r];
                ds_all[r] = in ? ds : ds_all[r];
                ds_pass[r] = in ? ds : 0.f;
            }
            if (twice) {
#pragma unroll
                for (int r = kR - 1; r >= 1; --r) {
#pragma unroll
                    for (int r2 = 0; r2 < r; ++r2) {
                        // the first run with the same cluster collects the gradients of its repeats (same K rows)
                        bool firstmatch = us[r] == us[r2] && ((repeats >> r) & 1) && !((repeats >> r2) & 1);
                        ds_pass[r2] += firstmatch ? ds_pass[r] : 0.f;
                    }
                }
            }
            lds_sync();  // the scores have been picked: their area takes the re-indexed logit gradients
            *reinterpret_cast<Piece*>(stage + D_BASE + lane * 16) = Piece{0u, 0u, 0u, 0u};
            if (lane < (D_BYTES - 1024) / 16) {
                *reinterpret_cast<Piece*>(stage + D_BASE + 1024 + lane * 16) = Piece{0u, 0u, 0u, 0u};
            }
            lds_sync();
            {
                float* drow = reinterpret_cast<float*>(stage + D_BASE) + t * fPRow + i;
#pragma unroll
                for (int r = 0; r < kR; ++r) {
                    // runs of other passes (their gradient is zero here) and repeats (already added to their first run)
                    // go to the spare cells
                    const unsigned u = ((repeats >> r) & 1) ? ~0u : (unsigned)(us[r] - pass * fPassRuns);
                    drow[min(u, (unsigned)fPassRuns) * 8] = ds_pass[r];
                }
            }
            lds_sync();
            // ---- d_q += dS_pass (8 x 48) * K_pass (48 x 32) ---------------------------------------------------
#pragma unroll
            for (int j = 0; j < fBlocks; ++j) {
                if (j * 16 < rows_here) {
                    // k-step (j, e): pass row 16 j + 4 kq + e
                    const F32x4 a = *reinterpret_cast<const F32x4*>(stage + D_BASE + ((r16 & 7) * fPRow + 16 * j + 4 * kq) * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = 16 * j + 4 * kq + e;
                        const char* krow = stage + K_BASE + row * fRB + (r16 & 3) * 4;
#pragma unroll
                        for (int cb = 0; cb < 2; ++cb) {
                            const float bval = *reinterpret_cast<const float*>(krow + (((4 * cb + (r16 >> 2)) ^ (row & 7)) * 16));
                            acc[cb] = mfma_16x16x4(a[e], bval, acc[cb]);
                        }
                    }
                }
            }
            lds_sync();  // the K and V rows and the logit gradients have been read
            if (pass + 1 < passes) {
                uint32_t rr[fAccesses];
                pass_rows(pass + 1, rr);
                const int next_rows = min(fPassRows, total_rows - (pass + 1) * fPassRows);
                gather(k_bh, k_pitch, rr, next_rows, K_BASE);
                gather(v_bh, v_pitch, rr, next_rows, V_BASE);
            } else if (h + 1 < H) {
                gather(k_b + (int64_t)(h + 1) * ks.h * 4, k_pitch, rr0, rows0, K_BASE);
                gather(v_b + (int64_t)(h + 1) * vs.h * 4, v_pitch, rr0, rows0, V_BASE);
                if (h + 2 < H) fetch_rows(h + 2);
            }
        }

        // ---- d_q chunk (8 tokens x 32 channels), p and dS rows (8 tokens x 48 slots) -------------------------------
        if (i == 0) {
            reinterpret_cast<float*>(stage + S2_BASE)[t] = ds_b;   // (the dP area is free)
        }
        {
            float* pw = reinterpret_cast<float*>(stage + PW_BASE) + t * kM + i;
            float* dw = reinterpret_cast<float*>(stage + PW_BASE + PW_BYTES) + t * kM + i;
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                pw[8 * r] = p_all[r];
                dw[8 * r] = ds_all[r];
            }
        }
        lds_sync();
        if (kq < 2) {
            const F32x4 dsb = *reinterpret_cast<const F32x4*>(stage + S2_BASE + 16 * kq);
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
                const float bkc = blank_k[hh * kC + 16 * cb + r16];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    reinterpret_cast<float*>(stage + O_BASE)[(4 * kq + e) * kC + 16 * cb + r16] = (acc[cb][e] + dsb[e] * bkc) * scale;
                }
            }
        }
        lds_sync();
        if (g_sub < nt) {
            const Piece o = *reinterpret_cast<const Piece*>(stage + O_BASE + lane * 16);
            char* dst = reinterpret_cast<char*>(d_q + (int64_t)b * dqs.b + (int64_t)hh * dqs.h + (int64_t)(i0 + g_sub) * dqs.n);
            store_streaming(reinterpret_cast<Piece*>(dst + g_pos * 16), o);
        }
        {
            // the tile's rows of p and dS are contiguous: nt * 192 bytes each
            const int64_t row0 = (((int64_t)b * H_all + hh) * N + i0) * kM;
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                const int piece = lane + kWave * z;
                if (piece < nt * (kM * 4 / 16)) {
                    store_streaming(reinterpret_cast<Piece*>(reinterpret_cast<char*>(probs + row0) + piece * 16),
                                    *reinterpret_cast<const Piece*>(stage + PW_BASE + piece * 16));
                    store_streaming(reinterpret_cast<Piece*>(reinterpret_cast<char*>(d_logit + row0) + piece * 16),
                                    *reinterpret_cast<const Piece*>(stage + PW_BASE + PW_BYTES + piece * 16));
                }
            }
            if (i == 0 && t < nt) {
                const int64_t cell = ((int64_t)b * H_all + hh) * N + i0 + t;
                p_blank[cell] = p_b;
                ds_blank[cell] = ds_b;
            }
        }
        lds_sync();   // the staging areas have been read before the next head writes them
    }
}

}  // namespace

int launch_cluster_attention_backward_f32(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                          clusten_strides vs, const void* d_out, clusten_strides gs, const void* out,
                                          clusten_strides os, const float* lse, const int32_t* cluster_idx,
                                          const void* table, const int64_t* pe_idx, const int64_t* mask,
                                          const float* blank_k, const float* blank_v, void* d_q, clusten_strides dqs,
                                          void* probs, void* d_logit, float* p_blank, float* ds_blank, float scale,
                                          int lists_shared, const void* plan, const clusten_attn_shape& s,
                                          hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int groups = head_groups_for(total, s.H);
    hipLaunchKernelGGL(cluster_attention_bwd_f32_kernel, dim3(xcd_grid(total * groups)), dim3(kWave), 0, stream,
                       static_cast<const float*>(q), qs, static_cast<const float*>(k), ks, static_cast<const float*>(v), vs,
                       static_cast<const float*>(d_out), gs, static_cast<const float*>(out), os, lse, cluster_idx,
                       static_cast<const float*>(table), pe_idx, mask, blank_k, blank_v, static_cast<float*>(d_q), dqs,
                       static_cast<float*>(probs), static_cast<float*>(d_logit), p_blank, ds_blank, s.H, s.N, scale,
                       tiles_per_batch, total, lists_shared, groups, static_cast<const char*>(plan));
    return launch_status();
}

}  // namespace clusten
