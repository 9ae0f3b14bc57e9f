// cluster_attention_backward: the query-side half of the backward of cluster_attention (cluster_attention.hip), in
// one kernel, with the probabilities recomputed from the saved logarithm of each softmax's denominator.
//
// With  x[t,j] = scale * q[t].k[row(t,j)] + bias[t,j] - 100 * (1 - mask[t,j]),  p = exp(x - lse),  p_b = exp(x_b - lse)
// (x_b = scale * q[t].blank_k), and  delta[t] = sum_c d_out[t,c] * out[t,c]  (= sum_j p[t,j] dP[t,j] + p_b[t] dP_b[t]: the
// kernel forms it that way, without the rounding of `out` to 16 bits - inside its one pass, or in a sweep of its own
// ahead of the passes for a tile that needs several) :
//   dP[t,j]   = d_out[t] . v[row(t,j)]              dP_b[t]  = d_out[t] . blank_v
//   dS[t,j]   = p[t,j] * (dP[t,j] - delta[t])       dS_b[t]  = p_b[t] * (dP_b[t] - delta[t])
//   d_q[t]    = scale * (sum_j dS[t,j] * k[row(t,j)] + dS_b[t] * blank_k)
// It writes d_q, the probabilities p and the logit gradients dS as (B,H,N,48) tensors of the storage type, and p_b and
// dS_b as fp32 (B,H,N).  What is left of the backward are sums the library already has kernels for:
//   d_v = scatter of p * d_out,  d_k = scale * scatter of dS * q   (clusten_scatter_rows_by_cluster, no atomics),
//   d_table = clusten_bias_table_grad(dS),  d_blank_k = scale * sum dS_b * q,  d_blank_v = sum p_b * d_out.
// This is the backward of models/aff_transformer.py:120-155 (CLUSTENQKFunction, the tensor expressions between the two
// operators and CLUSTENAVFunction; kernels clusten/src/clustenqk_cuda_kernel.cu:51-132, clustenav_cuda_kernel.cu:51-127)
// with the (B,H,N,M) tensors written once each instead of being read and written by five kernels.
//
// The structure is the forward kernel's: one wave per cluster of 8 tokens walking the heads, the tile's distinct
// clusters numbered once (or read from the plan), their K and V rows in LDS by LDS-direct loads, 12 distinct clusters a
// pass.  Per pass: S = K q^T and dP = V d_out^T are six 16x16x32 matrix instructions each; every lane picks the scores
// and dP of its own slots, forms p and dS; dS re-indexed by distinct cluster (as the forward does with p) times the K
// rows is the query gradient, with the K operand read by `ds_read_b64_tr_b16` from the same row-major rows.
// 16-bit data (fp16 / bf16), head dim 32, M = 48; fp32 data goes to cluster_attention_bwd_f32.hip.
#include "cluster_attention_plan.hpp"

namespace clusten {

int launch_cluster_attention_backward_f32(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                          clusten_strides vs, const void* d_out, clusten_strides gs, const void* out,
                                          clusten_strides os, const float* lse, const int32_t* cluster_idx,
                                          const void* table, const int64_t* pe_idx, const int64_t* mask,
                                          const float* blank_k, const float* blank_v, void* d_q, clusten_strides dqs,
                                          void* probs, void* d_logit, float* p_blank, float* ds_blank, float scale,
                                          int lists_shared, const void* plan, const clusten_attn_shape& s,
                                          hipStream_t stream);   // cluster_attention_bwd_f32.hip

namespace {

using namespace ca;

constexpr int kRB = kC * 2;       // bytes per row
constexpr int kPassRuns = 12;     // distinct clusters per pass
constexpr int kPassRows = 8 * kPassRuns;
constexpr int kBlocks = kPassRows / 16;
constexpr int kSteps = kPassRows / 32;
constexpr int kAccesses = kPassRows / 16;
constexpr int kSRow = kPassRows + 4;   // floats per token row of a score matrix
constexpr int kPRow = kPassRows + 8;   // 16-bit elements per token row of the re-indexed logit gradients

constexpr int K_BASE = 0;
constexpr int V_BASE = K_BASE + kPassRows * kRB;
constexpr int S_BASE = V_BASE + kPassRows * kRB;           // scores; later the re-indexed logit gradients
constexpr int S_BYTES = kTileTokens * kSRow * 4;
constexpr int S2_BASE = S_BASE + S_BYTES;                  // dP
constexpr int D_BASE = S_BASE;
constexpr int D_BYTES = kTileTokens * kPRow * 2;
constexpr int Q_BASE = S2_BASE + S_BYTES;                  // q rows of two heads (slot h % 2)
constexpr int Q_SLOT = kTileTokens * kRB;
constexpr int G_BASE = Q_BASE + 2 * Q_SLOT;                // d_out rows of two heads
constexpr int O_BASE = G_BASE + 2 * Q_SLOT;                // d_q chunk of a head
constexpr int PW_BASE = O_BASE + kTileTokens * kRB;        // p rows of a head (8 x 48), then its dS rows
constexpr int PW_BYTES = kTileTokens * kM * 2;
constexpr int UL_BASE = PW_BASE + 2 * PW_BYTES;
constexpr int LDS_BYTES = UL_BASE + kTileTokens * kR * 4;
static_assert(D_BYTES > 1024 && D_BYTES <= 2048 && D_BYTES <= S_BYTES, "the logit gradients fit the score area");
static_assert(S_BASE % 16 == 0 && S2_BASE % 16 == 0 && Q_BASE % 16 == 0 && PW_BASE % 16 == 0, "aligned areas");

template <typename T>
__global__ __launch_bounds__(kWave) void cluster_attention_bwd_kernel(
    const T* __restrict__ q, clusten_strides qs, const T* __restrict__ k, clusten_strides ks, const T* __restrict__ v,
    clusten_strides vs, const T* __restrict__ d_out, clusten_strides gs, const T* __restrict__ out, clusten_strides os,
    const float* __restrict__ lse, const int32_t* __restrict__ cluster_idx, const T* __restrict__ table,
    const int64_t* __restrict__ pe_idx, const int64_t* __restrict__ mask, const float* __restrict__ blank_k,
    const float* __restrict__ blank_v, T* __restrict__ d_q, clusten_strides dqs, T* __restrict__ probs,
    T* __restrict__ d_logit, float* __restrict__ p_blank, float* __restrict__ ds_blank, int H_all, int N, float scale,
    int tiles_per_batch, int total_tiles, int lists_shared, int head_groups, const char* __restrict__ plan) {
    typedef short S4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) S4* LdsS4;
    typedef VecIO<T, 4> Quad4;

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
    const int g_sub = lane >> 2, g_pos = lane & 3; // gather side: row of a 16-row access, 16-byte piece of the row
    const int t = lane >> 3, i = lane & 7;         // softmax side: token of the tile, member of each cluster
    const int tc = min(t, nt - 1);
    const int64_t list_b = lists_shared ? 0 : b;
    const int64_t tok = list_b * N + i0 + tc;

    // q and d_out rows of head h -> slot h % 2 (lanes 0..31: token lane / 4, piece lane % 4)
    const char* q_tile = reinterpret_cast<const char*>(q + (int64_t)b * qs.b + (int64_t)h0 * qs.h + (int64_t)i0 * qs.n);
    const char* g_tile = reinterpret_cast<const char*>(d_out + (int64_t)b * gs.b + (int64_t)h0 * gs.h + (int64_t)i0 * gs.n);
    const int row8 = min(g_sub & 7, nt - 1);
    const uint32_t q_off = (uint32_t)row8 * (uint32_t)qs.n * 2 + (uint32_t)g_pos * 16;
    const uint32_t g_off = (uint32_t)row8 * (uint32_t)gs.n * 2 + (uint32_t)g_pos * 16;
    auto fetch_rows = [&](int h) {
        if (lane < 32) {
            CLUSTEN_LDS_DMA16(q_tile + (int64_t)h * qs.h * 2 + lane_offset(q_off), stage + Q_BASE + (h & 1) * Q_SLOT);
            CLUSTEN_LDS_DMA16(g_tile + (int64_t)h * gs.h * 2 + lane_offset(g_off), stage + G_BASE + (h & 1) * Q_SLOT);
        }
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
    const int passes = (U + kPassRuns - 1) / kPassRuns;
    const uint32_t k_pitch = (uint32_t)ks.n * 2, v_pitch = (uint32_t)vs.n * 2;
    const char* k_b = reinterpret_cast<const char*>(k + (int64_t)b * ks.b + (int64_t)h0 * ks.h);
    const char* v_b = reinterpret_cast<const char*>(v + (int64_t)b * vs.b + (int64_t)h0 * vs.h);

    auto pass_rows = [&](int pass, uint32_t (&rr)[kAccesses]) {
#pragma unroll
        for (int a = 0; a < kAccesses; ++a) {
            const int urow = a * 16 + g_sub;
            const int c = ulist[min(pass * kPassRuns + (urow >> 3), U - 1)];
            const int row = c * 8 + (urow & 7);
            rr[a] = (unsigned)row < (unsigned)N ? (uint32_t)row : 0u;
        }
    };
    // K and V rows together, access by access: when k and v are the two halves of one projection output a K row and its V
    // row share a 128-byte line, and the V access finds in the L1 what the K access just asked for
    auto gather_both = [&](const char* k_bh, const char* v_bh, const uint32_t (&rr)[kAccesses], int rows_here) {
#pragma unroll
        for (int a = 0; a < kAccesses; ++a) {
            if ((a & ~1) * 16 < rows_here) {
                CLUSTEN_LDS_DMA16(k_bh + lane_offset(rr[a] * k_pitch + (uint32_t)g_pos * 16), stage + K_BASE + a * 1024);
                CLUSTEN_LDS_DMA16(v_bh + lane_offset(rr[a] * v_pitch + (uint32_t)g_pos * 16), stage + V_BASE + a * 1024);
            }
        }
    };
    uint32_t rr0[kAccesses];
    pass_rows(0, rr0);
    const int rows0 = min(kPassRows, total_rows);
    gather_both(k_b, v_b, rr0, rows0);

    for (int h = 0; h < H; ++h) {
        const int hh = h0 + h;
        const char* k_bh = k_b + (int64_t)h * ks.h * 2;
        const char* v_bh = v_b + (int64_t)h * vs.h * 2;
        const char* q_lds = stage + Q_BASE + (h & 1) * Q_SLOT;
        const char* g_lds = stage + G_BASE + (h & 1) * Q_SLOT;

        // small per-head operands of the lane's token, requested before the wait for the rows
        float bias[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t cell = lane_offset(((uint32_t)(pe[r] & 0x7fffffff) * (uint32_t)H_all + (uint32_t)hh) * 2);
            bias[r] = to_acc(*reinterpret_cast<const T*>(reinterpret_cast<const char*>(table) + cell)) +
                      (pe[r] < 0 ? -100.f : 0.f);
        }
        const float4 bk = *reinterpret_cast<const float4*>(blank_k + hh * kC + 4 * i);
        const float4 bv4 = *reinterpret_cast<const float4*>(blank_v + hh * kC + 4 * i);
        const float lse_t = lse[((int64_t)b * H_all + hh) * N + i0 + tc];
        const typename Quad4::raw o_raw = *reinterpret_cast<const typename Quad4::raw*>(
            out + (int64_t)b * os.b + (int64_t)hh * os.h + (int64_t)(i0 + tc) * os.n + 4 * i);

        lds_sync_vm<0>();   // the rows of this head's first pass, its q and d_out rows, the operands above

        // per token: delta = d_out . out, the blank token's logit, probability and logit gradient.  (delta also equals
        // sum_j p_j dP_j + p_b dP_b and is replaced by that sum below: the rounding of `out` to 16 bits does not enter.)
        float delta, p_b, ds_b, dpb_t;
        {
            float o4[4], g4[4], q4[4];
            Quad4::unpack(o_raw, o4);
            Quad4::unpack(*reinterpret_cast<const typename Quad4::raw*>(g_lds + t * kRB + 8 * i), g4);
            Quad4::unpack(*reinterpret_cast<const typename Quad4::raw*>(q_lds + t * kRB + 8 * i), q4);
            delta = oct_sum(g4[0] * o4[0] + g4[1] * o4[1] + g4[2] * o4[2] + g4[3] * o4[3]);
            const float dpb = oct_sum(g4[0] * bv4.x + g4[1] * bv4.y + g4[2] * bv4.z + g4[3] * bv4.w);
            const float bl = oct_sum(q4[0] * bk.x + q4[1] * bk.y + q4[2] * bk.z + q4[3] * bk.w) * scale;
            p_b = __expf(bl - lse_t);
            ds_b = p_b * (dpb - delta);
            dpb_t = dpb;
        }

        if (passes > 1) {
            // A tile whose clusters take several passes: a first sweep over the passes forms only S and dP and adds up
            // p * dP, so that delta is the same fp32 sum a one-pass tile uses and does not depend on the 16-bit rounding
            // of `out` either (such tiles are rare on lists like the model's: more than 12 distinct clusters among the
            // 48 a tile names; they pay their rows twice).
            float pdp = 0.f;
            for (int pass = 0; pass < passes; ++pass) {
                const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
                if (pass > 0) lds_sync_vm<0>();  // the K and V rows of this pass are in LDS
                const Piece qraw = *reinterpret_cast<const Piece*>(q_lds + (r16 & 7) * kRB + kq * 16);
                const Piece graw = *reinterpret_cast<const Piece*>(g_lds + (r16 & 7) * kRB + kq * 16);
#pragma unroll
                for (int blk = 0; blk < kBlocks; ++blk) {
                    if (blk * 16 < rows_here) {
                        const Piece kraw = *reinterpret_cast<const Piece*>(stage + K_BASE + (blk * 16 + r16) * kRB + kq * 16);
                        const Piece vraw = *reinterpret_cast<const Piece*>(stage + V_BASE + (blk * 16 + r16) * kRB + kq * 16);
                        const F32x4 s = tile_mfma<T>(kraw, qraw, F32x4{0.f, 0.f, 0.f, 0.f});
                        const F32x4 d = tile_mfma<T>(vraw, graw, F32x4{0.f, 0.f, 0.f, 0.f});
                        if (r16 < kTileTokens) {
                            *reinterpret_cast<F32x4*>(stage + S_BASE + (r16 * kSRow + 16 * blk + 4 * kq) * 4) = s;
                            *reinterpret_cast<F32x4*>(stage + S2_BASE + (r16 * kSRow + 16 * blk + 4 * kq) * 4) = d;
                        }
                    }
                }
                lds_sync();
#pragma unroll
                for (int r = 0; r < kR; ++r) {
                    const unsigned u = (unsigned)(us[r] - pass * kPassRuns);
                    const int cell = (t * kSRow + (int)min(u, (unsigned)kPassRuns - 1) * 8 + i) * 4;
                    const float sc = *reinterpret_cast<const float*>(stage + S_BASE + cell);
                    const float dp = *reinterpret_cast<const float*>(stage + S2_BASE + cell);
                    pdp += u < (unsigned)kPassRuns ? __expf(sc * scale + bias[r] - lse_t) * dp : 0.f;
                }
                lds_sync();  // rows and scores have been read: the next pass's rows, or the first pass's again
                const int nxt = pass + 1 < passes ? pass + 1 : 0;
                uint32_t rr[kAccesses];
                pass_rows(nxt, rr);
                const int next_rows = min(kPassRows, total_rows - nxt * kPassRows);
                gather_both(k_bh, v_bh, rr, next_rows);
            }
            delta = oct_sum(pdp) + p_b * dpb_t;
            ds_b = p_b * (dpb_t - delta);
            lds_sync_vm<0>();   // the rows of the first pass are back
        }

        float p_all[kR], ds_all[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) p_all[r] = ds_all[r] = 0.f;
        F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
            if (pass > 0) lds_sync_vm<0>();  // the K and V rows of this pass are in LDS
            // ---- S = K q^T and dP = V d_out^T --------------------------------------------------------------
            {
                const Piece qraw = *reinterpret_cast<const Piece*>(q_lds + (r16 & 7) * kRB + kq * 16);
                const Piece graw = *reinterpret_cast<const Piece*>(g_lds + (r16 & 7) * kRB + kq * 16);
#pragma unroll
                for (int blk = 0; blk < kBlocks; ++blk) {
                    if (blk * 16 < rows_here) {
                        const Piece kraw = *reinterpret_cast<const Piece*>(stage + K_BASE + (blk * 16 + r16) * kRB + kq * 16);
                        const Piece vraw = *reinterpret_cast<const Piece*>(stage + V_BASE + (blk * 16 + r16) * kRB + kq * 16);
                        const F32x4 s = tile_mfma<T>(kraw, qraw, F32x4{0.f, 0.f, 0.f, 0.f});
                        const F32x4 d = tile_mfma<T>(vraw, graw, F32x4{0.f, 0.f, 0.f, 0.f});
                        // lane (r16, kq): pass rows 16*blk + 4*kq .. +3 of token r16
                        if (r16 < kTileTokens) {
                            *reinterpret_cast<F32x4*>(stage + S_BASE + (r16 * kSRow + 16 * blk + 4 * kq) * 4) = s;
                            *reinterpret_cast<F32x4*>(stage + S2_BASE + (r16 * kSRow + 16 * blk + 4 * kq) * 4) = d;
                        }
                    }
                }
            }
            lds_sync();
            // ---- the lane's own slots: p and dS ---------------------------------------------------------------
            float ds_pass[kR], pr_[kR], dp_[kR];
            bool in_[kR];
            float pdp = 0.f;
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const unsigned u = (unsigned)(us[r] - pass * kPassRuns);
                in_[r] = u < (unsigned)kPassRuns;
                const int cell = (t * kSRow + (int)min(u, (unsigned)kPassRuns - 1) * 8 + i) * 4;
                const float sc = *reinterpret_cast<const float*>(stage + S_BASE + cell);
                dp_[r] = *reinterpret_cast<const float*>(stage + S2_BASE + cell);
                pr_[r] = __expf(sc * scale + bias[r] - lse_t);
                pdp += in_[r] ? pr_[r] * dp_[r] : 0.f;
            }
            if (passes == 1) {
                delta = oct_sum(pdp) + p_b * dpb_t;
                ds_b = p_b * (dpb_t - delta);
            }
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const float ds = pr_[r] * (dp_[r] - delta);
                p_all[r] = in_[r] ? pr_[r] : p_all[r];
                ds_all[r] = in_[r] ? ds : ds_all[r];
                ds_pass[r] = in_[r] ? ds : 0.f;
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
                T* drow = reinterpret_cast<T*>(stage + D_BASE) + t * kPRow + i;
#pragma unroll
                for (int r = 0; r < kR; ++r) {
                    const unsigned u = ((repeats >> r) & 1) ? ~0u : (unsigned)(us[r] - pass * kPassRuns);
                    drow[min(u, (unsigned)kPassRuns) * 8] = from_acc<T>(ds_pass[r]);
                }
            }
            lds_sync();
            // ---- d_q += dS_pass (8 x 96) * K_pass (96 x 32) ---------------------------------------------------
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                if (s * 32 < rows_here) {
                    const Piece a = *reinterpret_cast<const Piece*>(stage + D_BASE + ((r16 & 7) * kPRow + 32 * s + 8 * kq) * 2);
                    const char* col = stage + K_BASE + (32 * s + 8 * kq + (r16 >> 2)) * kRB + (r16 & 3) * 8;
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        const S4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32));
                        const S4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32 + 4 * kRB));
                        const U32x2 lo = __builtin_bit_cast(U32x2, b0), hi = __builtin_bit_cast(U32x2, b1);
                        acc[cb] = tile_mfma<T>(a, Piece{lo[0], lo[1], hi[0], hi[1]}, acc[cb]);
                    }
                }
            }
            lds_sync();  // the K and V rows and the logit gradients have been read
            if (pass + 1 < passes) {
                uint32_t rr[kAccesses];
                pass_rows(pass + 1, rr);
                const int next_rows = min(kPassRows, total_rows - (pass + 1) * kPassRows);
                gather_both(k_bh, v_bh, rr, next_rows);
            } else if (h + 1 < H) {
                gather_both(k_b + (int64_t)(h + 1) * ks.h * 2, v_b + (int64_t)(h + 1) * vs.h * 2, rr0, rows0);
                if (h + 2 < H) fetch_rows(h + 2);
            }
        }

        // ---- d_q chunk (8 tokens x 32 channels), p and dS rows (8 tokens x 48 slots) -------------------------------
        if (i == 0) {
            reinterpret_cast<float*>(stage + S2_BASE)[t] = ds_b;   // (the dP area is free)
        }
        {
            T* pw = reinterpret_cast<T*>(stage + PW_BASE) + t * kM + i;
            T* dw = reinterpret_cast<T*>(stage + PW_BASE + PW_BYTES) + t * kM + i;
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                pw[8 * r] = from_acc<T>(p_all[r]);
                dw[8 * r] = from_acc<T>(ds_all[r]);
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
                    reinterpret_cast<T*>(stage + O_BASE)[(4 * kq + e) * kC + 16 * cb + r16] =
                        from_acc<T>((acc[cb][e] + dsb[e] * bkc) * scale);
                }
            }
        }
        lds_sync();
        if (lane < 32 && g_sub < nt) {
            const Piece o = *reinterpret_cast<const Piece*>(stage + O_BASE + lane * 16);
            char* dst = reinterpret_cast<char*>(d_q + (int64_t)b * dqs.b + (int64_t)hh * dqs.h + (int64_t)(i0 + g_sub) * dqs.n);
            store_streaming(reinterpret_cast<Piece*>(dst + g_pos * 16), o);
        }
        {
            // the tile's rows of p and dS are contiguous: nt * 96 bytes each
            const int64_t row0 = (((int64_t)b * H_all + hh) * N + i0) * kM;
            if (lane < nt * (kM * 2 / 16)) {
                store_streaming(reinterpret_cast<Piece*>(reinterpret_cast<char*>(probs + row0) + lane * 16),
                                *reinterpret_cast<const Piece*>(stage + PW_BASE + lane * 16));
                store_streaming(reinterpret_cast<Piece*>(reinterpret_cast<char*>(d_logit + row0) + lane * 16),
                                *reinterpret_cast<const Piece*>(stage + PW_BASE + PW_BYTES + lane * 16));
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

template <typename T>
int launch_typed(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v, clusten_strides vs,
                 const void* d_out, clusten_strides gs, const void* out, clusten_strides os, const float* lse,
                 const int32_t* cluster_idx, const void* table, const int64_t* pe_idx, const int64_t* mask,
                 const float* blank_k, const float* blank_v, void* d_q, clusten_strides dqs, void* probs, void* d_logit,
                 float* p_blank, float* ds_blank, float scale, int lists_shared, const void* plan,
                 const clusten_attn_shape& s, hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int groups = head_groups_for(total, s.H);
    hipLaunchKernelGGL((cluster_attention_bwd_kernel<T>), dim3(xcd_grid(total * groups)), dim3(kWave), 0, stream,
                       static_cast<const T*>(q), qs, static_cast<const T*>(k), ks, static_cast<const T*>(v), vs,
                       static_cast<const T*>(d_out), gs, static_cast<const T*>(out), os, lse, cluster_idx,
                       static_cast<const T*>(table), pe_idx, mask, blank_k, blank_v, static_cast<T*>(d_q), dqs,
                       static_cast<T*>(probs), static_cast<T*>(d_logit), p_blank, ds_blank, s.H, s.N, scale,
                       tiles_per_batch, total, lists_shared, groups, static_cast<const char*>(plan));
    return launch_status();
}

}  // namespace

int launch_cluster_attention_backward(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                      clusten_strides vs, const void* d_out, clusten_strides gs, const void* out,
                                      clusten_strides os, const float* lse, const int32_t* cluster_idx, const void* table,
                                      const int64_t* pe_idx, const int64_t* mask, const float* blank_k,
                                      const float* blank_v, void* d_q, clusten_strides dqs, void* probs, void* d_logit,
                                      float* p_blank, float* ds_blank, float scale, int lists_shared, const void* plan,
                                      clusten_attn_shape s, int dtype, hipStream_t stream) {
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16 && dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (s.C != kC || s.M != kM) return CLUSTEN_ERR_BAD_DIMS;
    const int es = dtype == CLUSTEN_F32 ? 4 : 2;
    const bool ok = rows_aligned16(q, qs, es) && rows_aligned16(k, ks, es) && rows_aligned16(v, vs, es) &&
                    rows_aligned16(d_out, gs, es) && rows_aligned16(out, os, es) && rows_aligned16(d_q, dqs, es) &&
                    aligned16(probs) && aligned16(d_logit) && aligned16(blank_k) && aligned16(blank_v) &&
                    slice_fits_int32(ks, s.H, s.N, s.C) && slice_fits_int32(vs, s.H, s.N, s.C) &&
                    slice_fits_int32(qs, s.H, s.N, s.C) && slice_fits_int32(gs, s.H, s.N, s.C);
    if (!ok) return CLUSTEN_ERR_UNALIGNED;
    if (dtype == CLUSTEN_F32) {
        return launch_cluster_attention_backward_f32(q, qs, k, ks, v, vs, d_out, gs, out, os, lse, cluster_idx, table, pe_idx,
                                                     mask, blank_k, blank_v, d_q, dqs, probs, d_logit, p_blank, ds_blank,
                                                     scale, lists_shared, plan, s, stream);
    }
    if (dtype == CLUSTEN_F16) {
        return launch_typed<f16_t>(q, qs, k, ks, v, vs, d_out, gs, out, os, lse, cluster_idx, table, pe_idx, mask, blank_k,
                                   blank_v, d_q, dqs, probs, d_logit, p_blank, ds_blank, scale, lists_shared, plan, s, stream);
    }
    return launch_typed<bf16_t>(q, qs, k, ks, v, vs, d_out, gs, out, os, lse, cluster_idx, table, pe_idx, mask, blank_k,
                                blank_v, d_q, dqs, probs, d_logit, p_blank, ds_blank, scale, lists_shared, plan, s, stream);
}

}  // namespace clusten
