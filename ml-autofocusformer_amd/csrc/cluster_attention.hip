// cluster_attention: local attention of a cluster-ordered token sequence in one kernel (inference).
//
//   logit[b,h,i,j] = scale * sum_c q[b,h,i,c] * k[b,h,row(i,j),c] + table[pe_idx[b,i,j], h] - 100 * (1 - mask[b,i,j])
//   blank[b,h,i]   = scale * sum_c q[b,h,i,c] * blank_k[h,c]
//   p[b,h,i,:], p_blank[b,h,i] = softmax over the M neighbours and the blank token
//   out[b,h,i,c]   = sum_j p[b,h,i,j] * v[b,h,row(i,j),c] + p_blank[b,h,i] * blank_v[h,c]
//   row(i,j)       = 8 * cluster_idx[b,i,j/8] + j%8   (row 0 where that is not in [0,N))
//
// This is CLUSTENQKFunction, the tensor expressions between the two operators and CLUSTENAVFunction of the
// reference model (models/aff_transformer.py:120-155; kernels clusten/src/clustenqk_cuda_kernel.cu:18-49 and
// clusten/src/clustenav_cuda_kernel.cu:18-49) with the (B,H,N,M) logits and probabilities never leaving the
// chip.  16-bit data (fp16 / bf16), head dim 32, M = 48 (six clusters of 8 per token): the shape of every
// attention layer of the shipped models under mixed precision.
//
// One wave owns 8 consecutive tokens (one cluster) and walks the heads.  The tile's 48 cluster numbers are
// numbered by distinct value (`U` of them, typically 8-14: neighbouring tokens choose among the same clusters);
// per head the rows of 8 distinct clusters at a time (a pass: 64 rows) travel to LDS by LDS-direct loads, and
//   QK  S[row][token] = K_pass (64 x 32) * q^T (32 x 8): four 16x16x32 matrix instructions; each token picks its own
//       slots from the score matrix in LDS;
//   softmax: lane (t = lane / 8, i = lane % 8) holds slots 8*r + i, r < 6, of token t; maxima and sums go across the
//       8 lanes of a token;
//   AV  out (8 x 32) = P_pass (8 x 64) * V_pass (64 x 32): the probabilities are written to LDS re-indexed by
//       distinct cluster (zero where a token does not hold the cluster; a cluster held twice adds up), rounded to
//       the storage type; the V operand needs consecutive rows of one channel per lane, which
//       `ds_read_b64_tr_b16` delivers from the row-major rows.
// The next pass's rows (the V rows during the softmax, the next head's K rows during the last AV pass) are
// requested as soon as the current operands are in registers.
//
// A token whose probabilities are zero for a cluster still multiplies that cluster's V rows by zero: non-finite
// values in rows a token does not list reach its output as NaN (the unfused operators share this on their
// union path).
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kC = 32;            // head dim
constexpr int kR = 6;             // clusters per token
constexpr int kM = 8 * kR;        // neighbours per token
constexpr int kRB = kC * 2;       // bytes per row
constexpr int kPassRuns = 8;      // distinct clusters per pass
constexpr int kPassRows = 64;
constexpr int kSRow = kPassRows + 4;   // floats per token row of the score matrix
constexpr int kPRow = kPassRows + 8;   // 16-bit elements per token row of the re-indexed probabilities

constexpr int K_BASE = 0;                                  // 64 K rows
constexpr int V_BASE = K_BASE + kPassRows * kRB;           // 64 V rows
constexpr int S_BASE = V_BASE + kPassRows * kRB;           // scores of a pass
constexpr int P_BASE = S_BASE + kTileTokens * kSRow * 4;   // probabilities of a pass; reused for the output chunk
constexpr int P_BYTES = kTileTokens * kPRow * 2;
constexpr int Q_BASE = P_BASE + P_BYTES;                   // q rows of two heads (slot h % 2)
constexpr int Q_SLOT = kTileTokens * kRB;
constexpr int UL_BASE = Q_BASE + 2 * Q_SLOT;               // cluster number of each distinct cluster
constexpr int PB_BASE = UL_BASE + kTileTokens * kR * 4;    // blank-token probability per token
constexpr int LDS_BYTES = PB_BASE + kTileTokens * 4;
static_assert(P_BYTES % 16 == 0 && P_BASE % 16 == 0 && Q_BASE % 16 == 0, "16-byte LDS accesses");
static_assert(P_BYTES >= kTileTokens * kRB, "the output chunk fits the probability area");

__device__ __forceinline__ float oct_max(float v) {
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}
__device__ __forceinline__ float oct_sum(float v) {
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) v += __shfl_xor(v, m);
    return v;
}

template <typename T>
__global__ __launch_bounds__(kWave) void cluster_attention_kernel(
    const T* __restrict__ q, clusten_strides qs, const T* __restrict__ k, clusten_strides ks, const T* __restrict__ v,
    clusten_strides vs, const int32_t* __restrict__ cluster_idx, const T* __restrict__ table,
    const int64_t* __restrict__ pe_idx, const int64_t* __restrict__ mask, const float* __restrict__ blank_k,
    const float* __restrict__ blank_v, T* __restrict__ out, clusten_strides os, int H, int N, float scale,
    int tiles_per_batch, int total_tiles) {
    typedef short S4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) S4* LdsS4;

    __shared__ __attribute__((aligned(1024))) char stage[LDS_BYTES];

    const int tile = xcd_tile(blockIdx.x, total_tiles);
    if (tile < 0) return;
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
    const int64_t tok = (int64_t)b * N + i0 + min(t, nt - 1);

    // q rows of head h -> slot h % 2 (lanes 0..31: token lane / 4, piece lane % 4)
    const char* q_tile = reinterpret_cast<const char*>(q + (int64_t)b * qs.b + (int64_t)i0 * qs.n);
    const uint32_t q_off = (uint32_t)min(g_sub, nt - 1) * (uint32_t)qs.n * 2 + (uint32_t)g_pos * 16;
    auto fetch_q = [&](int h) {
        if (lane < 32) {
            CLUSTEN_LDS_DMA16(q_tile + (int64_t)h * qs.h * 2 + q_off, stage + Q_BASE + (h & 1) * Q_SLOT);
        }
    };
    fetch_q(0);
    if (H > 1) fetch_q(1);

    // per-slot inputs the heads share
    int pe[kR];
    float off[kR];
#pragma unroll
    for (int r = 0; r < kR; ++r) {
        pe[r] = (int)pe_idx[tok * kM + 8 * r + i];
        off[r] = mask ? (float)(1 - mask[tok * kM + 8 * r + i]) * -100.f : 0.f;
    }

    // number the distinct cluster numbers of the tile in order of first appearance: lane rho < 48 owns run rho =
    // token * 6 + run
    const int rho = min(lane, kTileTokens * kR - 1);
    const int cid = cluster_idx[((int64_t)b * N + i0 + min(rho / kR, nt - 1)) * kR + rho % kR];
    uint64_t remaining = (1ull << (kTileTokens * kR)) - 1;
    int uslot = 0, U = 0;
    bool first = false;
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
    int* ulist = reinterpret_cast<int*>(stage + UL_BASE);
    if (first) ulist[uslot] = cid;
    int us[kR];  // distinct-cluster number of this lane's token's runs
#pragma unroll
    for (int r = 0; r < kR; ++r) us[r] = __shfl(uslot, t * kR + r);
    __syncthreads();

    const int total_rows = 8 * U;
    const int passes = (U + kPassRuns - 1) / kPassRuns;
    const uint32_t k_pitch = (uint32_t)ks.n * 2, v_pitch = (uint32_t)vs.n * 2;
    const char* k_b = reinterpret_cast<const char*>(k + (int64_t)b * ks.b);
    const char* v_b = reinterpret_cast<const char*>(v + (int64_t)b * vs.b);

    // rows of the distinct clusters 8*pass .. 8*pass+7 of one head -> LDS, 16 rows per access; clusters past the
    // last one repeat it so that every row of a 32-row step holds data
    auto gather = [&](const char* rows_bh, uint32_t pitch, int pass, int lds_base) {
        const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            if ((a & ~1) * 16 < rows_here) {
                const int urow = a * 16 + g_sub;
                const int c = ulist[min(pass * kPassRuns + (urow >> 3), U - 1)];
                const int row = c * 8 + (urow & 7);
                const uint32_t rr = (unsigned)row < (unsigned)N ? (uint32_t)row : 0u;
                CLUSTEN_LDS_DMA16(rows_bh + (rr * pitch + (uint32_t)g_pos * 16), stage + lds_base + a * 1024);
            }
        }
    };

    gather(k_b, k_pitch, 0, K_BASE);

    for (int h = 0; h < H; ++h) {
        const char* k_bh = k_b + (int64_t)h * ks.h * 2;
        const char* v_bh = v_b + (int64_t)h * vs.h * 2;
        const char* q_lds = stage + Q_BASE + (h & 1) * Q_SLOT;

        // ---- scores -------------------------------------------------------------------------------------
        float logit[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) logit[r] = 0.f;
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            __syncthreads();  // the K rows of this pass (and the q rows) are in LDS; the previous pass has picked
            Piece kraw[4];
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                if (blk * 16 < rows_here) {
                    kraw[blk] = *reinterpret_cast<const Piece*>(stage + K_BASE + (blk * 16 + r16) * kRB + kq * 16);
                }
            }
            const Piece qraw = *reinterpret_cast<const Piece*>(q_lds + (r16 & 7) * kRB + kq * 16);
            __syncthreads();  // operands are in registers: the K area is free
            if (pass + 1 < passes) {
                gather(k_bh, k_pitch, pass + 1, K_BASE);
            } else {
                gather(v_bh, v_pitch, 0, V_BASE);
            }
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                if (blk * 16 < rows_here) {
                    const F32x4 d = tile_mfma<T>(kraw[blk], qraw, F32x4{0.f, 0.f, 0.f, 0.f});
                    // lane (r16, kq): pass rows 16*blk + 4*kq .. +3 of token r16
                    if (r16 < kTileTokens) {
                        *reinterpret_cast<F32x4*>(stage + S_BASE + (r16 * kSRow + 16 * blk + 4 * kq) * 4) = d;
                    }
                }
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const int u = us[r] - pass * kPassRuns;
                if (u >= 0 && u < kPassRuns) {
                    logit[r] = *reinterpret_cast<const float*>(stage + S_BASE + (t * kSRow + u * 8 + i) * 4);
                }
            }
        }

        // ---- softmax over the 48 neighbours and the blank token ----------------------------------------------
        float x[kR];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            x[r] = logit[r] * scale + to_acc(table[(int64_t)pe[r] * H + h]) + off[r];
            mx = fmaxf(mx, x[r]);
        }
        float part = 0.f;
        {
            const T* qrow = reinterpret_cast<const T*>(q_lds + t * kRB) + 4 * i;
            const float4 bk = *reinterpret_cast<const float4*>(blank_k + h * kC + 4 * i);
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
        const float inv = 1.f / (oct_sum(sum) + eb);
#pragma unroll
        for (int r = 0; r < kR; ++r) p[r] *= inv;
        if (i == 0) *reinterpret_cast<float*>(stage + PB_BASE + t * 4) = eb * inv;

        // ---- weighted sum of the V rows --------------------------------------------------------------------------
        F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
        for (int pass = 0; pass < passes; ++pass) {
            const int rows_here = min(kPassRows, total_rows - pass * kPassRows);
            __syncthreads();  // the previous pass's (or head's) reads of the probability area are complete
            // probabilities of this pass, re-indexed by distinct cluster: zero, then each lane adds its own
            *reinterpret_cast<Piece*>(stage + P_BASE + lane * 16) = Piece{0u, 0u, 0u, 0u};
            if (lane < (P_BYTES - 1024) / 16) {
                *reinterpret_cast<Piece*>(stage + P_BASE + 1024 + lane * 16) = Piece{0u, 0u, 0u, 0u};
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const int u = us[r] - pass * kPassRuns;
                if (u >= 0 && u < kPassRuns) {
                    T* cell = reinterpret_cast<T*>(stage + P_BASE) + t * kPRow + u * 8 + i;
                    *cell = from_acc<T>(to_acc(*cell) + p[r]);
                }
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            __syncthreads();  // the V rows of this pass are in LDS, the probabilities are written
            Piece a[2];
            S4 bt[2][2][2];  // [step][channel block][rows 0-3 / 4-7 of the lane's 8]
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if (s * 32 < rows_here) {
                    a[s] = *reinterpret_cast<const Piece*>(stage + P_BASE + ((r16 & 7) * kPRow + 32 * s + 8 * kq) * 2);
                    const char* col = stage + V_BASE + (32 * s + 8 * kq + (r16 >> 2)) * kRB + (r16 & 3) * 8;
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        bt[s][cb][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32));
                        bt[s][cb][1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32 + 4 * kRB));
                    }
                }
            }
            __syncthreads();  // operands are in registers: the V area is free
            if (pass + 1 < passes) {
                gather(v_bh, v_pitch, pass + 1, V_BASE);
            } else if (h + 1 < H) {
                gather(k_b + (int64_t)(h + 1) * ks.h * 2, k_pitch, 0, K_BASE);
                if (h + 2 < H) fetch_q(h + 2);
            }
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if (s * 32 < rows_here) {
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        const U32x2 lo = __builtin_bit_cast(U32x2, bt[s][cb][0]);
                        const U32x2 hi = __builtin_bit_cast(U32x2, bt[s][cb][1]);
                        acc[cb] = tile_mfma<T>(a[s], Piece{lo[0], lo[1], hi[0], hi[1]}, acc[cb]);
                    }
                }
            }
        }

        // ---- blank token, output chunk (8 tokens x 32 channels, row-major over the probability area) ---------------
        __syncthreads();
        if (kq < 2) {
            const F32x4 pb = *reinterpret_cast<const F32x4*>(stage + PB_BASE + 16 * kq);
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
                const float bv = blank_v[h * kC + 16 * cb + r16];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    reinterpret_cast<T*>(stage + P_BASE)[(4 * kq + e) * kC + 16 * cb + r16] =
                        from_acc<T>(acc[cb][e] + pb[e] * bv);
                }
            }
        }
        __syncthreads();
        if (lane < 32 && g_sub < nt) {
            const Piece o = *reinterpret_cast<const Piece*>(stage + P_BASE + lane * 16);
            char* dst = reinterpret_cast<char*>(out + (int64_t)b * os.b + (int64_t)h * os.h + (int64_t)(i0 + g_sub) * os.n);
            store_streaming(reinterpret_cast<Piece*>(dst + g_pos * 16), o);
        }
    }
}

template <typename T>
int launch_typed(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                 clusten_strides vs, const int32_t* cluster_idx, const void* table, const int64_t* pe_idx,
                 const int64_t* mask, const float* blank_k, const float* blank_v, void* out, clusten_strides os,
                 float scale, const clusten_attn_shape& s, hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    hipLaunchKernelGGL((cluster_attention_kernel<T>), dim3(xcd_grid(total)), dim3(kWave), 0, stream,
                       static_cast<const T*>(q), qs, static_cast<const T*>(k), ks, static_cast<const T*>(v), vs,
                       cluster_idx, static_cast<const T*>(table), pe_idx, mask, blank_k, blank_v, static_cast<T*>(out),
                       os, s.H, s.N, scale, tiles_per_batch, total);
    return launch_status();
}

}  // namespace

int launch_cluster_attention(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                             clusten_strides vs, const int32_t* cluster_idx, const void* table, const int64_t* pe_idx,
                             const int64_t* mask, const float* blank_k, const float* blank_v, void* out,
                             clusten_strides os, float scale, clusten_attn_shape s, int dtype, hipStream_t stream) {
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (s.C != kC || s.M != kM) return CLUSTEN_ERR_BAD_DIMS;
    const bool ok = rows_aligned16(q, qs, 2) && rows_aligned16(k, ks, 2) && rows_aligned16(v, vs, 2) &&
                    rows_aligned16(out, os, 2) && aligned16(blank_k) && slice_fits_int32(ks, s.H, s.N, s.C) &&
                    slice_fits_int32(vs, s.H, s.N, s.C) && slice_fits_int32(qs, s.H, s.N, s.C);
    if (!ok) return CLUSTEN_ERR_UNALIGNED;
    if (dtype == CLUSTEN_F16) {
        return launch_typed<f16_t>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os, scale,
                                   s, stream);
    }
    return launch_typed<bf16_t>(q, qs, k, ks, v, vs, cluster_idx, table, pe_idx, mask, blank_k, blank_v, out, os, scale, s,
                                stream);
}

}  // namespace clusten
