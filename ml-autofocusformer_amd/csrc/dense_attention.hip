// dense_attention: attention of every token over every token of a short sequence in one kernel (inference).
//
//   logit[b,h,i,j] = scale * sum_c q[b,h,i,c] * k[b,h,j,c] + table[pe_idx[b,i,j], h]          (i, j < N)
//   blank[b,h,i]   = scale * sum_c q[b,h,i,c] * blank_k[h,c]
//   p[b,h,i,:], p_blank[b,h,i] = softmax over the N tokens and the blank token
//   out[b,h,i,c]   = sum_j p[b,h,i,j] * v[b,h,j,c] + p_blank[b,h,i] * blank_v[h,c]
//
// This is the branch the reference model takes in a stage whose neighbourhood size reaches the number of tokens
// (models/aff_transformer.py:108-113, 125-155: two batched matrix products with the position bias, the blank token
// and the softmax between them); the last stage of the shipped models at 224 x 224 has N = 49.  16-bit data
// (fp16 / bf16), head dim 32, N <= 64.  It has no counterpart in the reference's extension modules.
//
// One wave owns one (image, head): the 3 x N rows travel to LDS by LDS-direct loads, the N x N scores are sixteen
// 16x16x32 matrix instructions whose results stay in registers (lane (r16, kq) holds rows 16*bi + 4*kq + j, column
// 16*bj + r16), row maxima and sums go across the 16 lanes of a register row with data-parallel-primitive moves, the
// probabilities are rounded to the storage type and written to LDS, and the N x 32 output is sixteen more matrix
// instructions whose V operand (consecutive rows of one channel per lane) `ds_read_b64_tr_b16` delivers from the
// row-major rows.
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kC = 32;          // head dim
constexpr int kRB = kC * 2;     // bytes per row
constexpr int kNMax = 64;       // tokens
constexpr int kNB = kNMax / 16; // 16-row blocks
constexpr int kPRow = kNMax + 8;  // 16-bit elements per row of the probabilities (the pad spreads the rows over the banks)

constexpr int Q_BASE = 0;                      // q rows; later the output rows
constexpr int O_BASE = Q_BASE;
constexpr int K_BASE = Q_BASE + kNMax * kRB;
constexpr int V_BASE = K_BASE + kNMax * kRB;
constexpr int P_BASE = V_BASE + kNMax * kRB;
constexpr int BL_BASE = P_BASE + kNMax * kPRow * 2;  // blank logit per row
constexpr int LDS_BYTES = BL_BASE + kNMax * 4;
static_assert((kPRow * 2) % 16 == 0 && P_BASE % 16 == 0 && BL_BASE % 16 == 0, "16-byte operand reads");

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// Reductions over the 16 lanes of a register row (lanes 16*kq .. 16*kq+15): neighbours in a quad, the other pair of
// the quad, the mirrored lane of the other quad of the half, the mirrored lane of the other half.
__device__ __forceinline__ float row_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    return fmaxf(v, dpp_move<0x140>(v));
}
__device__ __forceinline__ float row_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    return v + dpp_move<0x140>(v);
}

template <typename T>
__global__ __launch_bounds__(kWave) void dense_attention_kernel(
    const T* __restrict__ q, clusten_strides qs, const T* __restrict__ k, clusten_strides ks, const T* __restrict__ v,
    clusten_strides vs, const T* __restrict__ table, const int64_t* __restrict__ pe_idx,
    const float* __restrict__ blank_k, const float* __restrict__ blank_v, T* __restrict__ out, clusten_strides os, int H,
    int N, float scale) {
    typedef short S4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) S4* LdsS4;

    __shared__ __attribute__((aligned(1024))) char stage[LDS_BYTES];

    const int b = blockIdx.x / H;
    const int h = blockIdx.x - b * H;
    const int lane = threadIdx.x;
    const int r16 = lane & 15;     // matrix side: row of A / column of B and of the result
    const int kq = lane >> 4;      //              k group; rows 4*kq .. 4*kq+3 of the result
    const int g_sub = lane >> 2;   // copy side: row of a 16-row access
    const int g_pos = lane & 3;    //            16-byte piece of the row

    // all 64 rows of each area are filled (rows past the sequence repeat its last row): the probabilities of the
    // columns past the sequence are zero, and zero times the V row they meet must be zero
    {
        const char* q_bh = reinterpret_cast<const char*>(q + (int64_t)b * qs.b + (int64_t)h * qs.h);
        const char* k_bh = reinterpret_cast<const char*>(k + (int64_t)b * ks.b + (int64_t)h * ks.h);
        const char* v_bh = reinterpret_cast<const char*>(v + (int64_t)b * vs.b + (int64_t)h * vs.h);
#pragma unroll
        for (int a = 0; a < kNB; ++a) {
            const uint32_t row = (uint32_t)min(16 * a + g_sub, N - 1);
            CLUSTEN_LDS_DMA16(q_bh + lane_offset(row * (uint32_t)qs.n * 2 + (uint32_t)g_pos * 16), stage + Q_BASE + a * 1024);
            CLUSTEN_LDS_DMA16(k_bh + lane_offset(row * (uint32_t)ks.n * 2 + (uint32_t)g_pos * 16), stage + K_BASE + a * 1024);
            CLUSTEN_LDS_DMA16(v_bh + lane_offset(row * (uint32_t)vs.n * 2 + (uint32_t)g_pos * 16), stage + V_BASE + a * 1024);
        }
    }

    // rows of the bias table: the low words of pe_idx (its values are table rows, far below 2^31)
    const int32_t* pe_lo = reinterpret_cast<const int32_t*>(pe_idx + (int64_t)b * N * N);
    const int col_of[kNB] = {min(r16, N - 1), min(16 + r16, N - 1), min(32 + r16, N - 1), min(48 + r16, N - 1)};
    int pe[kNB][kNB][4];
#pragma unroll
    for (int bi = 0; bi < kNB; ++bi) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = min(16 * bi + 4 * kq + j, N - 1);
#pragma unroll
            for (int bj = 0; bj < kNB; ++bj) pe[bi][bj][j] = pe_lo[2 * (row * N + col_of[bj])];
        }
    }
    lds_sync_vm<0>();  // the rows are in LDS, the table rows in registers

    float bias[kNB][kNB][4];
#pragma unroll
    for (int bi = 0; bi < kNB; ++bi) {
#pragma unroll
        for (int bj = 0; bj < kNB; ++bj) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t cell = lane_offset(((uint32_t)pe[bi][bj][j] * (uint32_t)H + (uint32_t)h) * 2);
                bias[bi][bj][j] = to_acc(*reinterpret_cast<const T*>(reinterpret_cast<const char*>(table) + cell));
            }
        }
    }

    // blank logit of row `lane`
    {
        float part = 0.f;
        const char* qrow = stage + Q_BASE + lane * kRB;
#pragma unroll
        for (int c4 = 0; c4 < kC / 4; ++c4) {
            float x[4];
            Quad<T>::unpack(*reinterpret_cast<const typename Quad<T>::raw*>(qrow + c4 * 8), x);
            const float4 bk = *reinterpret_cast<const float4*>(blank_k + h * kC + 4 * c4);
            part += x[0] * bk.x + x[1] * bk.y + x[2] * bk.z + x[3] * bk.w;
        }
        *reinterpret_cast<float*>(stage + BL_BASE + lane * 4) = part * scale;
    }
    const float bv[2] = {blank_v[h * kC + r16], blank_v[h * kC + 16 + r16]};

    Piece kb[kNB];
#pragma unroll
    for (int bj = 0; bj < kNB; ++bj) {
        kb[bj] = *reinterpret_cast<const Piece*>(stage + K_BASE + (16 * bj + r16) * kRB + kq * 16);
    }
    lds_sync();  // the blank logits are written

    // ---- scores and softmax, 16 rows at a time ------------------------------------------------------------------
    float pb[kNB][4];  // probability of the blank token for the lane's rows
#pragma unroll
    for (int bi = 0; bi < kNB; ++bi) {
        if (16 * bi < N) {
            const Piece qa = *reinterpret_cast<const Piece*>(stage + Q_BASE + (16 * bi + r16) * kRB + kq * 16);
            const F32x4 bl = *reinterpret_cast<const F32x4*>(stage + BL_BASE + (16 * bi + 4 * kq) * 4);
            F32x4 s[kNB];
#pragma unroll
            for (int bj = 0; bj < kNB; ++bj) s[bj] = tile_mfma<T>(qa, kb[bj], F32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float x[kNB];
                float mx = -INFINITY;
#pragma unroll
                for (int bj = 0; bj < kNB; ++bj) {
                    x[bj] = 16 * bj + r16 < N ? s[bj][j] * scale + bias[bi][bj][j] : -INFINITY;
                    mx = fmaxf(mx, x[bj]);
                }
                mx = fmaxf(row_max(mx), bl[j]);
                float sum = 0.f;
#pragma unroll
                for (int bj = 0; bj < kNB; ++bj) {
                    x[bj] = __expf(x[bj] - mx);
                    sum += x[bj];
                }
                const float eb = __expf(bl[j] - mx);
                const float inv = 1.f / (row_sum(sum) + eb);
                pb[bi][j] = eb * inv;
                T* prow = reinterpret_cast<T*>(stage + P_BASE) + (16 * bi + 4 * kq + j) * kPRow + r16;
#pragma unroll
                for (int bj = 0; bj < kNB; ++bj) prow[16 * bj] = from_acc<T>(x[bj] * inv);
            }
        }
    }
    lds_sync();  // the probabilities are written; the q rows are no longer read

    // ---- weighted sum of the V rows -------------------------------------------------------------------------------
    Piece vb[2][2];  // [32-key step][16-channel block]
#pragma unroll
    for (int st = 0; st < 2; ++st) {
        const char* col = stage + V_BASE + (32 * st + 8 * kq + (r16 >> 2)) * kRB + (r16 & 3) * 8;
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
            // keys 0-3 and 4-7 of the lane's 8, transposed to channel 16*cb + r16
            const S4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32));
            const S4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(col + cb * 32 + 4 * kRB));
            const U32x2 lo = __builtin_bit_cast(U32x2, b0), hi = __builtin_bit_cast(U32x2, b1);
            vb[st][cb] = Piece{lo[0], lo[1], hi[0], hi[1]};
        }
    }
#pragma unroll
    for (int bi = 0; bi < kNB; ++bi) {
        if (16 * bi < N) {
            F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                const Piece a = *reinterpret_cast<const Piece*>(stage + P_BASE + ((16 * bi + r16) * kPRow + 32 * st + 8 * kq) * 2);
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) acc[cb] = tile_mfma<T>(a, vb[st][cb], acc[cb]);
            }
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    reinterpret_cast<T*>(stage + O_BASE)[(16 * bi + 4 * kq + j) * kC + 16 * cb + r16] =
                        from_acc<T>(acc[cb][j] + pb[bi][j] * bv[cb]);
                }
            }
        }
    }
    lds_sync();

    // ---- output rows (N x 32, heads side by side in memory) ---------------------------------------------------------
    char* out_bh = reinterpret_cast<char*>(out + (int64_t)b * os.b + (int64_t)h * os.h);
#pragma unroll
    for (int a = 0; a < kNB; ++a) {
        const int row = 16 * a + g_sub;
        if (row < N) {
            const Piece o = *reinterpret_cast<const Piece*>(stage + O_BASE + a * 1024 + lane * 16);
            // plain store: the output projection reads it next
            *reinterpret_cast<Piece*>(out_bh + (int64_t)row * os.n * 2 + g_pos * 16) = o;
        }
    }
}

template <typename T>
int launch_typed(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                 clusten_strides vs, const void* table, const int64_t* pe_idx, const float* blank_k,
                 const float* blank_v, void* out, clusten_strides os, float scale, const clusten_attn_shape& s,
                 hipStream_t stream) {
    hipLaunchKernelGGL((dense_attention_kernel<T>), dim3((unsigned)(s.B * s.H)), dim3(kWave), 0, stream,
                       static_cast<const T*>(q), qs, static_cast<const T*>(k), ks, static_cast<const T*>(v), vs,
                       static_cast<const T*>(table), pe_idx, blank_k, blank_v, static_cast<T*>(out), os, s.H, s.N, scale);
    return launch_status();
}

}  // namespace

int launch_dense_attention(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                           clusten_strides vs, const void* table, const int64_t* pe_idx, const float* blank_k,
                           const float* blank_v, void* out, clusten_strides os, float scale, clusten_attn_shape s,
                           int dtype, hipStream_t stream) {
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (s.C != kC || s.N > kNMax || s.M != s.N || (int64_t)s.B * s.H >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    const bool ok = rows_aligned16(q, qs, 2) && rows_aligned16(k, ks, 2) && rows_aligned16(v, vs, 2) &&
                    rows_aligned16(out, os, 2) && aligned16(blank_k) && slice_fits_int32(ks, s.H, s.N, s.C) &&
                    slice_fits_int32(vs, s.H, s.N, s.C) && slice_fits_int32(qs, s.H, s.N, s.C);
    if (!ok) return CLUSTEN_ERR_UNALIGNED;
    if (dtype == CLUSTEN_F16) {
        return launch_typed<f16_t>(q, qs, k, ks, v, vs, table, pe_idx, blank_k, blank_v, out, os, scale, s, stream);
    }
    return launch_typed<bf16_t>(q, qs, k, ks, v, vs, table, pe_idx, blank_k, blank_v, out, os, scale, s, stream);
}

}  // namespace clusten
