// WF (adaptive down-sampling) kernels.
//
//   forward   out[b,i,ic,c]  = sum_j w[b,i,j,ic] * feat[b,idx[b,i,j],c]
//             (reference kernel clusten/src/clustenwf_cuda_kernel.cu:18-53)
//   d_weights d_w[b,i,j,ic]  = sum_c feat[b,idx[b,i,j],c] * d_out[b,i,ic,c]
//             (clustenwf_cuda_kernel.cu:137-169)
//   d_feat    d_feat[b,idx[b,i,j],c] += sum_ic d_out[b,i,ic,c] * w[b,i,j,ic]
//             (clustenwf_cuda_kernel.cu:96-135)
//
// Forward.  A gathered feature row is C*sizeof(T) bytes; LPT = that / 16 lanes cover it with one
// 16-byte access each, so a wave serves 64/LPT consecutive output tokens at once (4 tokens of 64
// fp32 channels) and every gather instruction moves whole rows, 1 KiB per wave access, straight
// into registers.  Each row is read once for all IC inner channels (the reference re-gathers it
// IC times).
// fp16 / bf16 weights over rows of the same type go four slots per instruction through `v_mfma_f32_4x4x4_16b_f16` /
// `_bf16` with the operands as they are stored (a quarter of the matrix instructions, no widening); everything else
// as below.
// The products run on the matrix cores as `v_mfma_f32_4x4x1_16b_f32`: 16 independent 4x4 blocks,
// one slot (k = 1) per instruction.  Block l/4 takes, as its B row, element e of the 16-byte groups
// that lanes 4*(l/4)..+3 hold (four channels of one token), and as its A column the token's four
// weights w[slot][0..3]; its D block is out[ic][those channels].  One MFMA per element e does the
// work of 4 VALU FMAs per lane at twice their rate, and leaves the accumulators exactly where a
// 16-byte store per inner channel needs them.
// The weights of the wave's tokens are one contiguous run of 64/LPT * M * IC elements; they go to
// LDS with LDS-direct loads and every lane reads weight (token, slot, l % 4) back as its A operand.
// The neighbour list of a token is spread over the rows of 16 lanes that belong to it and row
// indices are fetched by DPP row broadcast (see dpp.hpp).  Rows wider than 64 lanes are taken in
// 1 KiB column blocks.
// Rows that are not a multiple of 256 bytes, more than 4 inner channels, and weight rows that are
// not whole 16-byte pieces take the element-per-thread kernel.
//
// Backward: d_weights is a tile product on the matrix cores, one wave per output token (see
// wf_dweights_tile_kernel; other shapes take one thread per element); d_feat is one workgroup per output token,
// threads over channels, one fp32 atomic per (slot, channel) onto a contiguous destination row.
//
// This header holds the templates; wf_{f32,f16,bf16}.hip instantiate them per storage type so that
// the translation units build in parallel, wf.hip holds the dtype dispatch.
#pragma once

#include "dpp.hpp"
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {

// The lists and the merge weights are read once and loaded with the non-temporal hint (107.4 -> 106.4 us at 128 x
// (3136 -> 784) C=64 IC=4 fp32; either alone 107.0).
constexpr bool kWfHintLists = true;
constexpr bool kWfHintWeights = true;

// LPT = lanes per token (16, 32 or 64).  GUARD = false: the list has exactly 16*Q slots;
// GUARD = true: any length, taken 64 slots at a time (Q = 4) with every slot range-checked.
// TF = storage type of feat when it differs from T, the type of w and out: fp32 weights over fp16 / bf16 features, read
// in place (a lane takes its VEC channels of a row as 8 bytes and widens them): the same values and arithmetic as a cast
// of feat to fp32 ahead of the call, without that pass.
template <typename T, int LPT, int Q, bool GUARD, typename TF = T>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4))) void wf_forward_row_kernel(
    const T* __restrict__ w, const TF* __restrict__ feat, const int64_t* __restrict__ idx, T* __restrict__ out, int N,
    int Nout, int C, int M, int IC, int total_tokens, int total_groups) {
    typedef typename VecIO<TF, 16 / (int)sizeof(T)>::raw FeatRaw;   // the lane's channels of a gathered row
    constexpr int TPW = kWave / LPT;               // output tokens per wave
    constexpr int VEC = 16 / (int)sizeof(T);       // channels per lane and column block
    constexpr int SLOTS = 16 * Q;
    constexpr int NL = Q;                          // registers that hold one chunk of a token's list
    constexpr int GS = 4;                          // gather accesses per pipeline group (two groups in flight)
    constexpr int W_BYTES = TPW * SLOTS * 4 * (int)sizeof(T);  // weights of one chunk of the wave's tokens (IC <= 4)
    constexpr int NI_W = (W_BYTES + 1023) / 1024;
    static_assert(LPT == 16 || LPT == 32 || LPT == 64, "a row of 16 lanes must belong to one token");
    static_assert(!GUARD || Q == 4, "guarded lists are taken 64 slots at a time");
    static_assert(GS == 4, "the 16-bit path multiplies the four slots of a pipeline group at once");

    __shared__ __attribute__((aligned(1024))) char wbuf[NI_W * 1024];

    const int group = xcd_tile(blockIdx.x, total_groups);
    if (group < 0) return;
    const int lane = threadIdx.x;
    const int rl = lane & 15;
    // the lane's token (lanes past the last token repeat it; their stores are masked)
    const int tl = lane / LPT;                            // token of the lane inside the wave
    const int token0 = group * TPW;
    const int ntok = min(TPW, total_tokens - token0);    // tokens of this wave
    const bool token_ok = tl < ntok;
    const int token = token0 + min(tl, ntok - 1);
    const int b = token / Nout;
    const int col = (lane % LPT) * VEC;  // first channel of the lane inside a column block
    const int ic_lane = lane & 3;        // the row of the 4x4 blocks this lane feeds: inner channel

    const int64_t* list_p = idx + (int64_t)token * M;
    const char* feat_b = reinterpret_cast<const char*>(feat + (int64_t)b * N * C);
    T* out_tok = out + (int64_t)token * IC * C;
    const uint32_t row_bytes = (uint32_t)C * sizeof(TF);
    // weights: the wave's tokens are consecutive, so their rows are one contiguous run
    const char* w_wave = reinterpret_cast<const char*>(w + (int64_t)token0 * M * IC);
    const int w_tok_bytes = M * IC * (int)sizeof(T);

    for (int c0 = 0; c0 < C; c0 += LPT * VEC) {
        F32x4 acc[VEC];  // acc[e][ic] = out[ic][c0 + col + e]
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = F32x4{0.f, 0.f, 0.f, 0.f};
        const uint32_t lane_bytes = (uint32_t)(c0 + col) * sizeof(TF);

        for (int j0 = 0; j0 < M; j0 += kWave) {
            const int mc = min(kWave, M - j0);

            // list: slot 16*k + rl of the token in register k of its row(s) of 16 lanes
            int lst[NL];
#pragma unroll
            for (int k = 0; k < NL; ++k) lst[k] = (int)load_stream<kWfHintLists>(list_p + j0 + min(16 * k + rl, mc - 1));

            // weights of this chunk -> LDS.  A single chunk (M <= 64) of all the wave's tokens is one
            // contiguous run; otherwise each token's mc*IC elements are moved separately to t*mc*IC.
            __syncthreads();  // the previous chunk's / column block's reads are complete
            const int w_chunk_bytes = mc * IC * (int)sizeof(T);
            if (mc == M) {
                const int pieces = ntok * w_chunk_bytes / 16;
#pragma unroll
                for (int i = 0; i < NI_W; ++i) {
                    CLUSTEN_LDS_DMA16_STREAM(w_wave + min(i * kWave + lane, pieces - 1) * 16, wbuf + i * 1024, kWfHintWeights);
                }
            } else {
                const int ppt = w_chunk_bytes / 16;  // pieces per token
#pragma unroll
                for (int i = 0; i < NI_W; ++i) {
                    const int q = min(i * kWave + lane, ntok * ppt - 1);
                    const int t = q / ppt, pc = q - t * ppt;
                    CLUSTEN_LDS_DMA16(w_wave + (int64_t)t * w_tok_bytes + (int64_t)j0 * IC * sizeof(T) + pc * 16,
                                      wbuf + i * 1024);
                }
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            __syncthreads();
            // this lane's A operands: weight (its token, slot j, inner channel l % 4).  Lanes of an inner channel past
            // IC read the last one: the rows of the 4x4 blocks they feed are never stored.
            const char* w_lane = wbuf + min(tl, ntok - 1) * w_chunk_bytes + min(ic_lane, IC - 1) * (int)sizeof(T);

            FeatRaw fv[SLOTS];
            T wv[SLOTS];
            slot_pipeline<SLOTS, GS>(
                [&](auto ji) {
                    constexpr int j = decltype(ji)::value;
                    // row index of slot j: lane j % 16 of list register j / 16, broadcast inside each row of 16.
                    // Row index and row size are below 2^24 and the offset fits 32 bits (checked by the launcher):
                    // one 24-bit multiply-add, and the access is encoded as uniform base + lane offset.
                    const int row = rowlane_bcast<j % 16>(lst[j / 16]);
                    const uint32_t off = __umul24((uint32_t)((GUARD && j >= mc) ? 0 : row), row_bytes) + lane_bytes;
                    fv[j] = *reinterpret_cast<const FeatRaw*>(feat_b + lane_offset(off));
                    // the weight of the slot comes from LDS with the group's rows, a pipeline group ahead of its use
                    wv[j] = *reinterpret_cast<const T*>(w_lane + (GUARD ? min(j, mc - 1) : j) * IC * (int)sizeof(T));
                },
                [&](auto ji) {
                    constexpr int j = decltype(ji)::value;
                    if constexpr (sizeof(T) == 2 && std::is_same<T, TF>::value) {
                        // 16-bit weights and rows: four slots per matrix instruction (k = 4), operands as stored.
                        // A = the lane's inner channel of the weights of slots j-3..j; B = one channel of the four
                        // gathered rows: the low (high) halves of word d of the four rows are channel 2d (2d+1).
                        if constexpr (j % 4 == 3) {
                            uint32_t wbits[4];
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                wbits[q] = (!GUARD || j - 3 + q < mc) ? storage_bits(wv[j - 3 + q]) : 0u;
                            }
                            const U32x2 aop = U32x2{wbits[0] | (wbits[1] << 16), wbits[2] | (wbits[3] << 16)};
#pragma unroll
                            for (int d = 0; d < 4; ++d) {
                                uint32_t x[4];
#pragma unroll
                                for (int q = 0; q < 4; ++q) x[q] = (!GUARD || j - 3 + q < mc) ? fv[j - 3 + q][d] : 0u;
                                const U32x2 lo = U32x2{__builtin_amdgcn_perm(x[1], x[0], 0x05040100u),
                                                       __builtin_amdgcn_perm(x[3], x[2], 0x05040100u)};
                                const U32x2 hi = U32x2{__builtin_amdgcn_perm(x[1], x[0], 0x07060302u),
                                                       __builtin_amdgcn_perm(x[3], x[2], 0x07060302u)};
                                acc[2 * d] = mfma_4x4x4_16b<T>(aop, lo, acc[2 * d]);
                                acc[2 * d + 1] = mfma_4x4x4_16b<T>(aop, hi, acc[2 * d + 1]);
                            }
                        }
                    } else {
                        const float aop = (!GUARD || j < mc) ? to_acc(wv[j]) : 0.f;
                        float x[VEC];
                        VecIO<TF, VEC>::unpack(fv[j], x);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            const float bop = (!GUARD || j < mc) ? x[e] : 0.f;
                            acc[e] = mfma_4x4x1(aop, bop, acc[e]);
                        }
                    }
                });
        }

        if (token_ok) {
#pragma unroll
            for (int ic = 0; ic < 4; ++ic) {
                if (ic < IC) {
                    float v[VEC];
#pragma unroll
                    for (int e = 0; e < VEC; ++e) v[e] = acc[e][ic];
                    store_streaming(reinterpret_cast<Piece*>(out_tok + (int64_t)ic * C + c0 + col), VecIO<T, VEC>::pack(v));
                }
            }
        }
    }
}

// One thread per output element; any dtype and shape.
template <typename T>
__global__ __launch_bounds__(256) void wf_forward_elem_kernel(const T* __restrict__ w, const T* __restrict__ feat,
                                                              const int64_t* __restrict__ idx, T* __restrict__ out,
                                                              int B, int N, int Nout, int C, int M, int IC) {
    const int64_t total = (int64_t)B * Nout * IC * C;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(o % C);
        const int64_t q1 = o / C;
        const int ic = (int)(q1 % IC);
        const int64_t token = q1 / IC;  // b*Nout + i
        const int b = (int)(token / Nout);
        const int64_t* list = idx + token * M;
        const T* wrow = w + token * M * IC + ic;
        const T* base = feat + (int64_t)b * N * C + c;
        typename Acc<T>::type acc = 0;
        for (int j = 0; j < M; ++j) acc += to_acc(wrow[(int64_t)j * IC]) * to_acc(base[list[j] * C]);
        out[o] = from_acc<T>(acc);
    }
}

// d_w: one thread per (b,i,j,ic) element, a serial dot product over the C channels.
template <typename T>
__global__ __launch_bounds__(256) void wf_dweights_kernel(const T* __restrict__ d_out, const T* __restrict__ feat,
                                                          const int64_t* __restrict__ idx, T* __restrict__ d_w, int B,
                                                          int N, int Nout, int C, int M, int IC) {
    const int64_t total = (int64_t)B * Nout * M * IC;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int ic = (int)(o % IC);
        const int64_t q1 = o / IC;  // token*M + j
        const int64_t token = q1 / M;
        const int b = (int)(token / Nout);
        const T* frow = feat + ((int64_t)b * N + idx[q1]) * C;
        const T* grow = d_out + (token * IC + ic) * C;
        typename Acc<T>::type acc = 0;
        for (int c = 0; c < C; ++c) acc += to_acc(frow[c]) * to_acc(grow[c]);
        d_w[o] = from_acc<T>(acc);
    }
}

// d_w on the matrix cores.  For one output token  D[slot][ic] = sum_c G[slot][c] * dO[ic][c]  with G the rows its
// list gathers and dO its IC rows of d_out: the shared-list tile product of the QK kernel with the inner
// channels in the place of the tile's tokens.  One wave per output token; the channels are taken 256 bytes of a
// row at a time (rows and d_out rows by LDS-direct load, XOR-swizzled so that the 16-byte operand reads of the 16
// lanes of an MFMA row fall into different bank groups), 16x16 MFMA blocks, D accumulated over the column blocks.
// The result leaves through LDS in the (slot, ic) order of d_w as full-width stores.  fp32 with at most four inner
// channels takes sixteen 4x4 blocks per instruction instead, lane = slot (see below): a third of the matrix-pipe time
// and the result already in the order of d_w.  The rows in flight are bounded by the LDS they land in (14 KB a wave),
// so a wave takes four consecutive tokens and has the next one's list on its way while the present one's rows
// arrive.  Stage 1 (B128, 3136 -> 784 tokens, C64, IC4, fp32): 177 -> 150 us (4x4 blocks) -> 135 us (four tokens).
constexpr int kDwTokens = 4;   // output tokens per wave of wf_dweights_tile_kernel

template <typename T, int Q>
__global__ __launch_bounds__(kWave) void wf_dweights_tile_kernel(const T* __restrict__ d_out,
                                                                 const T* __restrict__ feat,
                                                                 const int64_t* __restrict__ idx, T* __restrict__ d_w,
                                                                 int N, int Nout, int C, int M, int IC,
                                                                 int total_tokens) {
    constexpr int RB = 256;                       // bytes of a row handled per column block
    constexpr int CB = RB / (int)sizeof(T);       // channels per column block
    constexpr int ROWS = 16 * Q;                  // list slots (staging rows)
    constexpr int NI_G = ROWS / 4;                // a wave access moves 4 rows of 256 bytes
    constexpr int G_BYTES = ROWS * RB;
    constexpr int VEC = 16 / (int)sizeof(T);      // elements per 16-byte piece
    constexpr int NU = 4;                         // pieces per lane: a quarter row
    typedef VecIO<T, VEC> RunIO;

    __shared__ __attribute__((aligned(1024))) char stage[G_BYTES + 8 * RB];

    // a wave takes kDwTokens consecutive output tokens; the list of the next one is requested while the rows of the
    // present one are on their way (a wave that waits for its list holds LDS that nothing is being loaded into)
    const int unit = xcd_tile(blockIdx.x, (total_tokens + kDwTokens - 1) / kDwTokens);
    if (unit < 0) return;
    const int token0 = unit * kDwTokens;
    const int lane = threadIdx.x;
    const int r = lane & 15, kq = lane >> 4;      // MFMA row / k index: the lane holds quarter kq of row r
    const int g_sub = lane >> 4, g_pos = lane & 15;  // gather side: piece g_pos of staging row 4*i + g_sub
    const uint32_t row_pitch = (uint32_t)C * sizeof(T);
    // lists of more than 16*Q slots go 16*Q slots at a time
    const int chunks = (M + ROWS - 1) / ROWS;
    const int items = min(kDwTokens, total_tokens - token0) * chunks;
    auto list_of = [&](int item) {
        const int t = item / chunks, j0 = (item - t * chunks) * ROWS;
        return (int)idx[(int64_t)(token0 + t) * M + j0 + min(lane, min(ROWS, M - j0) - 1)];
    };
    int mine_next = list_of(0);
    for (int item = 0; item < items; ++item) {
    const int mine = mine_next;
    if (item + 1 < items) mine_next = list_of(item + 1);
    const int token = token0 + item / chunks;
    const int j0 = (item % chunks) * ROWS;
    const int mc = min(ROWS, M - j0);
    const int b = token / Nout;
    const char* feat_b = reinterpret_cast<const char*>(feat + (int64_t)b * N * C);
    const char* g_tok = reinterpret_cast<const char*>(d_out + (int64_t)token * IC * C);

    uint32_t g_off[NI_G];
#pragma unroll
    for (int i = 0; i < NI_G; ++i) {
        const int srow = 4 * i + g_sub;
        g_off[i] = (uint32_t)__shfl(mine, min(srow, mc - 1)) * row_pitch + (uint32_t)((g_pos ^ (srow & 15)) * 16);
    }
    uint32_t a_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int srow = 4 * i + g_sub;
        a_off[i] = (uint32_t)min(srow, IC - 1) * row_pitch + (uint32_t)((g_pos ^ (srow & 15)) * 16);
    }
    int lds_g[NU], lds_a[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        lds_g[u] = r * RB + (((kq * NU + u) ^ r) * 16);
        lds_a[u] = G_BYTES + (r & 7) * RB + (((kq * NU + u) ^ (r & 7)) * 16);
    }

    if constexpr (sizeof(T) == 4) {
        if (IC <= 4) {
            // fp32, at most four inner channels: sixteen 4x4 blocks per instruction (`v_mfma_f32_4x4x1_16b_f32`) with
            // lane = slot.  Block l/4: A = dO[ic = l%4][c], B = G[slot l][c]; the lane ends with D[ic 0..3][slot l],
            // the four consecutive elements of d_w it stores.  64 instructions of 8 clocks per 64 channels in the
            // place of 48 16x16x4 instructions of 32 clocks that use four of their sixteen columns.
            const int srow = min(lane, ROWS - 1);
            const int ic = min(lane & 3, IC - 1);
            F32x4 acc = F32x4{0.f, 0.f, 0.f, 0.f};
            for (int c0 = 0; c0 < C; c0 += CB) {
                const uint32_t col_bytes = (uint32_t)c0 * sizeof(T);
                lds_sync();  // the previous column block's operands are in registers
#pragma unroll
                for (int i = 0; i < 2; ++i) CLUSTEN_LDS_DMA16(g_tok + (a_off[i] + col_bytes), stage + G_BYTES + i * 1024);
#pragma unroll
                for (int i = 0; i < NI_G; ++i) CLUSTEN_LDS_DMA16(feat_b + (g_off[i] + col_bytes), stage + i * 1024);
                lds_sync_vm<0>();
#pragma unroll 4
                for (int u = 0; u < 16; ++u) {
                    const Piece g = *reinterpret_cast<const Piece*>(stage + srow * RB + ((u ^ (srow & 15)) * 16));
                    const Piece a = *reinterpret_cast<const Piece*>(stage + G_BYTES + ic * RB + ((u ^ ic) * 16));
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc = mfma_4x4x1(__uint_as_float(a[e]), __uint_as_float(g[e]), acc);
                }
            }
            if (lane < mc) {
                T* dst = d_w + ((int64_t)token * M + j0 + lane) * IC;
                if (IC == 4) {
                    store_streaming(reinterpret_cast<Piece*>(dst), __builtin_bit_cast(Piece, acc));
                } else {
                    for (int v = 0; v < IC; ++v) dst[v] = acc[v];
                }
            }
            lds_sync();  // the rows have been read before the next chunk's arrive
            continue;
        }
    }

    F32x4 d[Q];
#pragma unroll
    for (int blk = 0; blk < Q; ++blk) d[blk] = F32x4{0.f, 0.f, 0.f, 0.f};

    for (int c0 = 0; c0 < C; c0 += CB) {
        const uint32_t col_bytes = (uint32_t)c0 * sizeof(T);
        lds_sync();  // the previous column block's operands are in registers
#pragma unroll
        for (int i = 0; i < 2; ++i) CLUSTEN_LDS_DMA16(g_tok + (a_off[i] + col_bytes), stage + G_BYTES + i * 1024);
#pragma unroll
        for (int i = 0; i < NI_G; ++i) CLUSTEN_LDS_DMA16(feat_b + (g_off[i] + col_bytes), stage + i * 1024);
        lds_sync_vm<0>();

        typename RunIO::raw a_raw[NU];
#pragma unroll
        for (int u = 0; u < NU; ++u) a_raw[u] = *reinterpret_cast<const typename RunIO::raw*>(stage + lds_a[u]);
#pragma unroll
        for (int blk = 0; blk < Q; ++blk) {
            typename RunIO::raw g_raw[NU];
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                g_raw[u] = *reinterpret_cast<const typename RunIO::raw*>(stage + lds_g[u] + blk * 16 * RB);
            }
#pragma unroll
            for (int u = 0; u < NU; ++u) d[blk] = tile_mfma<T>(g_raw[u], a_raw[u], d[blk]);
        }
    }

    // lane (r, kq) holds slots 16*blk + 4*kq .. +3 of inner channel r; d_w of the token is M*IC contiguous elements
    lds_sync();
    if (r < IC) {
#pragma unroll
        for (int blk = 0; blk < Q; ++blk) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int slot = 16 * blk + 4 * kq + e;
                if (slot < mc) reinterpret_cast<T*>(stage)[slot * IC + r] = from_acc<T>(d[blk][e]);
            }
        }
    }
    lds_sync();
    const int out_bytes = mc * IC * (int)sizeof(T);
    char* dst = reinterpret_cast<char*>(d_w + ((int64_t)token * M + j0) * IC);
    for (int off = lane * 16; off < out_bytes; off += kWave * 16) {
        store_streaming(reinterpret_cast<Piece*>(dst + off), *reinterpret_cast<const Piece*>(stage + off));
    }
    lds_sync();  // the chunk has left LDS before the next one's rows arrive
    }
}

// d_feat: one workgroup per output token, threads over channels; per slot the IC products are
// summed in registers and leave as one atomic per channel onto a contiguous destination row.
template <typename T, typename A>
__global__ __launch_bounds__(256) void wf_dfeat_kernel(const T* __restrict__ d_out, const T* __restrict__ w,
                                                       const int64_t* __restrict__ idx, A* __restrict__ d_feat, int N,
                                                       int Nout, int C, int M, int IC, int total_tokens,
                                                       const int32_t* __restrict__ only_if) {
    if (only_if != nullptr && *only_if == 0) return;   // the cluster-by-cluster kernel has these lists
    const int token = xcd_tile(blockIdx.x, total_tokens);
    if (token < 0) return;
    {
    const int b = token / Nout;
    const int64_t* list = idx + (int64_t)token * M;
    const T* wtok = w + (int64_t)token * M * IC;
    const T* gtok = d_out + (int64_t)token * IC * C;
    A* dst_b = d_feat + (int64_t)b * N * C;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        for (int j = 0; j < M; ++j) {
            A sum = 0;
            for (int ic = 0; ic < IC; ++ic) sum += (A)to_acc(gtok[(int64_t)ic * C + c]) * (A)to_acc(wtok[j * IC + ic]);
            unsafeAtomicAdd(dst_b + list[j] * C + c, sum);
        }
    }
    }
}

inline int elem_grid(int64_t total) {
    const int64_t want = (total + 255) / 256;
    return (int)(want < (int64_t)1 << 20 ? want : (int64_t)1 << 20);
}

template <typename T, int LPT, typename TF = T>
int wf_forward_row(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    const int total = s.B * s.Nout;
    const int groups = (total + kWave / LPT - 1) / (kWave / LPT);
    if (s.M == 48) {  // the neighbourhood size of every 224x224 model: no range checks
        hipLaunchKernelGGL((wf_forward_row_kernel<T, LPT, 3, false, TF>), dim3(xcd_grid(groups)), dim3(kWave), 0, stream,
                           static_cast<const T*>(w), static_cast<const TF*>(feat), idx, static_cast<T*>(out), s.N,
                           s.Nout, s.C, s.M, s.IC, total, groups);
    } else {
        hipLaunchKernelGGL((wf_forward_row_kernel<T, LPT, 4, true, TF>), dim3(xcd_grid(groups)), dim3(kWave), 0, stream,
                           static_cast<const T*>(w), static_cast<const TF*>(feat), idx, static_cast<T*>(out), s.N,
                           s.Nout, s.C, s.M, s.IC, total, groups);
    }
    return launch_status();
}

template <typename T, typename TF = T>
int wf_forward_vec(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    // lanes per token: the widest of 64, 32, 16 whose 16-byte accesses (of T) tile the row
    const int row_bytes = s.C * (int)sizeof(T);
    if (row_bytes % 1024 == 0) return wf_forward_row<T, 64, TF>(w, feat, idx, out, s, stream);
    if (row_bytes % 512 == 0) return wf_forward_row<T, 32, TF>(w, feat, idx, out, s, stream);
    return wf_forward_row<T, 16, TF>(w, feat, idx, out, s, stream);
}

template <typename T>
int wf_forward_elem(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                    hipStream_t stream) {
    const int64_t total = (int64_t)s.B * s.Nout * s.IC * s.C;
    hipLaunchKernelGGL((wf_forward_elem_kernel<T>), dim3(elem_grid(total)), dim3(256), 0, stream,
                       static_cast<const T*>(w), static_cast<const T*>(feat), idx, static_cast<T*>(out), s.B, s.N,
                       s.Nout, s.C, s.M, s.IC);
    return launch_status();
}

template <typename T>
int wf_forward_typed(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                     hipStream_t stream) {
    // whole 256-byte rows, and 32-bit byte offsets inside one batch element of feat
    const bool rows_ok = (s.C * (int)sizeof(T)) % 256 == 0 && aligned16(feat) && aligned16(out) &&
                         (int64_t)s.N * s.C * (int64_t)sizeof(T) < ((int64_t)1 << 31);
    // weight rows (and every 64-slot chunk of one) are whole 16-byte pieces; at most 4 inner channels
    const bool w_ok = s.IC <= 4 && ((int64_t)s.M * s.IC * sizeof(T)) % 16 == 0 && aligned16(w) &&
                      (s.M <= 64 || (64 * s.IC * (int)sizeof(T)) % 16 == 0);
    if (rows_ok && w_ok) return wf_forward_vec<T>(w, feat, idx, out, s, stream);
    return wf_forward_elem<T>(w, feat, idx, out, s, stream);
}

// One thread per output element, feat of another storage type than w and out.
template <typename T, typename TF>
__global__ __launch_bounds__(256) void wf_forward_mixed_elem_kernel(const T* __restrict__ w, const TF* __restrict__ feat,
                                                                    const int64_t* __restrict__ idx, T* __restrict__ out,
                                                                    int B, int N, int Nout, int C, int M, int IC) {
    const int64_t total = (int64_t)B * Nout * IC * C;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(o % C);
        const int64_t q1 = o / C;
        const int ic = (int)(q1 % IC);
        const int64_t token = q1 / IC;  // b*Nout + i
        const int b = (int)(token / Nout);
        const int64_t* list = idx + token * M;
        const T* wrow = w + token * M * IC + ic;
        const TF* base = feat + (int64_t)b * N * C + c;
        float acc = 0.f;
        for (int j = 0; j < M; ++j) acc += to_acc(wrow[(int64_t)j * IC]) * to_acc(base[list[j] * C]);
        out[o] = from_acc<T>(acc);
    }
}

// fp32 weights and output with features of TF = fp16 / bf16, read in place (see the TF parameter of the row kernel).
template <typename TF>
int wf_forward_mixed_typed(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                           hipStream_t stream) {
    const bool rows_ok = (s.C * 4) % 256 == 0 && (reinterpret_cast<uintptr_t>(feat) & 7u) == 0 && aligned16(out) &&
                         (int64_t)s.N * s.C * 2 < ((int64_t)1 << 31);
    const bool w_ok = s.IC <= 4 && ((int64_t)s.M * s.IC * 4) % 16 == 0 && aligned16(w) && (s.M <= 64 || (64 * s.IC * 4) % 16 == 0);
    if (rows_ok && w_ok) return wf_forward_vec<float, TF>(w, feat, idx, out, s, stream);
    const int64_t total = (int64_t)s.B * s.Nout * s.IC * s.C;
    hipLaunchKernelGGL((wf_forward_mixed_elem_kernel<float, TF>), dim3(elem_grid(total)), dim3(256), 0, stream,
                       static_cast<const float*>(w), static_cast<const TF*>(feat), idx, static_cast<float*>(out), s.B, s.N,
                       s.Nout, s.C, s.M, s.IC);
    return launch_status();
}

template <typename T>
int wf_dweights_typed(const void* d_out, const void* feat, const int64_t* idx, void* d_w, const clusten_wf_shape& s,
                      hipStream_t stream) {
    // whole 256-byte row blocks, 32-bit byte offsets inside one batch element of feat, d_w rows in 16-byte pieces
    const bool tile_ok = (s.C * (int)sizeof(T)) % 256 == 0 && aligned16(feat) && aligned16(d_out) && aligned16(d_w) &&
                         (int64_t)s.N * s.C * (int64_t)sizeof(T) < ((int64_t)1 << 31) && s.IC <= 8 &&
                         ((int64_t)s.M * s.IC * sizeof(T)) % 16 == 0 &&
                         (s.M <= 64 || (64 * s.IC * (int)sizeof(T)) % 16 == 0);
    if constexpr (sizeof(T) <= 4) if (tile_ok) {
        const int total_tokens = s.B * s.Nout;
        if (s.M <= 48) {
            hipLaunchKernelGGL((wf_dweights_tile_kernel<T, 3>), dim3(xcd_grid((total_tokens + kDwTokens - 1) / kDwTokens)), dim3(kWave), 0, stream,
                               static_cast<const T*>(d_out), static_cast<const T*>(feat), idx, static_cast<T*>(d_w),
                               s.N, s.Nout, s.C, s.M, s.IC, total_tokens);
        } else {
            hipLaunchKernelGGL((wf_dweights_tile_kernel<T, 4>), dim3(xcd_grid((total_tokens + kDwTokens - 1) / kDwTokens)), dim3(kWave), 0, stream,
                               static_cast<const T*>(d_out), static_cast<const T*>(feat), idx, static_cast<T*>(d_w),
                               s.N, s.Nout, s.C, s.M, s.IC, total_tokens);
        }
        return launch_status();
    }
    const int64_t total = (int64_t)s.B * s.Nout * s.M * s.IC;
    hipLaunchKernelGGL((wf_dweights_kernel<T>), dim3(elem_grid(total)), dim3(256), 0, stream,
                       static_cast<const T*>(d_out), static_cast<const T*>(feat), idx, static_cast<T*>(d_w), s.B, s.N,
                       s.Nout, s.C, s.M, s.IC);
    return launch_status();
}

template <typename T, typename A>
int wf_dfeat_typed(const void* d_out, const void* w, const int64_t* idx, A* acc, const clusten_wf_shape& s,
                   hipStream_t stream, const int32_t* only_if) {
    const int total = s.B * s.Nout;
    const int threads = s.C >= 256 ? 256 : (s.C > 64 ? 128 : 64);
    hipLaunchKernelGGL((wf_dfeat_kernel<T, A>), dim3(xcd_grid(total)), dim3(threads), 0, stream,
                       static_cast<const T*>(d_out), static_cast<const T*>(w), idx, acc, s.N, s.Nout, s.C, s.M, s.IC,
                       total, only_if);
    return launch_status();
}

}  // namespace clusten
