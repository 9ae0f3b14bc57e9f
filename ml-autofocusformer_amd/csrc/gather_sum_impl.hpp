// gather_sum: out[b,h,i,c] = sum_j p[b,h,i,j] * rows[b,h,idx[b,i,j],c]
//
// This is the CLUSTEN AV forward (p = attn, rows = value; reference kernel
// clusten/src/clustenav_cuda_kernel.cu:18-50) and the d_query half of the QK backward
// (p = d_attn, rows = key; clusten/src/clustenqk_cuda_kernel.cu:91-132, the dq_update sum).
//
// Work decomposition.  One wave owns a tile of 8 consecutive tokens of one batch element and
// walks all heads, so the int64 neighbour lists of the tile are read from HBM exactly once.
// Per head the tile is a small matrix product  D[token][c] = P[token][slot] * G[slot][c]  with G
// the gathered rows; it runs on the matrix cores as fp32 MFMA 16x16x4 blocks (16 tokens of which
// 8 are real x 16 channels, 4 slots per step).
//
// Data path per head:
//   1. gather: `global_load_lds_dwordx4` moves the gathered rows straight into LDS, row-coalesced
//      (consecutive lanes on consecutive 16-byte pieces of one row), and the tile's p-rows as well.
//      The p pieces (4 slots of one token, 16 bytes) are laid out piece-transposed, [slot group][token],
//      so that the 8 tokens' pieces of one slot group are contiguous.
//   2. operands: lane (n = lane % 16, kq = lane / 16) is column n of the B operand and k-index kq.
//      For MFMA step s it reads channels [n*C/16, (n+1)*C/16) of gathered row 4*s + kq (channel
//      n*C/16 + e belongs to channel block e), and element kq of p piece (token n % 8, slot group s).
//   3. the D blocks leave lane (n, mq = lane / 16) with tokens 4*mq..4*mq+3 of channels
//      n*C/16 + e.  When the out rows of the tile are contiguous they are laid out row-major in
//      LDS and leave with full-width 16-byte stores.
// One short-lived one-wave workgroup per tile; the latency of its dependent chain (lists, rows,
// product, store) is hidden by the other waves resident on the CU.
//
//   shared-list path — all tokens of the tile carry the same list: one gather and one set of MFMAs
//     per head serve the 8 tokens.
//   union path — lists that differ but are made of runs of 8 slots of which the tile's tokens share most
//     (the neighbourhoods of a cluster-ordered sequence): every distinct run is gathered once, the p values
//     are re-indexed by distinct run in LDS (zero where a token does not hold a run), one set of MFMAs per
//     pass of 6 or 8 runs serves the 8 tokens.
//   per-token path — any other tile: the gather and the MFMAs are repeated per token and only that
//     token's row is kept.  Exact for arbitrary indices (duplicates, any order), only slower.
//
// Storage types narrower than fp32 are widened in registers; all products and sums are fp32.  One case goes
// through the 16-bit matrix instructions instead: fp16 / bf16 data with a shared list of 48 slots.  The p pieces
// are A operands as they lie in LDS; the B operand (8 consecutive slots of one channel) is a column of the
// row-major gathered rows, read with `ds_read_b64_tr_b16`; two 16x16x32 steps per 16 channels replace twelve
// fp32 steps and their conversions (products of 16-bit values are exact in fp32, sums are fp32).
// Head dims other than 16/32/64, p rows that are not whole 16-byte pieces (M*sizeof(T) % 16 != 0),
// rows whose start is not 16-byte aligned and fp64 take the element-per-thread kernel at the
// bottom of the file.
//
// This header holds the templates; gather_sum_{f32,f16,bf16}.hip and gather_sum_clusters_{...}.hip (lists
// given as cluster numbers) instantiate them per storage type so that the translation units build in
// parallel, gather_sum.hip holds the dtype dispatch.
#pragma once

#include "launch.hpp"
#include "mfma.hpp"
#include "gather_runs24_impl.hpp"

namespace clusten {

// The tile's attention weights are read once and loaded with the non-temporal hint (108.1 -> 101.4 us at B=128 H=2
// N=3136 M=48 C=32 fp32, after the launch that made the weights from the same lists).  The lists are not: part of them
// is still in the memory-side cache from that launch, and a hinted load does not use it (110 us).
constexpr bool kSumHintLists = false;
constexpr bool kSumHintWeights = true;

// Geometry of the gather_sum staging buffer in LDS.
//   [0, G_BYTES)          gathered rows of one chunk (16*Q rows of RB bytes); reused to turn the D
//                         blocks into the row-major output chunk
//   [P_BASE, +2*P_SLOT)   p pieces of two heads (slot h % 2), piece-transposed: piece (slot group s,
//                         token t) at (s*8 + t)*16
//   union path only (FAST kernels):
//   (over the p slots)    p of one pass re-indexed by distinct run, as MFMA A operands: element
//                         (k index kq, token t, step s) at ((kq*8 + t)*PM_STRIDE + s)*4;
//                         distinct-run number of each of the tile's runs; row indices of up to
//                         U_MAX distinct runs, 8 per run
template <typename T, int C, int Q, bool UNION>
struct SumStaging {
    static constexpr int RB = C * (int)sizeof(T);               // bytes per gathered row
    static constexpr int PPR = RB / 16;                         // 16-byte pieces per row
    static constexpr int RPI = kWave / PPR;                     // rows per wave access
    static constexpr int NI_G = (16 * Q + RPI - 1) / RPI;       // accesses for the gathered rows of a chunk
    static constexpr int G_BYTES = NI_G * 1024 > kTileTokens * RB ? NI_G * 1024 : kTileTokens * RB;
    static constexpr int SPP = 16 / (int)sizeof(T);             // slots per p piece
    static constexpr int STEPS_PER_PIECE = SPP / 4;             // MFMA steps (4 slots) per p piece
    static constexpr int P_PIECES = 16 * Q / SPP * kTileTokens;  // p pieces of one (tile, head, chunk)
    static constexpr int NI_P = (P_PIECES + kWave - 1) / kWave;  // accesses for them
    static constexpr int P_BASE = G_BYTES;
    static constexpr int P_SLOT_BYTES = NI_P * 1024;
    static constexpr int ECH = C / 16;                          // channels per lane = channel blocks
    static constexpr int STEPS = 4 * Q;                         // MFMA steps per chunk
    // the union path's tables take the place of the two p slots once their pieces are in registers
    static constexpr int PM_STRIDE = STEPS % 8 == 4 ? STEPS : STEPS + 4;  // floats; odd multiple of 4: conflict-free rows
    static constexpr int PM_BASE = P_BASE;
    static constexpr int PM_BYTES = 4 * kTileTokens * PM_STRIDE * 4;
    static constexpr int USLOT_BASE = PM_BASE + PM_BYTES;       // one byte per run of the tile
    static constexpr int ULIST_BASE = USLOT_BASE + kWave;
    static constexpr int U_FIT = (2 * P_SLOT_BYTES - PM_BYTES - kWave) / 32;
    static constexpr int U_MAX = !UNION || U_FIT < 1 ? 0 : (U_FIT < 16 ? U_FIT : 16);  // distinct runs the union path holds
    static constexpr int BYTES = G_BYTES + 2 * P_SLOT_BYTES;
    static_assert(RB >= 32 && kWave % PPR == 0, "row size");
};

// FAST = the list has at most 64 slots: one chunk, p-rows of two heads prefetched before the lists
// are read.  Otherwise lists go 64 slots at a time and the D blocks accumulate over the chunks.
// EXACT = the list has exactly 16*Q slots (no slot of the chunk is missing).
// CLUSTERS (FAST kernels only) = the lists arrive as int32 cluster numbers, M/8 per token: slot j of a token is row
// 8*g + j%8 of its cluster g = number j/8 (row 0 where that is past the last row); `idx` then points to (B, N, M/8) int32.
// TR = storage type of the gathered rows when it differs from T, the type of p and out: fp32 p with fp16 / bf16 rows
// (attention weights straight from a softmax times 16-bit values under mixed precision).  The rows are then read in
// place, eight bytes per lane, widened and written to the staging buffer in the layout the fp32 kernel keeps there:
// the same values and the same arithmetic as a cast of the rows to fp32 ahead of the call, without that pass.
template <typename T, int C, int Q, bool FAST, bool EXACT, bool CLUSTERS = false, typename TR = T>
__global__ __launch_bounds__(kWave) void gather_sum_tile_kernel(const T* __restrict__ p, const TR* __restrict__ rows,
                                                                const int64_t* __restrict__ idx,
                                                                T* __restrict__ out, int H_all, int N, int M,
                                                                clusten_strides rs, clusten_strides os,
                                                                int tiles_per_batch, int total_tiles, int head_groups) {
    typedef SumStaging<T, C, Q, FAST> S;
    typedef VecIO<T, S::ECH> ChIO;   // the lane's channels of one gathered row
    typedef VecIO<T, S::SPP> PieceIO;
    static_assert(C == 16 || C == 32 || C == 64, "channel blocks of 16");
    static_assert(FAST || Q == 4, "long lists are taken 64 slots at a time");
    static_assert(sizeof(TR) == sizeof(T) || (sizeof(T) == 4 && sizeof(TR) == 2), "rows of T, or 16-bit rows under fp32");
    constexpr int NARROW = (int)(sizeof(T) / sizeof(TR));   // 1, or 2 for 16-bit rows under fp32 p

    __shared__ __attribute__((aligned(1024))) char stage[S::BYTES];

    // One access of a gather: every lane brings 16 bytes of staging — its piece of a row — to `dst` + 16 * lane.
    // `off` is the byte offset of the piece inside (b, h) as if the rows were stored as T.
    auto stage_rows = [&](const char* rows_bh, uint32_t off, char* dst) {
        if constexpr (NARROW == 1) {
            CLUSTEN_LDS_DMA16(rows_bh + off, dst);
        } else {
            const U32x2 raw = *reinterpret_cast<const U32x2*>(rows_bh + lane_offset(off >> 1));
            float x[4];
            VecIO<TR, 4>::unpack(raw, x);
            *reinterpret_cast<F32x4*>(dst + threadIdx.x * 16) = F32x4{x[0], x[1], x[2], x[3]};
        }
    };

    // a workgroup serves the heads [h0, h0 + H) of its tile: short sequences with many heads are launched with
    // several head groups per tile (neighbours in the grid, so the later ones find the tile's lists in the L2)
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
    const int n = lane & 15;   // MFMA column of the B operand / row (token) of the A operand
    const int kq = lane >> 4;  // MFMA k index: slot 4*s + kq in step s; also the token group of the D rows
    const int g_sub = lane / S::PPR;  // gather side: in access i this lane moves one piece of row i*RPI + g_sub
    const int g_pos = lane % S::PPR;

    const char* rows_b = reinterpret_cast<const char*>(rows + (int64_t)b * rs.b + (int64_t)h0 * rs.h);
    const int64_t* idx_tile = idx + ((int64_t)b * N + i0) * M;
    const int32_t* cid_tile = reinterpret_cast<const int32_t*>(idx) + ((int64_t)b * N + i0) * (M >> 3);
    int cid = 0;  // CLUSTERS: the cluster number of run `lane` of the tile (token lane / R, run lane % R)
    const uint32_t row_pitch = (uint32_t)rs.n * sizeof(T);

    // p pieces of head h, chunk at slot j0 -> slot `ps` of the staging buffer.  Access i moves pieces
    // 64*i + lane; piece q is slot group q / 8 of token q % 8 (tokens past the end of a partial tile
    // repeat its last token, slot groups past the end of the list repeat its last group).
    auto fetch_p = [&](int h, int j0, int mc, int ps) {
        const char* p_head = reinterpret_cast<const char*>(p + (((int64_t)b * H_all + h0 + h) * N + i0) * M + j0);
#pragma unroll
        for (int i = 0; i < S::NI_P; ++i) {
            const int q = i * kWave + lane;
            const int grp = min(q / kTileTokens, mc / S::SPP - 1);
            const int tok = min(q % kTileTokens, nt - 1);
            CLUSTEN_LDS_DMA16_STREAM(p_head + ((int64_t)tok * M + grp * S::SPP) * sizeof(T),
                                     stage + S::P_BASE + ps * S::P_SLOT_BYTES + i * 1024, kSumHintWeights);
        }
    };
    if (FAST) {
        fetch_p(0, 0, M, 0);
        if (H > 1) fetch_p(1, 0, M, 1);
    }

    // Are all lists of the tile the same?  (over all chunks; the first list of each chunk stays in registers)
    constexpr int MAXCH = FAST ? 1 : 4;  // chunks whose first list is kept in registers; longer lists re-read
    int list0[MAXCH];
    bool same = true;
    if constexpr (CLUSTERS) {
        const int R = M >> 3, nruns = nt * R;
        const int slot = min(lane, M - 1);
        cid = cid_tile[min(lane, nruns - 1)];
        same = lane >= nruns || cid == __shfl(cid, lane % R);   // against the same run of the tile's first token
        const int row = __shfl(cid, slot >> 3) * 8 + (slot & 7);
        list0[0] = (unsigned)row < (unsigned)N ? row : 0;  // also catches a negative cluster number
    } else
    for (int j0 = 0, ch = 0; j0 < M; j0 += kWave, ++ch) {
        const int mc = min(kWave, M - j0);
        const int slot = min(lane, mc - 1);  // lanes past the list repeat its last slot
        int64_t wide[kTileTokens];
#pragma unroll
        for (int t = 0; t < kTileTokens; ++t) wide[t] = load_stream<kSumHintLists>(idx_tile + (int64_t)min(t, nt - 1) * M + j0 + slot);
#pragma unroll
        for (int t = 1; t < kTileTokens; ++t) same = same && (wide[t] == wide[0]);
#pragma unroll
        for (int k = 0; k < MAXCH; ++k) {
            if (k == ch) list0[k] = (int)wide[0];
        }
    }
    const bool shared_list = __all(same ? 1 : 0) != 0;

    // operand side
    const int lds_g = kq * S::RB + n * S::ECH * (int)sizeof(T);         // row kq of a step's 4 rows, the lane's channels
    const int lds_p = (n & 7) * 16;                                     // the lane's token inside a slot group
    // out: lane (n, kq) holds tokens 4*kq + i of channels n*ECH + e
    const bool rows_contiguous = os.n == C;

    // store of one head: lane (n, kq) holds tokens 4*kq + i of channels n*ECH + e.  `whole` = every token of
    // the tile is written: when the out rows of the tile are contiguous too, they are laid out row-major in
    // LDS (over the gathered rows) and leave with full-width 16-byte stores.
    auto store_head = [&](int h, F32x4 (&d)[S::ECH], int tok_lo, int tok_hi, bool whole) {
        char* out_h = reinterpret_cast<char*>(out + (int64_t)b * os.b + (int64_t)(h0 + h) * os.h + (int64_t)i0 * os.n);
        if (FAST && whole && rows_contiguous) {
            __syncthreads();  // every operand read of this head is complete: reuse the row area
            if (kq < 2) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v[S::ECH];
#pragma unroll
                    for (int e = 0; e < S::ECH; ++e) v[e] = d[e][i];
                    *reinterpret_cast<typename ChIO::raw*>(stage + ((4 * kq + i) * C + n * S::ECH) * (int)sizeof(T)) =
                        ChIO::pack(v);
                }
            }
            __syncthreads();
            constexpr int NO = (kTileTokens * S::RB + 1023) / 1024;
            Piece o[NO];
#pragma unroll
            for (int i = 0; i < NO; ++i) {
                o[i] = *reinterpret_cast<const Piece*>(stage + min(i * 1024 + lane * 16, S::G_BYTES - 16));
            }
            __syncthreads();  // the chunk is in registers: the next head's gather may overwrite it
            const int chunk_bytes = nt * S::RB;
#pragma unroll
            for (int i = 0; i < NO; ++i) {
                const int off = i * 1024 + lane * 16;
                if (off < chunk_bytes) store_streaming(reinterpret_cast<Piece*>(out_h + off), o[i]);
            }
        } else {
            if (FAST) __syncthreads();  // operand reads complete before the next head's gather
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tok = 4 * kq + i;
                if (tok >= tok_lo && tok < tok_hi) {
                    float v[S::ECH];
#pragma unroll
                    for (int e = 0; e < S::ECH; ++e) v[e] = d[e][i];
                    store_streaming(reinterpret_cast<typename ChIO::raw*>(out_h + ((int64_t)tok * os.n + n * S::ECH) * sizeof(T)),
                                    ChIO::pack(v));
                }
            }
        }
    };

    if constexpr (FAST && S::U_MAX > 0) {
        if (!shared_list && (M & 7) == 0) {
            // ---- union path: lists made of runs of 8 slots, many of them common to several tokens ----
            // (the neighbourhoods of a cluster-ordered sequence: a run is the 8 members of one cluster.)
            // Every distinct run is gathered once per head; the p values are re-indexed by distinct run
            // (zero where a token does not hold the run), so one set of MFMAs serves the 8 tokens.
            constexpr int PROWS = 16 * Q;     // union rows per pass
            const int R = M >> 3;             // runs per token
            const int nruns = nt * R;         // <= 64: lane rho owns run rho = token * R + run
            int v[8];
            if constexpr (CLUSTERS) {
#pragma unroll
                for (int t = 0; t < 8; ++t) v[t] = (unsigned)(cid * 8 + t) < (unsigned)N ? cid * 8 + t : 0;
            } else {
                const int64_t* lp = idx_tile + (int64_t)min(lane, nruns - 1) * 8;  // the tile's lists are contiguous
#pragma unroll
                for (int t = 0; t < 8; ++t) v[t] = (int)lp[t];
            }
            // 8 consecutive rows, or the short last cluster of the sequence followed by the row 0 its pad slots hold:
            // either way the first row tells the other seven
            const int own = ((N & 7) != 0 && v[0] == N - (N & 7)) ? (N & 7) : 8;
            bool regular = true;
#pragma unroll
            for (int t = 1; t < 8; ++t) regular = regular && (v[t] == (t < own ? v[0] + t : 0));
            const int key = regular ? v[0] : ~lane;  // other runs never merge

            // number the distinct keys in order of first appearance
            uint64_t remaining = nruns >= 64 ? ~0ull : ((1ull << nruns) - 1);
            // lanes below this one that hold runs of the same token: a run held twice by one token would need
            // two p values in one place of the re-indexed p
            const uint64_t same_token_below = ((1ull << lane) - 1) & ~((1ull << (lane / R * R)) - 1);
            int uslot = 0, U = 0;
            bool first = false, twice = false;
            while (remaining != 0 && U < S::U_MAX) {
                const int sl = __builtin_ctzll(remaining);
                const int ks = __builtin_amdgcn_readlane(key, sl);
                const bool hit = key == ks;
                const uint64_t match = __ballot(hit) & remaining;
                if (hit) uslot = U;
                twice = twice || (hit && lane < nruns && (match & same_token_below) != 0);
                first = first || lane == sl;
                remaining &= ~match;
                ++U;
            }
            // at most U_MAX distinct runs and no token holds a run twice; other tiles take the per-token passes
            if (remaining == 0 && __any(twice ? 1 : 0) == 0) {
                // The p pieces of heads 0 and 1 are on their way into the two p slots: take them into
                // registers; from then on the slots hold the run tables and the re-indexed p, and the
                // pieces of the later heads come straight from global memory, one head ahead.
                typename PieceIO::raw cur[S::NI_P], nxt[S::NI_P];
                __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                __syncthreads();
#pragma unroll
                for (int k = 0; k < S::NI_P; ++k) {
                    cur[k] = *reinterpret_cast<const typename PieceIO::raw*>(stage + S::P_BASE + (k * kWave + lane) * 16);
                    nxt[k] = *reinterpret_cast<const typename PieceIO::raw*>(stage + S::P_BASE + S::P_SLOT_BYTES +
                                                                            (k * kWave + lane) * 16);
                }
                __syncthreads();
                int* ulist = reinterpret_cast<int*>(stage + S::ULIST_BASE);
                unsigned char* uslots = reinterpret_cast<unsigned char*>(stage + S::USLOT_BASE);
                float* pm = reinterpret_cast<float*>(stage + S::PM_BASE);
                if (first) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) ulist[uslot * 8 + t] = v[t];
                }
                if (lane < nruns) uslots[lane] = (unsigned char)uslot;
                __syncthreads();

                // p piece q = 64*k + lane of a head: SPP slots of token q % 8 from slot (q / 8) * SPP on.
                // They go to union rows prow .. prow + SPP - 1, i.e. pass prow / PROWS, elements
                // pm[pm_at + (e % 4) * 8 * PM_STRIDE + e / 4].
                int ppass[S::NI_P], pm_at[S::NI_P];
                const T* p_src[S::NI_P];
#pragma unroll
                for (int k = 0; k < S::NI_P; ++k) {
                    const int q = k * kWave + lane;
                    const int j = (q / kTileTokens) * S::SPP;
                    const int tok = q % kTileTokens;
                    const bool valid = j < M && tok < nt;
                    const int prow = valid ? uslots[tok * R + (j >> 3)] * 8 + (j & 7) : 0;
                    ppass[k] = valid ? prow / PROWS : -1;
                    const int rr = prow % PROWS;
                    pm_at[k] = tok * S::PM_STRIDE + (rr >> 2);
                    p_src[k] = p + (((int64_t)b * H_all + h0) * N + i0 + min(tok, nt - 1)) * M + min(j, M - S::SPP);
                }
                const int total_rows = 8 * U;
                const float* pm_lane = pm + (kq * kTileTokens + (n & 7)) * S::PM_STRIDE;

                for (int h = 0; h < H; ++h) {
                    const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(TR);
                    if (h >= 1 && h + 1 < H) {
#pragma unroll
                        for (int k = 0; k < S::NI_P; ++k) {
                            nxt[k] = *reinterpret_cast<const typename PieceIO::raw*>(p_src[k] + (int64_t)(h + 1) * N * M);
                        }
                    }
                    F32x4 d[S::ECH];
#pragma unroll
                    for (int e = 0; e < S::ECH; ++e) d[e] = F32x4{0.f, 0.f, 0.f, 0.f};
                    float pv[S::NI_P][S::SPP];
#pragma unroll
                    for (int k = 0; k < S::NI_P; ++k) PieceIO::unpack(cur[k], pv[k]);

                    for (int base = 0, pass = 0; base < total_rows; base += PROWS, ++pass) {
                        const int rows_here = min(PROWS, total_rows - base);
                        const int rows_batched = (rows_here + 15) & ~15;  // MFMA batches cover 16 rows
                        lds_sync();  // the previous pass (or head) has read its operands
#pragma unroll
                        for (int i = 0; i < S::NI_G; ++i) {
                            if (i * S::RPI < rows_batched) {  // rows past the last one repeat it (their p is zero)
                                const uint32_t urow = (uint32_t)ulist[min(base + i * S::RPI + g_sub, total_rows - 1)];
                                stage_rows(rows_bh, urow * row_pitch + (uint32_t)(g_pos * 16), stage + i * 1024);
                            }
                        }
                        // clear the re-indexed p of this pass, then add this pass's pieces
#pragma unroll
                        for (int z = lane * 16; z < S::PM_BYTES; z += kWave * 16) {
                            *reinterpret_cast<F32x4*>(stage + S::PM_BASE + z) = F32x4{0.f, 0.f, 0.f, 0.f};
                        }
                        lds_sync();
#pragma unroll
                        for (int k = 0; k < S::NI_P; ++k) {
                            if (ppass[k] == pass) {
#pragma unroll
                                for (int e = 0; e < S::SPP; ++e) {
                                    pm[pm_at[k] + (e & 3) * kTileTokens * S::PM_STRIDE + (e >> 2)] = pv[k][e];
                                }
                            }
                        }
                        lds_sync_vm<0>();

                        // batches of 4 steps (16 union rows = 2 runs); batches past the last row are skipped
#pragma unroll
                        for (int sb = 0; sb < S::STEPS; sb += 4) {
                            if (sb * 4 < rows_here) {
                                const F32x4 a4 = *reinterpret_cast<const F32x4*>(pm_lane + sb);
                                typename ChIO::raw g_raw[4];
#pragma unroll
                                for (int ss = 0; ss < 4; ++ss) {
                                    g_raw[ss] = *reinterpret_cast<const typename ChIO::raw*>(stage + 4 * (sb + ss) * S::RB + lds_g);
                                }
#pragma unroll
                                for (int ss = 0; ss < 4; ++ss) {
                                    float g[S::ECH];
                                    ChIO::unpack(g_raw[ss], g);
#pragma unroll
                                    for (int e = 0; e < S::ECH; ++e) {
                                        d[e] = mfma_16x16x4(a4[ss], g[e], d[e]);
                                    }
                                }
                            }
                        }
                    }
                    store_head(h, d, 0, nt, true);
#pragma unroll
                    for (int k = 0; k < S::NI_P; ++k) cur[k] = nxt[k];
                }
                return;
            }
        }
    }

    // shared list: one pass that serves all tokens; otherwise one pass per token that keeps its row
    const int passes = shared_list ? 1 : nt;
    for (int pass = 0; pass < passes; ++pass) {
        const int tok_lo = shared_list ? 0 : pass;
        const int tok_hi = shared_list ? nt : pass + 1;
        if (FAST && pass > 0) {  // the p slots hold the last heads of the previous pass
            __syncthreads();
            fetch_p(0, 0, M, 0);
            if (H > 1) fetch_p(1, 0, M, 1);
        }
        // FAST: one chunk; the byte offsets of its rows do not depend on the head
        uint32_t g_off[S::NI_G];
        if constexpr (FAST) {
            int mine = list0[0];
            if (pass > 0) {
                const int slot = min(lane, M - 1);
                if constexpr (CLUSTERS) {
                    const int row = cid_tile[pass * (M >> 3) + (slot >> 3)] * 8 + (slot & 7);
                    mine = (unsigned)row < (unsigned)N ? row : 0;  // also catches a negative cluster number
                } else {
                    mine = (int)idx_tile[(int64_t)pass * M + slot];
                }
            }
#pragma unroll
            for (int i = 0; i < S::NI_G; ++i) {
                g_off[i] = (uint32_t)__shfl(mine, min(i * S::RPI + g_sub, M - 1)) * row_pitch + (uint32_t)(g_pos * 16);
            }
        }
        for (int h = 0; h < H; ++h) {
            const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(TR);
            F32x4 d[S::ECH];
#pragma unroll
            for (int e = 0; e < S::ECH; ++e) d[e] = F32x4{0.f, 0.f, 0.f, 0.f};
            bool stored = false;  // the 16-bit shared-list path writes its output itself

            for (int j0 = 0, ch = 0; j0 < (FAST ? 1 : M); j0 += kWave, ++ch) {
                const int mc = FAST ? M : min(kWave, M - j0);
                const int slot = min(lane, mc - 1);
                // gather: rows of this chunk -> LDS (and the p pieces when they were not prefetched)
                if constexpr (FAST) {
#pragma unroll
                    for (int i = 0; i < S::NI_G; ++i) stage_rows(rows_bh, g_off[i], stage + i * 1024);
                } else {
                    // this pass's list of the chunk
                    int mine;
                    if (pass == 0 && ch < MAXCH) {
                        mine = list0[0];
#pragma unroll
                        for (int k = 1; k < MAXCH; ++k) mine = (k == ch) ? list0[k] : mine;
                    } else {
                        mine = (int)idx_tile[(int64_t)pass * M + j0 + slot];
                    }
                    __syncthreads();  // the previous chunk's operand reads are complete
#pragma unroll
                    for (int i = 0; i < S::NI_G; ++i) {
                        const int srow = min(i * S::RPI + g_sub, mc - 1);
                        const uint32_t off = (uint32_t)__shfl(mine, srow) * row_pitch + (uint32_t)(g_pos * 16);
                        stage_rows(rows_bh, off, stage + i * 1024);
                    }
                }
                const int ps = FAST ? (h & 1) : 0;
                if (!FAST) {
                    fetch_p(h, j0, mc, 0);
                } else if (h >= 2) {
                    fetch_p(h, 0, M, ps);
                }
                __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                __syncthreads();

                if constexpr (sizeof(T) == 2 && FAST && EXACT) {
                    if (shared_list && rows_contiguous) {
                        // 16-bit data, 48 shared slots: the 16-bit matrix instructions take the operands as they
                        // lie in LDS.  A (tokens x slots) is a p piece: 8 consecutive slots of a token.  B (slots
                        // x 16 channels) needs, per lane, consecutive slots of one channel — a column of the
                        // row-major gathered rows: `ds_read_b64_tr_b16` delivers it (lane r of a group of 16 points
                        // at 4 channels of slot r / 4; lane n receives channel n of the 4 slots).  One 16x16x32
                        // step covers slots 0..31, a second one slots 32..47 in the lower half of each lane's k
                        // values (upper half zero: both steps are the same instruction, so the accumulator chain
                        // is one the hardware orders by itself); products of 16-bit values are exact in fp32 and
                        // the sums are fp32.
                        typedef short S4 __attribute__((ext_vector_type(4)));
                        typedef __attribute__((address_space(3))) S4* LdsS4;
                        constexpr int CBN = C / 16;
                        const char* p_tok = stage + S::P_BASE + ps * S::P_SLOT_BYTES + (n & 7) * 16;
                        const Piece a32 = *reinterpret_cast<const Piece*>(p_tok + kq * kTileTokens * 16);
                        const U32x2 a16 =
                            *reinterpret_cast<const U32x2*>(p_tok + (4 + (kq >> 1)) * kTileTokens * 16 + (kq & 1) * 8);
                        const char* col = stage + (n >> 2) * S::RB + (n & 3) * 8;  // slot n / 4 of a group of 4, 4 channels
                        F32x4 dh[CBN];
#pragma unroll
                        for (int cb = 0; cb < CBN; ++cb) {
                            const char* cbp = col + cb * 32;
                            const S4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(cbp + (8 * kq) * S::RB));
                            const S4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(cbp + (8 * kq + 4) * S::RB));
                            const S4 b2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS4)(cbp + (32 + 4 * kq) * S::RB));
                            const U32x2 lo = __builtin_bit_cast(U32x2, b0), hi = __builtin_bit_cast(U32x2, b1);
                            const Piece b32 = Piece{lo[0], lo[1], hi[0], hi[1]};
                            dh[cb] = tile_mfma<T>(a32, b32, F32x4{0.f, 0.f, 0.f, 0.f});
                            const U32x2 t2 = __builtin_bit_cast(U32x2, b2);
                            dh[cb] = tile_mfma<T>(Piece{a16[0], a16[1], 0u, 0u}, Piece{t2[0], t2[1], 0u, 0u}, dh[cb]);
                        }
                        // lane (n, kq) holds tokens 4*kq + i of channel 16*cb + n: row-major chunk in LDS, then
                        // full-width stores
                        __syncthreads();
                        if (kq < 2) {
#pragma unroll
                            for (int cb = 0; cb < CBN; ++cb) {
#pragma unroll
                                for (int i = 0; i < 4; ++i) {
                                    reinterpret_cast<T*>(stage)[(4 * kq + i) * C + 16 * cb + n] = from_acc<T>(dh[cb][i]);
                                }
                            }
                        }
                        __syncthreads();
                        constexpr int NO = (kTileTokens * S::RB + 1023) / 1024;
                        Piece o[NO];
#pragma unroll
                        for (int i = 0; i < NO; ++i) {
                            o[i] = *reinterpret_cast<const Piece*>(stage + min(i * 1024 + lane * 16, S::G_BYTES - 16));
                        }
                        __syncthreads();
                        char* out_h =
                            reinterpret_cast<char*>(out + (int64_t)b * os.b + (int64_t)(h0 + h) * os.h + (int64_t)i0 * os.n);
                        const int chunk_bytes = nt * S::RB;
#pragma unroll
                        for (int i = 0; i < NO; ++i) {
                            const int off = i * 1024 + lane * 16;
                            if (off < chunk_bytes) store_streaming(reinterpret_cast<Piece*>(out_h + off), o[i]);
                        }
                        stored = true;
                        continue;
                    }
                }

                // steps of 4 slots, taken one p piece at a time: all LDS reads of a batch of pieces (8 steps) are
                // issued before its MFMAs so that their latency is paid once per batch, not once per step.
                // No branches: when the list can end inside the chunk (!EXACT) the operands of the
                // missing slots are replaced by zeros.
                constexpr int NPIECE = S::STEPS / S::STEPS_PER_PIECE;
                constexpr int BATCH = 8 / S::STEPS_PER_PIECE;  // pieces per batch = 8 steps
                const char* p_lds = stage + S::P_BASE + ps * S::P_SLOT_BYTES + lds_p;
#pragma unroll
                for (int sb = 0; sb < NPIECE; sb += BATCH) {
                    // the lane's A operand of a step is one element of a p piece: element kq of the step's 4 slots,
                    // read from LDS on its own (no 16-byte read to unpack and select from)
                    T p_one[BATCH * S::STEPS_PER_PIECE];
                    typename ChIO::raw g_raw[BATCH * S::STEPS_PER_PIECE];
#pragma unroll
                    for (int q = 0; q < BATCH; ++q) {
                        if (sb + q < NPIECE) {
#pragma unroll
                            for (int ss = 0; ss < S::STEPS_PER_PIECE; ++ss) {
                                const int s = (sb + q) * S::STEPS_PER_PIECE + ss;
                                p_one[q * S::STEPS_PER_PIECE + ss] = *reinterpret_cast<const T*>(
                                    p_lds + (sb + q) * kTileTokens * 16 + (4 * ss + kq) * (int)sizeof(T));
                                g_raw[q * S::STEPS_PER_PIECE + ss] =
                                    *reinterpret_cast<const typename ChIO::raw*>(stage + 4 * s * S::RB + lds_g);
                            }
                        }
                    }
#pragma unroll
                    for (int q = 0; q < BATCH; ++q) {
                        if (sb + q < NPIECE) {
#pragma unroll
                            for (int ss = 0; ss < S::STEPS_PER_PIECE; ++ss) {
                                const int s = (sb + q) * S::STEPS_PER_PIECE + ss;
                                float aop = to_acc(p_one[q * S::STEPS_PER_PIECE + ss]);
                                float g[S::ECH];
                                ChIO::unpack(g_raw[q * S::STEPS_PER_PIECE + ss], g);
                                if (!EXACT) {
                                    const bool live = 4 * s < mc;  // mc is a multiple of 4: a step is whole or missing
                                    aop = live ? aop : 0.f;
#pragma unroll
                                    for (int e = 0; e < S::ECH; ++e) g[e] = live ? g[e] : 0.f;
                                }
#pragma unroll
                                for (int e = 0; e < S::ECH; ++e) {
                                    d[e] = mfma_16x16x4(aop, g[e], d[e]);
                                }
                            }
                        }
                    }
                }
            }

            if (!stored) store_head(h, d, tok_lo, tok_hi, shared_list);
        }
    }
}

// One thread per output element; any dtype, any head dim, any list length, any alignment.
template <typename T>
__global__ __launch_bounds__(256) void gather_sum_elem_kernel(const T* __restrict__ p, const T* __restrict__ rows,
                                                              const int64_t* __restrict__ idx, T* __restrict__ out,
                                                              int B, int H, int N, int C, int M, clusten_strides rs,
                                                              clusten_strides os) {
    const int64_t total = (int64_t)B * H * N * C;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(o % C);
        const int64_t q1 = o / C;
        const int i = (int)(q1 % N);
        const int64_t q2 = q1 / N;
        const int h = (int)(q2 % H);
        const int b = (int)(q2 / H);
        const int64_t* list = idx + ((int64_t)b * N + i) * M;
        const T* prow = p + (((int64_t)b * H + h) * N + i) * M;
        const T* base = rows + b * rs.b + h * rs.h + c;
        typename Acc<T>::type acc = 0;
        for (int j = 0; j < M; ++j) acc += to_acc(prow[j]) * to_acc(base[list[j] * rs.n]);
        out[b * os.b + h * os.h + i * os.n + c] = from_acc<T>(acc);
    }
}

template <typename T, int C, int Q, bool FAST, bool EXACT, bool CLUSTERS = false, typename TR = T>
int launch_tile_q(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                  clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int groups = head_groups_for(total, s.H);
    const int grid = xcd_grid(total * groups);
    hipLaunchKernelGGL((gather_sum_tile_kernel<T, C, Q, FAST, EXACT, CLUSTERS, TR>), dim3(grid), dim3(kWave), 0, stream,
                       static_cast<const T*>(p), static_cast<const TR*>(rows), idx, static_cast<T*>(out), s.H, s.N,
                       s.M, rs, os, tiles_per_batch, total, groups);
    return launch_status();
}

template <typename T, int C, typename TR = T>
int launch_tile(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out, clusten_strides os,
                const clusten_attn_shape& s, hipStream_t stream) {
    // 48 slots is the neighbourhood size of every 224x224 model: three slot blocks, no range checks
    if (s.M == 48) return launch_tile_q<T, C, 3, true, true, false, TR>(p, rows, rs, idx, out, os, s, stream);
    if (s.M <= 64) return launch_tile_q<T, C, 4, true, false, false, TR>(p, rows, rs, idx, out, os, s, stream);
    return launch_tile_q<T, C, 4, false, false, false, TR>(p, rows, rs, idx, out, os, s, stream);
}

template <typename T>
int launch_elem(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out, clusten_strides os,
                const clusten_attn_shape& s, hipStream_t stream) {
    const int64_t total = (int64_t)s.B * s.H * s.N * s.C;
    const int64_t want = (total + 255) / 256;
    const int grid = (int)(want < (int64_t)1 << 20 ? want : (int64_t)1 << 20);
    hipLaunchKernelGGL((gather_sum_elem_kernel<T>), dim3(grid), dim3(256), 0, stream, static_cast<const T*>(p),
                       static_cast<const T*>(rows), idx, static_cast<T*>(out), s.B, s.H, s.N, s.C, s.M, rs, os);
    return launch_status();
}

// Lists given as cluster numbers (see CLUSTERS above): `cluster_idx` is (B, N, M/8) int32 for M <= 64 (clusters of 8)
// and (B, N, M/L) for longer lists, L = runs_length_for(M) the cluster size (24 for the 144 slots of the 384 x 384
// models).  Only the tile kernels take this format: head dim 16/32/64, 16-byte aligned rows.
template <typename T>
int gather_sum_clusters_typed(const void* p, const void* rows, clusten_strides rs, const int32_t* cluster_idx, void* out,
                              clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    const bool quads_ok = ((int64_t)s.M * sizeof(T)) % 16 == 0 && aligned16(p) && rows_aligned16(rows, rs, sizeof(T)) &&
                          rows_aligned16(out, os, sizeof(T)) && slice_fits_int32(rs, s.H, s.N, s.C);
    if (!quads_ok) return CLUSTEN_ERR_UNALIGNED;
    if (const int L = runs_length_for(s.M); L != 0 && runs_head_dim_ok<T>(s.C)) {
        if (L == kRun24) return launch_gather_sum_runs24<T>(p, rows, rs, nullptr, out, os, s, stream, cluster_idx);
        return launch_gather_sum_runs<T>(p, rows, rs, nullptr, out, os, s, L, stream, cluster_idx);
    }
    if (s.M % 8 != 0 || s.M > 64) return CLUSTEN_ERR_BAD_DIMS;
    const int64_t* idx = reinterpret_cast<const int64_t*>(cluster_idx);
    switch (s.C) {
        case 16:
            return s.M == 48 ? launch_tile_q<T, 16, 3, true, true, true>(p, rows, rs, idx, out, os, s, stream)
                             : launch_tile_q<T, 16, 4, true, false, true>(p, rows, rs, idx, out, os, s, stream);
        case 32:
            return s.M == 48 ? launch_tile_q<T, 32, 3, true, true, true>(p, rows, rs, idx, out, os, s, stream)
                             : launch_tile_q<T, 32, 4, true, false, true>(p, rows, rs, idx, out, os, s, stream);
        case 64:
            return s.M == 48 ? launch_tile_q<T, 64, 3, true, true, true>(p, rows, rs, idx, out, os, s, stream)
                             : launch_tile_q<T, 64, 4, true, false, true>(p, rows, rs, idx, out, os, s, stream);
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
}

template <typename T>
int gather_sum_typed(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out, clusten_strides os,
                 const clusten_attn_shape& s, hipStream_t stream) {
    // p rows are whole 16-byte pieces; gathered rows and out rows are read / written in 16-byte (or, for the
    // strided store, C/16-element) groups
    const bool quads_ok = ((int64_t)s.M * sizeof(T)) % 16 == 0 && aligned16(p) && rows_aligned16(rows, rs, sizeof(T)) &&
                          rows_aligned16(out, os, sizeof(T)) && slice_fits_int32(rs, s.H, s.N, s.C);
    if (quads_ok) {
        // long lists made of long runs (the 384 x 384 models: 6 clusters of 24 tokens)
        if (const int L = runs_length_for(s.M); L != 0 && runs_head_dim_ok<T>(s.C)) {
            if (L == kRun24) return launch_gather_sum_runs24<T>(p, rows, rs, idx, out, os, s, stream);
            return launch_gather_sum_runs<T>(p, rows, rs, idx, out, os, s, L, stream);
        }
        switch (s.C) {
            case 16: return launch_tile<T, 16>(p, rows, rs, idx, out, os, s, stream);
            case 32: return launch_tile<T, 32>(p, rows, rs, idx, out, os, s, stream);
            case 64: return launch_tile<T, 64>(p, rows, rs, idx, out, os, s, stream);
            default: break;
        }
    }
    return launch_elem<T>(p, rows, rs, idx, out, os, s, stream);
}

// One thread per output element, rows of another storage type than p and out.
template <typename T, typename TR>
__global__ __launch_bounds__(256) void gather_sum_mixed_elem_kernel(const T* __restrict__ p, const TR* __restrict__ rows,
                                                                    const int64_t* __restrict__ idx, T* __restrict__ out,
                                                                    int B, int H, int N, int C, int M, clusten_strides rs,
                                                                    clusten_strides os) {
    const int64_t total = (int64_t)B * H * N * C;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(o % C);
        const int64_t q1 = o / C;
        const int i = (int)(q1 % N);
        const int64_t q2 = q1 / N;
        const int h = (int)(q2 % H);
        const int b = (int)(q2 / H);
        const int64_t* list = idx + ((int64_t)b * N + i) * M;
        const T* prow = p + (((int64_t)b * H + h) * N + i) * M;
        const TR* base = rows + b * rs.b + h * rs.h + c;
        float acc = 0.f;
        for (int j = 0; j < M; ++j) acc += to_acc(prow[j]) * to_acc(base[list[j] * rs.n]);
        out[b * os.b + h * os.h + i * os.n + c] = from_acc<T>(acc);
    }
}

// fp32 p and out with rows of TR = fp16 / bf16, read in place (see the TR parameter of the tile kernel).
template <typename TR>
int gather_sum_mixed_typed(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                           clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    // p rows are whole 16-byte pieces, out rows 16-byte groups, a lane's piece of a gathered row 8 bytes
    const bool rows8 = (reinterpret_cast<uintptr_t>(rows) & 7u) == 0 && (rs.b * 2) % 8 == 0 && (rs.h * 2) % 8 == 0 &&
                       (rs.n * 2) % 8 == 0;
    const bool quads_ok = ((int64_t)s.M * 4) % 16 == 0 && aligned16(p) && rows8 && rows_aligned16(out, os, 4) &&
                          slice_fits_int32(rs, s.H, s.N, s.C);
    // long lists made of long runs have kernels of their own for rows of the weights' type only: a result that equals
    // the cast-first path bit for bit needs the same kernel, so such a call is turned down (the caller casts)
    if (runs_length_for(s.M) != 0 && runs_head_dim_ok<float>(s.C)) return CLUSTEN_ERR_BAD_DIMS;
    if (quads_ok) {
        switch (s.C) {
            case 16: return launch_tile<float, 16, TR>(p, rows, rs, idx, out, os, s, stream);
            case 32: return launch_tile<float, 32, TR>(p, rows, rs, idx, out, os, s, stream);
            case 64: return launch_tile<float, 64, TR>(p, rows, rs, idx, out, os, s, stream);
            default: break;
        }
    }
    const int64_t total = (int64_t)s.B * s.H * s.N * s.C;
    const int64_t want = (total + 255) / 256;
    const int grid = (int)(want < (int64_t)1 << 20 ? want : (int64_t)1 << 20);
    hipLaunchKernelGGL((gather_sum_mixed_elem_kernel<float, TR>), dim3(grid), dim3(256), 0, stream,
                       static_cast<const float*>(p), static_cast<const TR*>(rows), idx, static_cast<float*>(out), s.B, s.H,
                       s.N, s.C, s.M, rs, os);
    return launch_status();
}

}  // namespace clusten
