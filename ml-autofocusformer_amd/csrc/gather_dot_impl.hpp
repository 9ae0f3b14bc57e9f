// gather_dot: out[b,h,i,j] = sum_c a[b,h,i,c] * rows[b,h,idx[b,i,j],c]
//
// This is the CLUSTEN QK forward (a = query, rows = key; reference kernel
// clusten/src/clustenqk_cuda_kernel.cu:18-49) and the d_attn half of the AV backward
// (a = d_feat, rows = value; clusten/src/clustenav_cuda_kernel.cu:129-160).
//
// Work decomposition.  One wave owns a tile of 8 consecutive tokens of one batch element and
// walks all heads, so the int64 neighbour lists of the tile are read from HBM exactly once.
// Per head the tile is a small matrix product  D[slot][token] = G[slot][c] * A^T[c][token]  with
// G the gathered rows, and it runs on the matrix cores as fp32 MFMA 16x16x4 blocks.
//
// Data path per head:
//   0. lists: the tile's 8 lists are one contiguous block; it travels by LDS-direct load and is compared
//      from LDS (FAST kernels) — 1 KiB accesses instead of 8-byte loads per lane.
//   1. gather: `global_load_lds_dwordx4` moves the rows from HBM/L2 straight into LDS, 16 bytes per
//      lane, consecutive lanes on consecutive pieces of one row (row-coalesced: a wave access covers
//      64/pieces-per-row whole rows).  No VGPRs are held while the data travels, so the bytes a CU
//      keeps in flight are bounded by its LDS, not by its register file.  The 8 a-rows of the tile
//      take the same path.
//   2. operands: lane (r = lane % 16, kq = lane / 16) reads the quarter [kq*C/4, (kq+1)*C/4) of row r
//      of every 16-slot block from LDS with 16-byte reads: the registers it fills are the MFMA A
//      operands (channel e of the quarter is the k-index kq of MFMA step e), and the same quarter of
//      a-row r % 8 gives the B operands.  The piece index is XOR-swizzled with the row number on
//      the way in so that these reads are free of bank conflicts.
//   3. the D block leaves lane (r, kq) with slots 4*kq..4*kq+3 of token r.  The output of one
//      (tile, head) is a single contiguous chunk of 8*M elements, so the blocks are laid out
//      row-major in LDS and leave with full-width 16-byte stores (lists of up to 64 slots).
//      On the shared-list path the chunk is laid out in the LDS slot the head's a-rows came from, the rows of
//      the next head are requested as soon as this head's operands are in registers, and the wait for them
//      leaves this head's stores in flight (LDS-only ordering between the steps, see lds_sync()).
// One short-lived one-wave workgroup per tile; the latency of its dependent chain (lists, rows,
// product, store) is hidden by the ~16 other waves resident on the CU.
//
//   shared-list path — all tokens of the tile carry the same list (true for every tile of a
//     cluster-ordered token sequence whose cluster shares its neighbourhood): one gather and one
//     set of MFMAs per head serve the 8 tokens.
//   union path — lists that differ but are made of runs of 8 slots of which the tile's tokens share most
//     (the neighbourhoods of a cluster-ordered sequence: a run is the 8 members of one cluster): every
//     distinct run is gathered and multiplied once per head, the scores go to an LDS matrix from which
//     each token picks its own slots.
//   per-token path — any other tile: the gather and the MFMAs are repeated per token and only that
//     token's column is kept.  Exact for arbitrary indices (duplicates, any order), only slower.
//
// fp32 data runs as fp32 MFMA 16x16x4; fp16 / bf16 data goes through the 16-bit matrix instructions as it came
// from memory (16x16x32, or 16x16x16 for head dim 16): their products are exact in fp32 and all sums are fp32.
// Rows whose start is not 16-byte aligned, head dims other than 16/32/64 and fp64 take the
// element-per-thread kernel at the bottom of the file.
//
// This header holds the templates; gather_dot_{f32,f16,bf16}.hip and gather_dot_clusters_{...}.hip (lists
// given as cluster numbers) instantiate them per storage type so that the translation units build in
// parallel, gather_dot.hip holds the dtype dispatch.
#pragma once

#include "launch.hpp"
#include "mfma.hpp"
#include "gather_runs_impl.hpp"

namespace clusten {

// A tile's query rows are read once and loaded with the non-temporal hint, which keeps them from displacing the
// gathered rows and the lists in the caches.  The lists are loaded plainly: the launch that follows in an attention
// layer (attention weights times values) reads the same lists and finds part of them in the memory-side cache.
// Measured at B=128 H=2 N=3136 M=48 C=32 fp32, this kernel / the weights-times-values kernel after it: no hints
// 105.9 / 108.1 us; rows hinted 102.8 / 101.4 (with that kernel's weights hinted); rows and lists 102.1 / 111.1.
constexpr bool kDotHintLists = false;
constexpr bool kDotHintRows = true;

// Geometry of the staging buffer in LDS: rows of RB bytes, filled 1 KiB (one wave access) at a time.
//   [0, G_BYTES)            gathered rows of one head (16*Q rows); reused to turn the D blocks into
//                           the row-major output chunk once the operands are in registers
//   [A_BASE, +2*OA_BYTES)   a-rows of two heads (slot h % 2); on the shared-list path of the FAST kernels a slot then
//                           takes the head's output chunk, so that the row area is free for the next head's rows
//   union path only (FAST kernels):
//   [0, G_BYTES)            rows of 2*Q distinct runs per pass; reused for the score matrix of the pass
//   [ULIST_BASE, +512)      row indices of up to U_MAX distinct runs, 8 per run
//   [USLOT_BASE, +256)      distinct-run number of each of the tile's runs
template <typename T, int C, int Q, bool UNION>
struct Staging {
    static constexpr int RB = C * (int)sizeof(T);               // bytes per row
    static constexpr int PPR = RB / 16;                         // 16-byte pieces per row
    static constexpr int RPI = kWave / PPR;                     // rows per wave access
    static constexpr int NI_G = (16 * Q + RPI - 1) / RPI;       // accesses for the gathered rows of a chunk
    static constexpr int NI_A = (kTileTokens + RPI - 1) / RPI;  // accesses for the tile's a-rows
    static constexpr int OUT_BYTES = kTileTokens * 16 * Q * (int)sizeof(T);  // one (tile, head) output chunk
    static constexpr int QU = Q;                                // slot blocks per pass of the union path
    static constexpr int NI_U = NI_G;                           // accesses for the rows of a union pass
    static constexpr int U_MAX = 16;                            // distinct runs the union path holds
    static constexpr int SROW = 16 * QU + 4;                    // floats per token row of the score matrix
    static constexpr int U_BYTES = UNION ? kTileTokens * SROW * 4 : 0;
    static constexpr int G_PLAIN = NI_G * 1024 > OUT_BYTES ? NI_G * 1024 : (OUT_BYTES + 1023) / 1024 * 1024;
    static constexpr int NI_L = Q;                              // accesses for the tile's lists (8 x 16*Q x 8 bytes)
    static constexpr int G_NEED = UNION ? (U_BYTES > NI_L * 1024 ? U_BYTES : NI_L * 1024) : 0;
    static constexpr int G_BYTES = G_PLAIN > G_NEED ? G_PLAIN : (G_NEED + 1023) / 1024 * 1024;
    static constexpr int A_BASE = G_BYTES;
    static constexpr int A_SLOT_BYTES = NI_A * 1024;
    static constexpr int OUT_PIECES = (OUT_BYTES + 15) / 16 * 16;
    static constexpr int OA_BYTES = A_SLOT_BYTES > OUT_PIECES ? A_SLOT_BYTES : OUT_PIECES;  // a-rows, then output chunk
    static constexpr int ULIST_BASE = A_BASE + 2 * OA_BYTES;
    static constexpr int USLOT_BASE = ULIST_BASE + (UNION ? U_MAX * 8 * 4 : 0);
    // union path: the score matrix of a pass lives outside the row area, so that the rows of the next pass can be
    // requested while it is picked from: in the a-row slot of the head where that is large enough (fp32 data: the
    // scores of a pass are as many bytes as the head's output chunk), else in an area of its own
    static constexpr bool SCORES_IN_A = OA_BYTES >= kTileTokens * 16 * QU * 4;
    static constexpr int SSTR = SCORES_IN_A ? 16 * QU : SROW;  // floats per token row of the score matrix
    static constexpr int SCORE_BASE = SCORES_IN_A ? A_BASE : USLOT_BASE + (UNION ? kWave * 4 : 0);
    static constexpr int BYTES = USLOT_BASE + (UNION ? kWave * 4 : 0) + (UNION && !SCORES_IN_A ? kTileTokens * SROW * 4 : 0);
    static constexpr int EL = C / 4;                            // channels per lane (a quarter row)
    static constexpr int QB = RB / 4;                           // bytes per lane
    static constexpr int UNIT = QB < 16 ? QB : 16;              // bytes per LDS read
    static constexpr int NU = QB / UNIT;                        // LDS reads per quarter row
    static constexpr int VEC = UNIT / (int)sizeof(T);           // elements per LDS read
    static_assert(RB >= 32 && kWave % PPR == 0, "row size");

    // XOR swizzle of the piece index: rows r, r+1, ... of a block land in different bank groups
    static __device__ __forceinline__ int swz(int row) { return ((row & 7) ^ ((row >> 3) & 1)) & (PPR - 1); }
};

// FAST = the list has at most 64 slots and a multiple of 4 of them: one chunk, and every access to
// an out row is a whole aligned 16-byte group.  Otherwise lists go 64 slots at a time and the last
// group of a row may be stored element by element.
// CLUSTERS (FAST kernels only) = the lists arrive as int32 cluster numbers, M/8 per token: slot j of a token is row
// 8*g + j%8 of its cluster g = number j/8 (row 0 where that is past the last row, as the padded last cluster of a
// cluster-ordered sequence is listed); `idx` then points to (B, N, M/8) int32.
template <typename T, int C, int Q, bool FAST, bool CLUSTERS = false>
__global__ __launch_bounds__(kWave) void gather_dot_tile_kernel(const T* __restrict__ a, const T* __restrict__ rows,
                                                                const int64_t* __restrict__ idx,
                                                                T* __restrict__ out, int H_all, int N, int M,
                                                                clusten_strides as, clusten_strides rs,
                                                                int tiles_per_batch, int total_tiles, int head_groups) {
    typedef Staging<T, C, Q, FAST> S;
    typedef VecIO<T, S::VEC> RunIO;
    typedef VecIO<T, 4> OutIO;
    static_assert(C % 16 == 0, "a lane holds a quarter of a row in whole 4-element groups");
    static_assert(Q >= 1 && Q <= 4, "a chunk holds 16, 32, 48 or 64 neighbour slots");

    __shared__ __attribute__((aligned(1024))) char stage[S::BYTES];

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
    const int r = lane & 15;   // MFMA row of the A operand / column of the B operand
    const int kq = lane >> 4;  // MFMA k index; also the quarter of the row this lane holds
    // gather side: in access i this lane moves one piece of staging row i*RPI + lane/PPR
    const int g_sub = lane / S::PPR;
    const int g_pos = lane % S::PPR;

    const char* rows_b = reinterpret_cast<const char*>(rows + (int64_t)b * rs.b + (int64_t)h0 * rs.h);
    const char* a_tile = reinterpret_cast<const char*>(a + (int64_t)b * as.b + (int64_t)h0 * as.h + (int64_t)i0 * as.n);
    char* out_tile = reinterpret_cast<char*>(out + (((int64_t)b * H_all + h0) * N + i0) * M);
    const int64_t* idx_tile = idx + ((int64_t)b * N + i0) * M;
    const int32_t* cid_tile = reinterpret_cast<const int32_t*>(idx) + ((int64_t)b * N + i0) * (M >> 3);
    int cid = 0;  // CLUSTERS: the cluster number of run `lane` of the tile (token lane / R, run lane % R)
    const uint32_t row_pitch = (uint32_t)rs.n * sizeof(T);

    // a-rows of head h -> slot h % 2.  Staging row = token; tokens past the end of a partial tile
    // repeat its last token.  They do not depend on the lists, so the first two heads are requested
    // before the lists are even read.
    uint32_t a_off[S::NI_A];
#pragma unroll
    for (int i = 0; i < S::NI_A; ++i) {
        const int srow = i * S::RPI + g_sub;
        a_off[i] = (uint32_t)min(srow, nt - 1) * (uint32_t)as.n * sizeof(T) + (uint32_t)((g_pos ^ S::swz(srow)) * 16);
    }
    auto fetch_a = [&](int h) {
        const char* a_bh = a_tile + (int64_t)h * as.h * sizeof(T);
#pragma unroll
        for (int i = 0; i < S::NI_A; ++i) {
            CLUSTEN_LDS_DMA16_STREAM(a_bh + a_off[i], stage + S::A_BASE + (h & 1) * S::OA_BYTES + i * 1024, kDotHintRows);
        }
    };
    fetch_a(0);
    if (H > 1) fetch_a(1);

    // operand side: byte offsets of this lane's quarter rows inside the staging buffer
    int lds_g[S::NU];  // row r of slot block 0; block blk is 16 rows further
    int lds_a[S::NU];
#pragma unroll
    for (int u = 0; u < S::NU; ++u) {
        const int byte = kq * S::QB + u * S::UNIT;  // offset inside the row
        const int piece = byte / 16, within = byte % 16;
        lds_g[u] = r * S::RB + ((piece ^ S::swz(r)) * 16) + within;  // swz(16*blk + r) == swz(r)
        lds_a[u] = S::A_BASE + (r & 7) * S::RB + ((piece ^ S::swz(r & 7)) * 16) + within;
    }

    const bool vec_store = FAST || (M & 3) == 0;  // 16-byte accesses to out rows need aligned rows

    for (int j0 = 0; j0 < (FAST ? 1 : M); j0 += kWave) {
        const int mc = min(kWave, M - j0);
        const int slot = min(lane, mc - 1);  // lanes past the list repeat its last slot

        // the tile's lists: are they all the same?  (only the first is kept in registers)
        int list0;
        bool same = true;
        if constexpr (CLUSTERS) {
            const int R = M >> 3, nruns = nt * R;
            cid = cid_tile[min(lane, nruns - 1)];
            same = lane >= nruns || cid == __shfl(cid, lane % R);   // against the same run of the tile's first token
            const int row = __shfl(cid, slot >> 3) * 8 + (slot & 7);
            list0 = (unsigned)row < (unsigned)N ? row : 0;  // also catches a negative cluster number
        } else if constexpr (FAST) {
            // the nt lists are one contiguous block of nt*M*8 bytes: it travels by LDS-direct load in 1 KiB
            // accesses (a third of the vector-memory instructions that 8-byte loads per lane need) and is
            // compared from LDS
            const int list_bytes = nt * M * 8;
            const char* idx_bytes = reinterpret_cast<const char*>(idx_tile);
#pragma unroll
            for (int i = 0; i < S::NI_L; ++i) {
                if (i * 1024 < list_bytes) {
                    CLUSTEN_LDS_DMA16_STREAM(idx_bytes + min(i * 1024 + lane * 16, list_bytes - 16), stage + i * 1024, kDotHintLists);
                }
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            __syncthreads();
            int64_t wide[kTileTokens];
#pragma unroll
            for (int t = 0; t < kTileTokens; ++t) {
                wide[t] = *reinterpret_cast<const int64_t*>(stage + (min(t, nt - 1) * M + slot) * 8);
            }
#pragma unroll
            for (int t = 1; t < kTileTokens; ++t) same = same && (wide[t] == wide[0]);
            list0 = (int)wide[0];
        } else {
            int64_t wide[kTileTokens];
#pragma unroll
            for (int t = 0; t < kTileTokens; ++t) wide[t] = idx_tile[(int64_t)min(t, nt - 1) * M + j0 + slot];
#pragma unroll
            for (int t = 1; t < kTileTokens; ++t) same = same && (wide[t] == wide[0]);
            list0 = (int)wide[0];
        }
        const bool shared_list = __all(same ? 1 : 0) != 0;

        if constexpr (FAST) {
            if (!shared_list && (M & 7) == 0) {
                // ---- union path: lists made of runs of 8 slots, many of them common to several tokens ----
                // (the neighbourhoods of a cluster-ordered sequence: a run is the 8 members of one cluster, and
                // the tokens of a tile pick their clusters from the same dozen.)  Every distinct run is gathered
                // and multiplied once per head; each token then picks its own slots from the score matrix.
                constexpr int QU = S::QU;
                constexpr int UROWS = 16 * QU;   // union rows per pass
                const int R = M >> 3;             // runs per token
                const int nruns = nt * R;         // <= 64: lane rho owns run rho = token * R + run
                int v[8];
                if constexpr (CLUSTERS) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) v[t] = (unsigned)(cid * 8 + t) < (unsigned)N ? cid * 8 + t : 0;
                } else {
                    const int64_t* p = reinterpret_cast<const int64_t*>(stage) + min(lane, nruns - 1) * 8;  // lists in LDS
#pragma unroll
                    for (int t = 0; t < 8; ++t) v[t] = (int)p[t];
                }
                __syncthreads();  // the lists are in registers: the staging buffer is free for the gathers
                // 8 consecutive rows, or the short last cluster of the sequence followed by the row 0 its pad slots hold:
                // either way the first row tells the other seven
                const int own = ((N & 7) != 0 && v[0] == N - (N & 7)) ? (N & 7) : 8;
                bool regular = true;
#pragma unroll
                for (int t = 1; t < 8; ++t) regular = regular && (v[t] == (t < own ? v[0] + t : 0));
                const int key = regular ? v[0] : ~lane;  // other runs never merge

                // number the distinct keys in order of first appearance
                uint64_t remaining = nruns >= 64 ? ~0ull : ((1ull << nruns) - 1);
                int uslot = 0, U = 0;
                bool first = false;
                while (remaining != 0 && U < S::U_MAX) {
                    const int s = __builtin_ctzll(remaining);
                    const int ks = __builtin_amdgcn_readlane(key, s);
                    const bool hit = key == ks;
                    const uint64_t match = __ballot(hit) & remaining;
                    if (hit) uslot = U;
                    first = first || lane == s;
                    remaining &= ~match;
                    ++U;
                }
                if (remaining == 0) {  // at most U_MAX distinct runs; tiles with more take the per-token passes
                int* ulist = reinterpret_cast<int*>(stage + S::ULIST_BASE);
                int* uslots = reinterpret_cast<int*>(stage + S::USLOT_BASE);
                if (first) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) ulist[uslot * 8 + t] = v[t];
                }
                if (lane < nruns) uslots[lane] = uslot;
                __syncthreads();

                // this lane's share of the output chunk: groups of 4 consecutive elements (inside one run)
                constexpr int NQD = (kTileTokens * 16 * Q / 4 + kWave - 1) / kWave;
                int sidx[NQD], qtok[NQD];
                bool qvalid[NQD];
#pragma unroll
                for (int k = 0; k < NQD; ++k) {
                    const int e = 4 * (lane + kWave * k);
                    qvalid[k] = e < nt * M;
                    const int ec = qvalid[k] ? e : 0;
                    const int i = ec / M, j = ec - i * M;
                    qtok[k] = i;
                    sidx[k] = uslots[i * R + (j >> 3)] * 8 + (j & 7);
                }

                const int total_rows = 8 * U;
                // Passes of UROWS union rows, heads outside.  The rows of the next pass (of this head or the next) are
                // requested as soon as the operands of the current one are in registers, so they travel while the
                // current pass is multiplied and picked; the stores of a head are issued after the first request of
                // the next head, and the wait for those rows leaves them in flight.
                auto gather_pass = [&](int h, int base) {
                    const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(T);
                    const int rows_here = min(UROWS, total_rows - base);
#pragma unroll
                    for (int i = 0; i < S::NI_U; ++i) {
                        if (i * S::RPI < rows_here) {
                            const int srow = i * S::RPI + g_sub;
                            const uint32_t urow = (uint32_t)ulist[min(base + srow, total_rows - 1)];
                            CLUSTEN_LDS_DMA16(rows_bh + (urow * row_pitch + (uint32_t)((g_pos ^ S::swz(srow)) * 16)),
                                              stage + i * 1024);
                        }
                    }
                };
                // store instructions of a head that have an active lane: all of them on a full tile
                bool all_stores = true;
#pragma unroll
                for (int k = 0; k < NQD; ++k) all_stores = all_stores && (4 * kWave * k < nt * M);
                gather_pass(0, 0);
                for (int h = 0; h < H; ++h) {
                    F32x4 val[NQD];
#pragma unroll
                    for (int k = 0; k < NQD; ++k) val[k] = F32x4{0.f, 0.f, 0.f, 0.f};
                    typename RunIO::raw a_raw[S::NU];
                    char* score = stage + S::SCORE_BASE + (S::SCORES_IN_A ? (h & 1) * S::OA_BYTES : 0);
                    for (int base = 0; base < total_rows; base += UROWS) {
                        const int rows_here = min(UROWS, total_rows - base);
                        if (base == 0 && h > 0 && all_stores) {
                            lds_sync_vm<NQD>();  // everything but the stores of the previous head
                        } else {
                            lds_sync_vm<0>();
                        }
                        typename RunIO::raw g_raw[QU][S::NU];
#pragma unroll
                        for (int u = 0; u < S::NU; ++u) {
#pragma unroll
                            for (int blk = 0; blk < QU; ++blk) {
                                if (blk * 16 < rows_here) {
                                    g_raw[blk][u] = *reinterpret_cast<const typename RunIO::raw*>(stage + lds_g[u] +
                                                                                                  blk * 16 * S::RB);
                                }
                            }
                            if (base == 0) {
                                a_raw[u] = *reinterpret_cast<const typename RunIO::raw*>(stage + lds_a[u] +
                                                                                         (h & 1) * S::OA_BYTES);
                            }
                        }
                        lds_sync();  // operands are in registers: the row area is free for the next pass
                        const bool last = base + UROWS >= total_rows;
                        if (base == 0 && h >= 1 && h + 1 < H) fetch_a(h + 1);  // into the slot head h-1 has left
                        if (!last) {
                            gather_pass(h, base + UROWS);
                        } else if (h + 1 < H) {
                            gather_pass(h + 1, 0);
                        }
#pragma unroll
                        for (int blk = 0; blk < QU; ++blk) {
                            if (blk * 16 < rows_here) {
                                F32x4 d = F32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                                for (int u = 0; u < S::NU; ++u) d = tile_mfma<T>(g_raw[blk][u], a_raw[u], d);
                                // lane (r, kq): union rows 16*blk + 4*kq .. +3 of token r
                                if (r < kTileTokens) {
                                    *reinterpret_cast<F32x4*>(score + (r * S::SSTR + 16 * blk + 4 * kq) * 4) = d;
                                }
                            }
                        }
                        lds_sync();
#pragma unroll
                        for (int k = 0; k < NQD; ++k) {
                            const int sl = sidx[k] - base;
                            if (sl >= 0 && sl < UROWS) {
                                val[k] = *reinterpret_cast<const F32x4*>(score + (qtok[k] * S::SSTR + sl) * 4);
                            }
                        }
                    }
                    char* out_h = out_tile + (int64_t)h * N * M * sizeof(T);
#pragma unroll
                    for (int k = 0; k < NQD; ++k) {
                        if (qvalid[k]) {
                            float o[4] = {val[k][0], val[k][1], val[k][2], val[k][3]};
                            store_streaming(reinterpret_cast<typename OutIO::raw*>(out_h + (lane + kWave * k) * 4 * (int)sizeof(T)),
                                            OutIO::pack(o));
                        }
                    }
                }
                return;
                }
            }
        }

        if (FAST) __syncthreads();  // the list block has been read: the staging buffer is free for the gathers

        if constexpr (FAST) {
            if (shared_list) {
                // ---- shared list: one gather and one set of MFMAs per head serve the 8 tokens; heads pipelined ----
                // The rows of head h+1 are requested as soon as the operands of head h are in registers; the output
                // chunk of head h is laid out in the slot its a-rows came from, so the row area stays free, and the
                // wait for the rows of head h+1 leaves the stores of head h in flight.
                uint32_t g_off[S::NI_G];
#pragma unroll
                for (int i = 0; i < S::NI_G; ++i) {
                    const int srow = i * S::RPI + g_sub;
                    g_off[i] = (uint32_t)__shfl(list0, min(srow, mc - 1)) * row_pitch + (uint32_t)((g_pos ^ S::swz(srow)) * 16);
                }
                auto gather = [&](int h) {
                    const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(T);
#pragma unroll
                    for (int i = 0; i < S::NI_G; ++i) CLUSTEN_LDS_DMA16(rows_bh + g_off[i], stage + i * 1024);
                };
                constexpr int NO = (S::OUT_BYTES + 1023) / 1024;  // store instructions per head
                const int chunk_bytes = nt * M * (int)sizeof(T);
                const bool all_stores = (NO - 1) * 1024 < chunk_bytes;  // each of them has an active lane
                gather(0);
                for (int h = 0; h < H; ++h) {
                    if (h == 0 || !all_stores) {
                        lds_sync_vm<0>();
                    } else {
                        lds_sync_vm<NO>();  // everything but the stores of the previous head
                    }
                    typename RunIO::raw g_raw[Q][S::NU];
                    typename RunIO::raw a_raw[S::NU];
#pragma unroll
                    for (int u = 0; u < S::NU; ++u) {
#pragma unroll
                        for (int blk = 0; blk < Q; ++blk) {
                            g_raw[blk][u] =
                                *reinterpret_cast<const typename RunIO::raw*>(stage + lds_g[u] + blk * 16 * S::RB);
                        }
                        a_raw[u] = *reinterpret_cast<const typename RunIO::raw*>(stage + lds_a[u] + (h & 1) * S::OA_BYTES);
                    }
                    lds_sync();  // operands are in registers: the row area and this head's a-row slot are free
                    if (h + 1 < H) {
                        gather(h + 1);
                        if (h + 1 >= 2) fetch_a(h + 1);
                    }
                    F32x4 d[Q];
#pragma unroll
                    for (int blk = 0; blk < Q; ++blk) {
                        d[blk] = F32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int u = 0; u < S::NU; ++u) d[blk] = tile_mfma<T>(g_raw[blk][u], a_raw[u], d[blk]);
                    }
                    // lane (r, kq) holds slots 16*blk + 4*kq .. +3 of token r: the (tile, head) output is one contiguous
                    // chunk of nt*M elements; it is laid out row-major in LDS and leaves with full-width 16-byte stores
                    char* chunk = stage + S::A_BASE + (h & 1) * S::OA_BYTES;
                    if (r < nt) {
#pragma unroll
                        for (int blk = 0; blk < Q; ++blk) {
                            const int s0 = 16 * blk + 4 * kq;
                            float v[4] = {d[blk][0], d[blk][1], d[blk][2], d[blk][3]};
                            if (s0 < mc) {
                                *reinterpret_cast<typename OutIO::raw*>(chunk + (r * M + s0) * (int)sizeof(T)) = OutIO::pack(v);
                            }
                        }
                    }
                    lds_sync();
                    Piece o[NO];
#pragma unroll
                    for (int i = 0; i < NO; ++i) {
                        o[i] = *reinterpret_cast<const Piece*>(chunk + min(i * 1024 + lane * 16, S::OA_BYTES - 16));
                    }
                    char* out_h = out_tile + (int64_t)h * N * M * sizeof(T);
#pragma unroll
                    for (int i = 0; i < NO; ++i) {
                        const int off = i * 1024 + lane * 16;
                        if (off < chunk_bytes) store_streaming(reinterpret_cast<Piece*>(out_h + off), o[i]);
                    }
                }
                return;
            }
        }

        // the list entry of staging row i*RPI + g_sub lives in the lane of that slot
        int src_lane[S::NI_G];
#pragma unroll
        for (int i = 0; i < S::NI_G; ++i) src_lane[i] = min(i * S::RPI + g_sub, mc - 1);

        // shared list (here only in the kernels for long or odd lists; the FAST kernels took the path above): one
        // pass that serves all tokens; otherwise one pass per token that keeps its column
        const int passes = shared_list ? 1 : nt;
        for (int pass = 0; pass < passes; ++pass) {
            const int tok_lo = shared_list ? 0 : pass;
            const int tok_hi = shared_list ? nt : pass + 1;
            // this pass's list: token `pass` of the tile (re-read from L2 for the per-token passes)
            int mine = list0;
            if (pass > 0) {
                if constexpr (CLUSTERS) {
                    const int row = cid_tile[pass * (M >> 3) + (slot >> 3)] * 8 + (slot & 7);
                    mine = (unsigned)row < (unsigned)N ? row : 0;  // also catches a negative cluster number
                } else {
                    mine = (int)idx_tile[(int64_t)pass * M + j0 + slot];
                }
            }
            uint32_t g_off[S::NI_G];
#pragma unroll
            for (int i = 0; i < S::NI_G; ++i) {
                const int srow = i * S::RPI + g_sub;
                g_off[i] = (uint32_t)__shfl(mine, src_lane[i]) * row_pitch + (uint32_t)((g_pos ^ S::swz(srow)) * 16);
            }
            if (pass > 0 || j0 > 0) {  // the a-row slots hold the last heads of the previous pass
                __syncthreads();
                fetch_a(0);
                if (H > 1) fetch_a(1);
            }

            for (int h = 0; h < H; ++h) {
                // gather: rows of head h -> LDS (and the a-rows of head h when they were not prefetched)
                const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(T);
#pragma unroll
                for (int i = 0; i < S::NI_G; ++i) CLUSTEN_LDS_DMA16(rows_bh + g_off[i], stage + i * 1024);
                if (h >= 2) fetch_a(h);
                __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                __syncthreads();

                // operands: LDS -> registers
                typename RunIO::raw g_raw[Q][S::NU];
                typename RunIO::raw a_raw[S::NU];
#pragma unroll
                for (int u = 0; u < S::NU; ++u) {
#pragma unroll
                    for (int blk = 0; blk < Q; ++blk) {
                        g_raw[blk][u] =
                            *reinterpret_cast<const typename RunIO::raw*>(stage + lds_g[u] + blk * 16 * S::RB);
                    }
                    a_raw[u] =
                        *reinterpret_cast<const typename RunIO::raw*>(stage + lds_a[u] + (h & 1) * S::OA_BYTES);
                }
                __syncthreads();  // operands are in registers: the staging buffer may be reused

                F32x4 d[Q];
#pragma unroll
                for (int blk = 0; blk < Q; ++blk) {
                    d[blk] = F32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int u = 0; u < S::NU; ++u) d[blk] = tile_mfma<T>(g_raw[blk][u], a_raw[u], d[blk]);
                }

                // lane (r, kq) holds slots 16*blk + 4*kq .. +3 of token r
                char* out_h = out_tile + (int64_t)h * N * M * sizeof(T);
                if (r >= tok_lo && r < tok_hi) {
                    T* out_row = reinterpret_cast<T*>(out_h) + r * M + j0;
#pragma unroll
                    for (int blk = 0; blk < Q; ++blk) {
                        const int s0 = 16 * blk + 4 * kq;
                        float v[4] = {d[blk][0], d[blk][1], d[blk][2], d[blk][3]};
                        if (FAST || vec_store) {
                            if (s0 < mc) store_streaming(reinterpret_cast<typename OutIO::raw*>(out_row + s0), OutIO::pack(v));
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                if (s0 + e < mc) out_row[s0 + e] = from_acc<T>(v[e]);
                            }
                        }
                    }
                }
            }
        }
    }
}

// One thread per output element; any dtype, any head dim, any alignment.
template <typename T>
__global__ __launch_bounds__(256) void gather_dot_elem_kernel(const T* __restrict__ a, const T* __restrict__ rows,
                                                              const int64_t* __restrict__ idx, T* __restrict__ out,
                                                              int B, int H, int N, int C, int M, clusten_strides as,
                                                              clusten_strides rs) {
    const int64_t total = (int64_t)B * H * N * M;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int j = (int)(o % M);
        const int64_t q1 = o / M;
        const int i = (int)(q1 % N);
        const int64_t q2 = q1 / N;
        const int h = (int)(q2 % H);
        const int b = (int)(q2 / H);
        const int64_t g = idx[((int64_t)b * N + i) * M + j];
        const T* arow = a + b * as.b + h * as.h + i * as.n;
        const T* krow = rows + b * rs.b + h * rs.h + g * rs.n;
        typename Acc<T>::type acc = 0;
        for (int c = 0; c < C; ++c) acc += to_acc(arow[c]) * to_acc(krow[c]);
        out[o] = from_acc<T>(acc);
    }
}

template <typename T, int C, int Q, bool FAST, bool CLUSTERS = false>
int launch_tile_q(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx,
                  void* out, const clusten_attn_shape& s, hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int groups = head_groups_for(total, s.H);
    hipLaunchKernelGGL((gather_dot_tile_kernel<T, C, Q, FAST, CLUSTERS>), dim3(xcd_grid(total * groups)), dim3(kWave), 0,
                       stream, static_cast<const T*>(a), static_cast<const T*>(rows), idx, static_cast<T*>(out), s.H, s.N,
                       s.M, as, rs, tiles_per_batch, total, groups);
    return launch_status();
}

// Lists of up to 48 slots (the neighbourhood size of every 224x224 model) are one chunk of three
// slot blocks; anything longer goes 64 slots (four blocks) at a time.
template <typename T, int C>
int launch_tile(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                const clusten_attn_shape& s, hipStream_t stream) {
    if (s.M % 4 == 0 && s.M <= 48) return launch_tile_q<T, C, 3, true>(a, as, rows, rs, idx, out, s, stream);
    if (s.M % 4 == 0 && s.M <= 64) return launch_tile_q<T, C, 4, true>(a, as, rows, rs, idx, out, s, stream);
    return launch_tile_q<T, C, 4, false>(a, as, rows, rs, idx, out, s, stream);
}

template <typename T>
int launch_elem(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                const clusten_attn_shape& s, hipStream_t stream) {
    const int64_t total = (int64_t)s.B * s.H * s.N * s.M;
    const int64_t want = (total + 255) / 256;
    const int grid = (int)(want < (int64_t)1 << 20 ? want : (int64_t)1 << 20);
    hipLaunchKernelGGL((gather_dot_elem_kernel<T>), dim3(grid), dim3(256), 0, stream, static_cast<const T*>(a),
                       static_cast<const T*>(rows), idx, static_cast<T*>(out), s.B, s.H, s.N, s.C, s.M, as, rs);
    return launch_status();
}

// Lists given as cluster numbers (see CLUSTERS above): `cluster_idx` is (B, N, M/8) int32 for M <= 64 (clusters of 8)
// and (B, N, M/L) for longer lists, L = runs_length_for(M) the cluster size (24 for the 144 slots of the 384 x 384
// models).  Only the tile kernels take this format: head dim 16/32/64, 16-byte aligned rows.
template <typename T>
int gather_dot_clusters_typed(const void* a, clusten_strides as, const void* rows, clusten_strides rs,
                              const int32_t* cluster_idx, void* out, const clusten_attn_shape& s, hipStream_t stream) {
    const bool vec_ok = rows_aligned16(rows, rs, sizeof(T)) && rows_aligned16(a, as, sizeof(T)) && aligned16(out) &&
                        slice_fits_int32(rs, s.H, s.N, s.C) && slice_fits_int32(as, s.H, s.N, s.C);
    if (!vec_ok) return CLUSTEN_ERR_UNALIGNED;
    if (const int L = runs_length_for(s.M); L != 0 && runs_head_dim_ok<T>(s.C)) {
        return launch_gather_dot_runs<T>(a, as, rows, rs, nullptr, out, s, L, stream, cluster_idx);
    }
    if (s.M % 8 != 0 || s.M > 64) return CLUSTEN_ERR_BAD_DIMS;
    const int64_t* idx = reinterpret_cast<const int64_t*>(cluster_idx);
    switch (s.C) {
        case 16:
            return s.M <= 48 ? launch_tile_q<T, 16, 3, true, true>(a, as, rows, rs, idx, out, s, stream)
                             : launch_tile_q<T, 16, 4, true, true>(a, as, rows, rs, idx, out, s, stream);
        case 32:
            return s.M <= 48 ? launch_tile_q<T, 32, 3, true, true>(a, as, rows, rs, idx, out, s, stream)
                             : launch_tile_q<T, 32, 4, true, true>(a, as, rows, rs, idx, out, s, stream);
        case 64:
            return s.M <= 48 ? launch_tile_q<T, 64, 3, true, true>(a, as, rows, rs, idx, out, s, stream)
                             : launch_tile_q<T, 64, 4, true, true>(a, as, rows, rs, idx, out, s, stream);
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
}

template <typename T>
int gather_dot_typed(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx,
                     void* out, const clusten_attn_shape& s, hipStream_t stream) {
    // the lane runs are 8- or 16-byte accesses at multiples of a quarter row; out rows start 16-byte aligned
    // when M is a multiple of 4 (checked in the kernel) and the base is aligned
    const bool vec_ok = rows_aligned16(rows, rs, sizeof(T)) && rows_aligned16(a, as, sizeof(T)) && aligned16(out) &&
                        slice_fits_int32(rs, s.H, s.N, s.C) && slice_fits_int32(as, s.H, s.N, s.C);
    if (vec_ok) {
        // long lists made of long runs (the 384 x 384 models: 6 clusters of 24 tokens)
        if (const int L = runs_length_for(s.M); L != 0 && runs_head_dim_ok<T>(s.C)) {
            return launch_gather_dot_runs<T>(a, as, rows, rs, idx, out, s, L, stream);
        }
        switch (s.C) {
            case 16: return launch_tile<T, 16>(a, as, rows, rs, idx, out, s, stream);
            case 32: return launch_tile<T, 32>(a, as, rows, rs, idx, out, s, stream);
            case 64: return launch_tile<T, 64>(a, as, rows, rs, idx, out, s, stream);
            default: break;
        }
    }
    return launch_elem<T>(a, as, rows, rs, idx, out, s, stream);
}

}  // namespace clusten
