// gather_dot / gather_sum for long lists made of long runs: the neighbourhoods of the 384 x 384 models.
//
//   gather_dot_runs   out[b,h,i,j] = sum_c a[b,h,i,c] * rows[b,h,idx[b,i,j],c]        (QK forward, AV's d_attn)
//   gather_sum_runs   out[b,h,i,c] = sum_j p[b,h,i,j] * rows[b,h,idx[b,i,j],c]        (AV forward, QK's d_query)
//
// The reference model builds a token's list from the members of its nearest clusters
// (models/aff_transformer.py:476-480); at 384 x 384 a cluster has 24 tokens and a list 144 slots
// (configs/aff_base_22kto1k_384.yaml:10-11): 6 runs of 24 consecutive rows.  The 8 consecutive tokens of a tile sit in
// one cluster and pick their clusters from the same 7-9, each in its own order, so no two lists are equal but nearly
// all their runs are.  As in the union path of the kernels for short lists (gather_dot_impl.hpp), every distinct run
// of the tile is gathered and multiplied once per head:
//
//   1. lane rho < tokens * R owns run rho of the tile (R = M / L runs of L slots per token), reads its L entries and
//      keys the run by its first row when the rows are consecutive (a short last cluster followed by the row 0 its pad
//      slots hold counts as consecutive); any other run gets a key of its own;
//   2. the distinct keys are numbered with a readlane / ballot loop (U of them, at most 16), their rows listed;
//   3. per head and pass of 48 union rows: rows by LDS-direct load, the products on `v_mfma_f32_16x16x4_f32`
//      (16-bit data widened at the LDS read), scores (dot) or sums (sum) per token;
//   4. dot: every lane picks groups of 4 consecutive output elements from the score matrix of the pass that holds
//      them; sum: the tile's p values are laid out by union row (zero where a token does not hold the row, repeats of a
//      run by one token add up) and the product accumulates over the passes.
// A tile with more than 16 distinct runs is taken token by token (a token has at most 8 runs), so any list of
// M = R * L slots is computed exactly, whatever its rows are; only tiles whose tokens share their runs are fast.
// Head dims 32 and 64 (and 16 for fp32), L a multiple of 4 up to 32, R <= 8, rows 16-byte aligned.
#pragma once

#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {

template <typename T, int C>
struct RunsStaging {
    static constexpr int RB = C * (int)sizeof(T);               // bytes per row
    static constexpr int PPR = RB / 16;                         // 16-byte pieces per row
    static constexpr int RPI = kWave / PPR;                     // rows per wave access
    static constexpr int UROWS = 48;                            // union rows per pass: three blocks of 16
    static constexpr int NI_U = (UROWS + RPI - 1) / RPI;        // accesses for the rows of a pass
    static constexpr int NI_A = (kTileTokens + RPI - 1) / RPI;  // accesses for the tile's a-rows / output rows
    static constexpr int G_BYTES = NI_U * 1024;
    static constexpr int SROW = UROWS + 4;                      // floats per token row of the score / weight matrix
    static constexpr int S_BASE = G_BYTES;
    static constexpr int S_BYTES = kTileTokens * SROW * 4;
    static constexpr int A_BASE = (S_BASE + S_BYTES + 1023) / 1024 * 1024;
    static constexpr int A_SLOT = NI_A * 1024;
    static constexpr int U_MAX = 16;                            // distinct runs of a tile
    static constexpr int L_MAX = 32;                            // slots of a run
    static constexpr int ULIST_BASE = A_BASE + 2 * A_SLOT;
    static constexpr int USLOT_BASE = ULIST_BASE + U_MAX * L_MAX * 4;
    static constexpr int BYTES = USLOT_BASE + kWave * 4;
    static constexpr int QB = RB / 4;                           // bytes of a quarter row
    static constexpr int NU = QB / 16;                          // 16-byte pieces per quarter row
    static constexpr int VEC = 16 / (int)sizeof(T);             // elements per piece
    static_assert(QB >= 16 && QB % 16 == 0 && kWave % PPR == 0, "quarter rows of whole 16-byte pieces");
    // XOR swizzle of the piece index: rows r, r+1, ... of a block land in different bank groups
    static __device__ __forceinline__ int swz(int row) { return ((row & 7) ^ ((row >> 3) & 1)) & (PPR - 1); }
};

// The runs of tokens [t0, t0 + ntok) of a tile: distinct runs numbered, their rows listed in LDS.  Returns the number
// of distinct runs, or -1 when there are more than U_MAX.  `uslots[rho]` = number of run rho (token-major), `ulist` =
// L rows per distinct run.
// `cid_tokens` != nullptr: the lists are given as cluster numbers instead (R per token, int32): run r of a token is rows
// L c .. L c + L - 1 of the sequence, row 0 where that is outside [0, N) — every run is regular by construction and
// nothing is read from `idx_tokens`.
template <int U_MAX>
__device__ __forceinline__ int number_runs(const int64_t* __restrict__ idx_tokens, const int32_t* __restrict__ cid_tokens,
                                           int ntok, int M, int L, int R, int N, int* ulist, int* uslots) {
    typedef long long I64x2 __attribute__((ext_vector_type(2)));
    const int lane = threadIdx.x;
    const int nruns = ntok * R;
    const int rho = min(lane, nruns - 1);
    if (cid_tokens != nullptr) {
        const int64_t first = (int64_t)cid_tokens[rho] * L;
        const int key = (first >= 0 && first < N) ? (int)first : -1;   // runs outside the sequence: L times row 0
        uint64_t remaining = nruns >= 64 ? ~0ull : ((1ull << nruns) - 1);
        int uslot = 0, U = 0;
        bool lead = false;
        while (remaining != 0 && U < U_MAX) {
            const int s = __builtin_ctzll(remaining);
            const int ks = __builtin_amdgcn_readlane(key, s);
            const bool hit = key == ks;
            const uint64_t match = __ballot(hit) & remaining;
            if (hit) uslot = U;
            lead = lead || lane == s;
            remaining &= ~match;
            ++U;
        }
        if (remaining != 0) return -1;
        if (lead && lane < nruns) {
            for (int t = 0; t < L; ++t) ulist[uslot * L + t] = (key >= 0 && key + t < N) ? key + t : 0;
        }
        if (lane < nruns) uslots[lane] = uslot;
        return U;
    }
    const int64_t* run = idx_tokens + (int64_t)(rho / R) * M + (rho % R) * L;
    const int v0 = (int)run[0];
    // L consecutive rows, or the short last cluster of the sequence followed by the row 0 its pad slots hold?
    // and: do all tokens carry the same list?  (lists without any structure but common to the tile, e.g. one drawn per
    // cluster: run r of every token then is run r of the first one, whatever its rows are)
    const int own = (v0 + L > N && v0 < N) ? N - v0 : L;
    bool regular = v0 >= 0 && v0 < N;
    bool same = true;
    // the run's entries, 8 loads of two at a time in flight (one after the other they would be L / 2 round trips to
    // memory before the tile's first gather)
    for (int t0 = 0; t0 < L; t0 += 16) {
        I64x2 two[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            two[u] = *reinterpret_cast<const I64x2*>(run + min(t0 + 2 * u, L - 2));
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = t0 + 2 * u;
            if (t < L) {   // uniform
                const int x = (int)two[u][0], y = (int)two[u][1];
                regular = regular && x == (t < own ? v0 + t : 0) && y == (t + 1 < own ? v0 + t + 1 : 0);
                same = same && x == __shfl(x, rho % R) && y == __shfl(y, rho % R);
            }
        }
    }
    const bool shared = __all((lane >= nruns || same) ? 1 : 0) != 0;
    const int key = regular ? v0 : (shared ? ~(rho % R) : ~lane);   // other runs never merge
    uint64_t remaining = nruns >= 64 ? ~0ull : ((1ull << nruns) - 1);
    int uslot = 0, U = 0;
    bool first = false;
    while (remaining != 0 && U < U_MAX) {
        const int s = __builtin_ctzll(remaining);
        const int ks = __builtin_amdgcn_readlane(key, s);
        const bool hit = key == ks;
        const uint64_t match = __ballot(hit) & remaining;
        if (hit) uslot = U;
        first = first || lane == s;
        remaining &= ~match;
        ++U;
    }
    if (remaining != 0) return -1;
    if (first && lane < nruns) {
        for (int t0 = 0; t0 < L; t0 += 16) {   // the rows of a distinct run, read again by the lane that stands for it
            I64x2 two[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                two[u] = *reinterpret_cast<const I64x2*>(run + min(t0 + 2 * u, L - 2));
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int t = t0 + 2 * u;
                if (t < L) {
                    ulist[uslot * L + t] = (int)two[u][0];
                    ulist[uslot * L + t + 1] = (int)two[u][1];
                }
            }
        }
    }
    if (lane < nruns) uslots[lane] = uslot;
    return U;
}

// ---- gather_dot ----------------------------------------------------------------------------------------------------

// Tokens [i0, i0 + nt) (nt <= 8) of batch element b, all heads; `stage`: RunsStaging<T, C>::BYTES bytes of LDS.
template <typename T, int C>
__device__ __forceinline__ void gather_dot_runs_tokens(char* stage, const T* __restrict__ a, const T* __restrict__ rows,
                                                       const int64_t* __restrict__ idx, const int32_t* __restrict__ cid,
                                                       T* __restrict__ out, int H, int N, int M, int L, clusten_strides as,
                                                       clusten_strides rs, int b, int i0, int nt) {
    typedef RunsStaging<T, C> S;
    typedef VecIO<T, S::VEC> PieceIO;
    typedef VecIO<T, 4> OutIO;
    constexpr int NQD_MAX = (kTileTokens * 256 / 4 + kWave - 1) / kWave;   // output groups of 4 per lane, M <= 256
    const int lane = threadIdx.x;
    const int r = lane & 15, kq = lane >> 4;
    const int g_sub = lane / S::PPR, g_pos = lane % S::PPR;
    const int R = M / L;
    const uint32_t row_pitch = (uint32_t)rs.n * sizeof(T);
    int* ulist = reinterpret_cast<int*>(stage + S::ULIST_BASE);
    int* uslots = reinterpret_cast<int*>(stage + S::USLOT_BASE);
    float* scores = reinterpret_cast<float*>(stage + S::S_BASE);
    const char* rows_b = reinterpret_cast<const char*>(rows + (int64_t)b * rs.b);

    // the whole tile when its tokens share their runs, else token by token
    int ntok = nt;
    for (int t0 = 0; t0 < nt;) {
        lds_sync();
        const int U = number_runs<S::U_MAX>(idx + ((int64_t)b * N + i0 + t0) * M,
                                            cid != nullptr ? cid + ((int64_t)b * N + i0 + t0) * R : nullptr, ntok, M, L, R, N,
                                            ulist, uslots);
        if (U < 0) {   // more distinct runs than the tables hold: one token at a time (at most R <= 8 runs)
            ntok = 1;
            continue;
        }
        lds_sync();
        // this lane's share of the output: groups of 4 consecutive elements (inside one run, L % 4 == 0)
        int sidx[NQD_MAX], qtok[NQD_MAX];
#pragma unroll
        for (int k = 0; k < NQD_MAX; ++k) {
            const int e = 4 * (lane + kWave * k);
            const int ec = e < ntok * M ? e : 0;
            const int i = ec / M, j = ec - i * M;
            const int run = j / L;
            qtok[k] = i;
            sidx[k] = e < ntok * M ? uslots[i * R + run] * L + (j - run * L) : -1000000;
        }
        const int total_rows = U * L;
        const char* a_part = reinterpret_cast<const char*>(a + (int64_t)b * as.b + (int64_t)(i0 + t0) * as.n);
        char* out_part = reinterpret_cast<char*>(out + (((int64_t)b * H) * N + i0 + t0) * M);
        // Heads outside, passes of UROWS union rows inside.  The rows of the next pass (of this head or the next one,
        // whose a-rows go along into the other a-row slot) are requested as soon as the operands of the current pass
        // are in registers, and the stores of a head are issued after the first request of the next head, whose wait
        // leaves them in flight: a tile's chain of passes is long (heads x 4 passes at 144 slots), and each link
        // would otherwise be a full trip to memory.
        auto fetch_a = [&](int h) {
#pragma unroll
            for (int i = 0; i < S::NI_A; ++i) {
                const int srow = i * S::RPI + g_sub;
                CLUSTEN_LDS_DMA16(a_part + (int64_t)h * as.h * sizeof(T) +
                                      lane_offset((uint32_t)min(srow, ntok - 1) * (uint32_t)as.n * sizeof(T) +
                                                  (uint32_t)((g_pos ^ S::swz(srow)) * 16)),
                                  stage + S::A_BASE + (h & 1) * S::A_SLOT + i * 1024);
            }
        };
        auto gather_pass = [&](int h, int base) {
            const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(T);
            const int rows_here = min(S::UROWS, total_rows - base);
#pragma unroll
            for (int i = 0; i < S::NI_U; ++i) {
                if (i * S::RPI < rows_here) {
                    const int srow = i * S::RPI + g_sub;
                    const uint32_t urow = (uint32_t)ulist[min(base + srow, total_rows - 1)];
                    CLUSTEN_LDS_DMA16(rows_bh + lane_offset(urow * row_pitch + (uint32_t)((g_pos ^ S::swz(srow)) * 16)),
                                      stage + i * 1024);
                }
            }
        };
        const int n_stores = (ntok * M + 4 * kWave - 1) / (4 * kWave);   // store instructions of a head, <= NQD_MAX
        lds_sync();  // the previous group of tokens has read its operands
        fetch_a(0);
        gather_pass(0, 0);
        for (int h = 0; h < H; ++h) {
            F32x4 val[NQD_MAX];
#pragma unroll
            for (int k = 0; k < NQD_MAX; ++k) val[k] = F32x4{0.f, 0.f, 0.f, 0.f};
            for (int base = 0; base < total_rows; base += S::UROWS) {
                const int rows_here = min(S::UROWS, total_rows - base);
                Piece a_raw[S::NU];
                if (base == 0 && h > 0) {
                    // everything but the stores of the previous head
                    switch (n_stores) {
                        case 1: lds_sync_vm<1>(); break;
                        case 2: lds_sync_vm<2>(); break;
                        case 3: lds_sync_vm<3>(); break;
                        case 4: lds_sync_vm<4>(); break;
                        case 5: lds_sync_vm<5>(); break;
                        case 6: lds_sync_vm<6>(); break;
                        case 7: lds_sync_vm<7>(); break;
                        case 8: lds_sync_vm<8>(); break;
                        default: lds_sync_vm<0>(); break;
                    }
                } else {
                    lds_sync_vm<0>();
                }
                Piece g_raw[S::UROWS / 16][S::NU];
#pragma unroll
                for (int u = 0; u < S::NU; ++u) {
                    const int piece = kq * S::NU + u;
#pragma unroll
                    for (int blk = 0; blk < S::UROWS / 16; ++blk) {
                        if (blk * 16 < rows_here) {
                            const int grow = 16 * blk + r;
                            g_raw[blk][u] = *reinterpret_cast<const Piece*>(stage + grow * S::RB + ((piece ^ S::swz(grow)) * 16));
                        }
                    }
                    a_raw[u] = *reinterpret_cast<const Piece*>(stage + S::A_BASE + (h & 1) * S::A_SLOT + (r & 7) * S::RB +
                                                               ((piece ^ S::swz(r & 7)) * 16));
                }
                lds_sync();  // operands are in registers: the row area is free for the next pass
                if (base + S::UROWS < total_rows) {
                    gather_pass(h, base + S::UROWS);
                } else if (h + 1 < H) {
                    fetch_a(h + 1);
                    gather_pass(h + 1, 0);
                }
#pragma unroll
                for (int blk = 0; blk < S::UROWS / 16; ++blk) {
                    if (blk * 16 < rows_here) {
                        F32x4 d = F32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int u = 0; u < S::NU; ++u) {
                            float gx[S::VEC], ax[S::VEC];
                            PieceIO::unpack(g_raw[blk][u], gx);
                            PieceIO::unpack(a_raw[u], ax);
#pragma unroll
                            for (int e = 0; e < S::VEC; ++e) d = mfma_16x16x4(gx[e], ax[e], d);
                        }
                        // lane (r, kq): union rows 16*blk + 4*kq .. +3 of token r
                        if (r < kTileTokens) *reinterpret_cast<F32x4*>(scores + r * S::SROW + 16 * blk + 4 * kq) = d;
                    }
                }
                lds_sync();
#pragma unroll
                for (int k = 0; k < NQD_MAX; ++k) {
                    const int sl = sidx[k] - base;
                    if (sl >= 0 && sl < S::UROWS) val[k] = *reinterpret_cast<const F32x4*>(scores + qtok[k] * S::SROW + sl);
                }
            }
            char* out_h = out_part + (int64_t)h * N * M * sizeof(T);
#pragma unroll
            for (int k = 0; k < NQD_MAX; ++k) {
                if (4 * (lane + kWave * k) < ntok * M) {
                    const float o[4] = {val[k][0], val[k][1], val[k][2], val[k][3]};
                    store_streaming(reinterpret_cast<typename OutIO::raw*>(out_h + (lane + kWave * k) * 4 * (int)sizeof(T)),
                                    OutIO::pack(o));
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));   // the next group's tables go over areas the stores do not touch, but
                                                      // its first wait counts from zero
        t0 += ntok;
    }
}

template <typename T, int C>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(C <= 32 ? 3 : 1))) void gather_dot_runs_kernel(
    const T* __restrict__ a, const T* __restrict__ rows, const int64_t* __restrict__ idx, const int32_t* __restrict__ cid,
    T* __restrict__ out, int H, int N, int M, int L, clusten_strides as, clusten_strides rs, int tiles_per_batch,
    int total_tiles) {
    __shared__ __attribute__((aligned(1024))) char stage[RunsStaging<T, C>::BYTES];
    const int tile = xcd_tile(blockIdx.x, total_tiles);
    if (tile < 0) return;
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTileTokens;
    gather_dot_runs_tokens<T, C>(stage, a, rows, idx, cid, out, H, N, M, L, as, rs, b, i0, min(kTileTokens, N - i0));
}

// ---- gather_sum ----------------------------------------------------------------------------------------------------

// Tokens [i0, i0 + nt) (nt <= 8) of batch element b, all heads; `stage`: RunsStaging<T, C>::BYTES bytes of LDS.
template <typename T, int C>
__device__ __forceinline__ void gather_sum_runs_tokens(char* stage, const T* __restrict__ p, const T* __restrict__ rows,
                                                       const int64_t* __restrict__ idx, const int32_t* __restrict__ cid,
                                                       T* __restrict__ out, int H, int N, int M, int L, clusten_strides rs,
                                                       clusten_strides os, int b, int i0, int nt) {
    typedef RunsStaging<T, C> S;
    typedef VecIO<T, 4> OutIO;
    constexpr int CB = C / 16;   // channel blocks of 16
    const int lane = threadIdx.x;
    const int n16 = lane & 15, kq = lane >> 4;
    const int g_sub = lane / S::PPR, g_pos = lane % S::PPR;
    const int R = M / L;
    const uint32_t row_pitch = (uint32_t)rs.n * sizeof(T);
    int* ulist = reinterpret_cast<int*>(stage + S::ULIST_BASE);
    int* uslots = reinterpret_cast<int*>(stage + S::USLOT_BASE);
    float* weights = reinterpret_cast<float*>(stage + S::S_BASE);   // p of the pass by union row: [token][SROW]
    float* chunk = reinterpret_cast<float*>(stage + S::A_BASE);     // the tile's output rows, fp32: 8 x C
    const char* rows_b = reinterpret_cast<const char*>(rows + (int64_t)b * rs.b);
    const int tb = lane >> 3, sub = lane & 7;                       // build side: token and slot phase of the lane

    int ntok = nt;
    for (int t0 = 0; t0 < nt;) {
        lds_sync();
        const int U = number_runs<S::U_MAX>(idx + ((int64_t)b * N + i0 + t0) * M,
                                            cid != nullptr ? cid + ((int64_t)b * N + i0 + t0) * R : nullptr, ntok, M, L, R, N,
                                            ulist, uslots);
        if (U < 0) {   // more distinct runs than the tables hold: one token at a time (at most R <= 8 runs)
            ntok = 1;
            continue;
        }
        lds_sync();
        const int total_rows = U * L;
        for (int h = 0; h < H; ++h) {
            const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(T);
            const T* p_tok = p + (((int64_t)b * H + h) * N + i0 + t0 + min(tb, ntok - 1)) * M;
            // the lane's p values of the head: slots sub, sub + 8, ... of every run of its token, requested together
            float pv[8][4];
#pragma unroll
            for (int run = 0; run < 8; ++run) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int t = sub + 8 * k;
                    pv[run][k] = (run < R && t < L) ? to_acc(p_tok[run * L + t]) : 0.f;
                }
            }
            F32x4 d[CB];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) d[cb] = F32x4{0.f, 0.f, 0.f, 0.f};
            for (int base = 0; base < total_rows; base += S::UROWS) {
                const int rows_here = min(S::UROWS, total_rows - base);
                lds_sync();  // the previous pass has read its operands
#pragma unroll
                for (int i = 0; i < S::NI_U; ++i) {
                    if (i * S::RPI < rows_here) {
                        const int srow = i * S::RPI + g_sub;
                        const uint32_t urow = (uint32_t)ulist[min(base + srow, total_rows - 1)];
                        CLUSTEN_LDS_DMA16(rows_bh + lane_offset(urow * row_pitch + (uint32_t)((g_pos ^ S::swz(srow)) * 16)),
                                          stage + i * 1024);
                    }
                }
                // p of this pass by union row: zero, then every token's runs in turn (a run held twice adds up: the
                // same lane meets both)
                for (int z = lane; z < kTileTokens * S::SROW; z += kWave) weights[z] = 0.f;
                lds_sync();
                if (tb < ntok) {
#pragma unroll
                    for (int run = 0; run < 8; ++run) {
                        if (run < R) {
                            const int first = uslots[tb * R + run] * L - base;   // union row of the run's first slot, in this pass
#pragma unroll
                            for (int k = 0; k < 4; ++k) {
                                const int row = first + sub + 8 * k;
                                if (sub + 8 * k < L && row >= 0 && row < S::UROWS) weights[tb * S::SROW + row] += pv[run][k];
                            }
                        }
                    }
                }
                lds_sync_vm<0>();
                // D[token][c] += W[token][row] * G[row][c]: k index kq of step s is row 12*kq + s of the pass, so that a
                // lane's weights are 12 consecutive floats; lane n16 holds channels n16*CB .. +CB-1 of a row
                F32x4 w4[3];
#pragma unroll
                for (int q = 0; q < 3; ++q) w4[q] = *reinterpret_cast<const F32x4*>(weights + (n16 & 7) * S::SROW + 12 * kq + 4 * q);
#pragma unroll
                for (int sstep = 0; sstep < S::UROWS / 4; ++sstep) {
                    const int grow = 12 * kq + sstep;
                    const bool live = grow < rows_here;
                    const float wa = live ? w4[sstep / 4][sstep % 4] : 0.f;
                    constexpr int CH_B = CB * (int)sizeof(T);                 // bytes of the lane's channels
                    const int byte = n16 * CH_B;
                    const typename VecIO<T, CB>::raw graw = *reinterpret_cast<const typename VecIO<T, CB>::raw*>(
                        stage + grow * S::RB + (((byte / 16) ^ S::swz(grow)) * 16) + byte % 16);
                    float g[CB];
                    VecIO<T, CB>::unpack(graw, g);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) d[cb] = mfma_16x16x4(wa, live ? g[cb] : 0.f, d[cb]);
                }
            }
            // lane (n16, kq): tokens 4*kq .. +3 (kq < 2: the tile's 8) of channels n16*CB + cb -> row-major chunk -> stores
            lds_sync();
            if (kq < 2) {
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) chunk[(4 * kq + j) * C + n16 * CB + cb] = d[cb][j];
                }
            }
            lds_sync();
            T* out_h = out + (int64_t)b * os.b + (int64_t)h * os.h + (int64_t)(i0 + t0) * os.n;
#pragma unroll
            for (int q0 = 0; q0 < kTileTokens * C / 4; q0 += kWave) {
                const int q = q0 + lane;
                const int tok = q / (C / 4), c4 = q - tok * (C / 4);
                if (q < kTileTokens * C / 4 && tok < ntok) {
                    const F32x4 o = *reinterpret_cast<const F32x4*>(chunk + tok * C + 4 * c4);
                    const float v[4] = {o[0], o[1], o[2], o[3]};
                    store_streaming(reinterpret_cast<typename OutIO::raw*>(out_h + (int64_t)tok * os.n + 4 * c4), OutIO::pack(v));
                }
            }
        }
        t0 += ntok;
    }
}

template <typename T, int C>
__global__ __launch_bounds__(kWave) void gather_sum_runs_kernel(const T* __restrict__ p, const T* __restrict__ rows,
                                                                const int64_t* __restrict__ idx,
                                                                const int32_t* __restrict__ cid, T* __restrict__ out,
                                                                int H, int N, int M, int L, clusten_strides rs,
                                                                clusten_strides os, int tiles_per_batch, int total_tiles) {
    __shared__ __attribute__((aligned(1024))) char stage[RunsStaging<T, C>::BYTES];
    const int tile = xcd_tile(blockIdx.x, total_tiles);
    if (tile < 0) return;
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTileTokens;
    gather_sum_runs_tokens<T, C>(stage, p, rows, idx, cid, out, H, N, M, L, rs, os, b, i0, min(kTileTokens, N - i0));
}

// ---- launch ----------------------------------------------------------------------------------------------------------

// The run length these kernels take a list of M slots in: the cluster size of the 384 x 384 models first.
inline int runs_length_for(int M) {
    if (M <= 64 || M > 256 || M % 8 != 0) return 0;
    const int candidates[3] = {24, 32, 16};
    for (int L : candidates) {
        if (M % L == 0 && M / L <= 8) return L;
    }
    return 0;
}

template <typename T>
constexpr bool runs_head_dim_ok(int C) {
    return (C == 32 || C == 64 || C == 16) && C * (int)sizeof(T) >= 64;
}

template <typename T, int C>
int launch_gather_dot_runs_c(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx,
                             void* out, const clusten_attn_shape& s, int L, hipStream_t stream, const int32_t* cid) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    hipLaunchKernelGGL((gather_dot_runs_kernel<T, C>), dim3(xcd_grid(total)), dim3(kWave), 0, stream,
                       static_cast<const T*>(a), static_cast<const T*>(rows), idx, cid, static_cast<T*>(out), s.H, s.N, s.M, L,
                       as, rs, tiles_per_batch, total);
    return launch_status();
}

// `cid` != nullptr: the lists as cluster numbers, (B, N, M / L) int32 (see number_runs); `idx` is not read then.
template <typename T>
int launch_gather_dot_runs(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx,
                           void* out, const clusten_attn_shape& s, int L, hipStream_t stream, const int32_t* cid = nullptr) {
    if constexpr (sizeof(T) == 4) {
        if (s.C == 16) return launch_gather_dot_runs_c<T, 16>(a, as, rows, rs, idx, out, s, L, stream, cid);
    }
    if (s.C == 32) return launch_gather_dot_runs_c<T, 32>(a, as, rows, rs, idx, out, s, L, stream, cid);
    return launch_gather_dot_runs_c<T, 64>(a, as, rows, rs, idx, out, s, L, stream, cid);
}

template <typename T, int C>
int launch_gather_sum_runs_c(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                             clusten_strides os, const clusten_attn_shape& s, int L, hipStream_t stream, const int32_t* cid) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    hipLaunchKernelGGL((gather_sum_runs_kernel<T, C>), dim3(xcd_grid(total)), dim3(kWave), 0, stream,
                       static_cast<const T*>(p), static_cast<const T*>(rows), idx, cid, static_cast<T*>(out), s.H, s.N, s.M, L,
                       rs, os, tiles_per_batch, total);
    return launch_status();
}

template <typename T>
int launch_gather_sum_runs(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                           clusten_strides os, const clusten_attn_shape& s, int L, hipStream_t stream,
                           const int32_t* cid = nullptr) {
    if constexpr (sizeof(T) == 4) {
        if (s.C == 16) return launch_gather_sum_runs_c<T, 16>(p, rows, rs, idx, out, os, s, L, stream, cid);
    }
    if (s.C == 32) return launch_gather_sum_runs_c<T, 32>(p, rows, rs, idx, out, os, s, L, stream, cid);
    return launch_gather_sum_runs_c<T, 64>(p, rows, rs, idx, out, os, s, L, stream, cid);
}

}  // namespace clusten
