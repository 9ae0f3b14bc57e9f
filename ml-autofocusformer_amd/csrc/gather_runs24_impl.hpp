// gather_sum on lists made of runs of 24 slots, one workgroup per 24 consecutive tokens: the neighbourhoods of the
// 384 x 384 models (clusters of 24 tokens, the members of the 6 nearest clusters:
// configs/aff_base_22kto1k_384.yaml:10-11, lists built by models/aff_transformer.py:476-480).
//
//   out[b,h,i,c] = sum_j p[b,h,i,j] * rows[b,h,idx[b,i,j],c]        (AV forward, QK's d_query)
//
// The 24 tokens of a tile are one cluster of the cluster-ordered sequence; they pick their clusters from the same
// 9-12, so the tile has some 10 distinct runs where its three groups of 8 tokens, taken on their own
// (gather_runs_impl.hpp), gather and multiply 8 each.  Per head and pass of 48 union rows = two distinct runs, the
// weights of the pass by union row come straight from global memory, 16 bytes per (token, run, quad) — zero where a
// token does not hold the run — and D[token][c] accumulates over the passes on `v_mfma_f32_16x16x4_f32`, tokens 0-15
// and 16-23 as two sets of rows.
// A tile whose runs are not all 24 consecutive rows, that has more than 16 distinct runs, or in which a token holds a
// run twice, is handed to the kernel for 8 tokens, one group of 8 after the other: any list is computed exactly.
// (The same tile for gather_dot was measured and not kept: it ran no faster than the 8-token kernel with its passes
// pipelined, 316 against 290 us at B16 H4 N9216 fp32.)
#pragma once

#include "gather_runs_impl.hpp"

namespace clusten {

constexpr int kRun24 = 24;          // slots of a run
constexpr int kTile24 = 24;         // tokens of a tile

template <typename T, int C>
struct Runs24Staging {
    typedef RunsStaging<T, C> S8;
    static constexpr int RB = S8::RB, PPR = S8::PPR, RPI = S8::RPI, UROWS = S8::UROWS, NI_U = S8::NI_U;
    static constexpr int G_BYTES = NI_U * 1024;
    static constexpr int SROW = UROWS + 4;                       // floats per token row of the score / weight matrix
    static constexpr int S_BASE = G_BYTES;
    static constexpr int S_BYTES = kTile24 * SROW * 4;
    static constexpr int A_BASE = (S_BASE + S_BYTES + 1023) / 1024 * 1024;
    static constexpr int A_SLOT = (kTile24 * C * 4 + 1023) / 1024 * 1024;   // the tile's output rows in fp32
    static constexpr int U_MAX = 16;                             // distinct runs of a tile
    static constexpr int ULIST_BASE = A_BASE + A_SLOT;           // rows of the distinct runs, 24 each
    static constexpr int INV_BASE = ULIST_BASE + U_MAX * kRun24 * 4;   // [token][distinct run] -> run of the token, or 255
    static constexpr int BYTES_24 = INV_BASE + kTile24 * U_MAX;
    static constexpr int BYTES = BYTES_24 > S8::BYTES ? BYTES_24 : S8::BYTES;
    static constexpr int NU = S8::NU, VEC = S8::VEC;
    static __device__ __forceinline__ int swz(int row) { return S8::swz(row); }
};

// The runs of the nt <= 24 tokens of a tile (R <= 8 runs of 24 each): distinct runs numbered in order of first
// appearance, their rows listed (ulist: 24 per distinct run), inv[token * U_MAX + number] = run of the token.
// Returns the number of distinct runs, or -1 when the tile is not for this path.
// `cid_tile` != nullptr: the lists as cluster numbers (R per token, int32; run r of a token = rows 24 c .. 24 c + 23, row
// 0 where that is outside [0, N)); nothing is read from `idx_tile` then.
template <int U_MAX>
__device__ __forceinline__ int number_runs24(const int64_t* __restrict__ idx_tile, const int32_t* __restrict__ cid_tile,
                                             int nt, int M, int R, int N, int* ulist, unsigned char* inv) {
    typedef long long I64x2 __attribute__((ext_vector_type(2)));
    constexpr int L = kRun24;
    const int lane = threadIdx.x;
    int key[3];
    bool live[3];
    bool bad = false;
#pragma unroll
    for (int g = 0; g < 3; ++g) {
        const int ntg = max(0, min(kTileTokens, nt - kTileTokens * g));
        const int nruns = ntg * R;
        live[g] = lane < nruns;
        const int rho = min(lane, max(nruns, 1) - 1);
        if (cid_tile != nullptr) {
            const int64_t first = (int64_t)cid_tile[(kTileTokens * min(g, (nt - 1) / kTileTokens) + rho / R) * R + rho % R] * L;
            key[g] = (first >= 0 && first < N) ? (int)first : -1;   // a run outside the sequence: 24 times row 0
            continue;
        }
        const int64_t* run = idx_tile + (int64_t)(kTileTokens * min(g, (nt - 1) / kTileTokens) + rho / R) * M + (rho % R) * L;
        I64x2 two[12];
#pragma unroll
        for (int u = 0; u < 12; ++u) two[u] = *reinterpret_cast<const I64x2*>(run + 2 * u);
        const int v0 = (int)two[0][0];
        const int own = (v0 + L > N && v0 < N) ? N - v0 : L;   // the short last cluster is followed by pad slots (row 0)
        bool regular = v0 >= 0 && v0 < N;
#pragma unroll
        for (int u = 0; u < 12; ++u) {
            const int t = 2 * u;
            regular = regular && (int)two[u][0] == (t < own ? v0 + t : 0) && (int)two[u][1] == (t + 1 < own ? v0 + t + 1 : 0);
        }
        key[g] = v0;
        bad = bad || (live[g] && !regular);
    }
    if (__any(bad ? 1 : 0) != 0) return -1;

    uint64_t remaining[3];
#pragma unroll
    for (int g = 0; g < 3; ++g) remaining[g] = __ballot(live[g]);
    // lanes below this one that hold runs of the same token
    const uint64_t same_token_below = ((1ull << lane) - 1) & ~((1ull << (lane / R * R)) - 1);
    int uslot[3] = {0, 0, 0};
    bool first[3] = {false, false, false};
    bool twice = false;
    int U = 0;
    while ((remaining[0] | remaining[1] | remaining[2]) != 0 && U < U_MAX) {
        int ks;
        if (remaining[0] != 0) {
            const int s = __builtin_ctzll(remaining[0]);
            ks = __builtin_amdgcn_readlane(key[0], s);
            first[0] = first[0] || lane == s;
        } else if (remaining[1] != 0) {
            const int s = __builtin_ctzll(remaining[1]);
            ks = __builtin_amdgcn_readlane(key[1], s);
            first[1] = first[1] || lane == s;
        } else {
            const int s = __builtin_ctzll(remaining[2]);
            ks = __builtin_amdgcn_readlane(key[2], s);
            first[2] = first[2] || lane == s;
        }
#pragma unroll
        for (int g = 0; g < 3; ++g) {
            const bool hit = live[g] && key[g] == ks;
            const uint64_t match = __ballot(hit) & remaining[g];
            if (hit) uslot[g] = U;
            twice = twice || (hit && (match & same_token_below) != 0);
            remaining[g] &= ~match;
        }
        ++U;
    }
    if ((remaining[0] | remaining[1] | remaining[2]) != 0 || __any(twice ? 1 : 0) != 0) return -1;

    // tables
    for (int z = lane; z < kTile24 * U_MAX / 4; z += kWave) reinterpret_cast<uint32_t*>(inv)[z] = ~0u;
    lds_sync();
#pragma unroll
    for (int g = 0; g < 3; ++g) {
        if (live[g]) {
            const int tok = kTileTokens * g + lane / R, run = lane % R;
            inv[tok * U_MAX + uslot[g]] = (unsigned char)run;
        }
        if (first[g] && live[g]) {   // consecutive rows from key[g] on; past the end of the sequence: row 0
#pragma unroll
            for (int t = 0; t < L; ++t) ulist[uslot[g] * L + t] = (key[g] >= 0 && key[g] + t < N) ? key[g] + t : 0;
        }
    }
    return U;
}

// ---- gather_sum ----------------------------------------------------------------------------------------------------

template <typename T, int C>
__global__ __launch_bounds__(kWave) void gather_sum_runs24_kernel(const T* __restrict__ p, const T* __restrict__ rows,
                                                                  const int64_t* __restrict__ idx,
                                                                  const int32_t* __restrict__ cid, T* __restrict__ out, int H,
                                                                  int N, int M, clusten_strides rs, clusten_strides os,
                                                                  int tiles_per_batch, int total_tiles) {
    typedef Runs24Staging<T, C> S;
    typedef VecIO<T, 4> QuadIO;
    constexpr int L = kRun24;
    constexpr int CB = C / 16;   // channel blocks of 16
    __shared__ __attribute__((aligned(1024))) char stage[S::BYTES];

    const int tile = xcd_tile(blockIdx.x, total_tiles);
    if (tile < 0) return;
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTile24;
    const int nt = min(kTile24, N - i0);
    const int lane = threadIdx.x;
    const int n16 = lane & 15, kq = lane >> 4;
    const int g_sub = lane / S::PPR, g_pos = lane % S::PPR;
    const int R = M / L;
    const uint32_t row_pitch = (uint32_t)rs.n * sizeof(T);
    int* ulist = reinterpret_cast<int*>(stage + S::ULIST_BASE);
    unsigned char* inv = reinterpret_cast<unsigned char*>(stage + S::INV_BASE);
    float* weights = reinterpret_cast<float*>(stage + S::S_BASE);   // p of the pass by union row: [token][SROW]
    float* chunk = reinterpret_cast<float*>(stage + S::A_BASE);     // the tile's output rows, fp32: 24 x C

    const int U = number_runs24<S::U_MAX>(idx + ((int64_t)b * N + i0) * M,
                                          cid != nullptr ? cid + ((int64_t)b * N + i0) * R : nullptr, nt, M, R, N, ulist, inv);
    if (U < 0) {
        for (int g = 0; g * kTileTokens < nt; ++g) {
            gather_sum_runs_tokens<T, C>(stage, p, rows, idx, cid, out, H, N, M, L, rs, os, b, i0 + g * kTileTokens,
                                         min(kTileTokens, nt - g * kTileTokens));
        }
        return;
    }
    lds_sync();

    const char* rows_b = reinterpret_cast<const char*>(rows + (int64_t)b * rs.b);
    const int total_rows = U * L;
    constexpr int TASKS = kTile24 * 2 * (L / 4);
    constexpr int NTASK = (TASKS + kWave - 1) / kWave;
    // this lane's tasks: (token, which of a pass's two runs, quad); the weight matrix cell they fill
    int t_tok[NTASK], t_w[NTASK], t_cell[NTASK], t_src[NTASK];
#pragma unroll
    for (int k = 0; k < NTASK; ++k) {
        const int q = min(lane + kWave * k, TASKS - 1);
        const int tok = q / (2 * (L / 4)), rest = q - tok * (2 * (L / 4));
        const int w = rest / (L / 4), j4 = rest - w * (L / 4);
        t_tok[k] = lane + kWave * k < TASKS ? tok : -1;
        t_w[k] = w;
        t_cell[k] = tok * S::SROW + L * w + 4 * j4;
        t_src[k] = min(tok, nt - 1) * M + 4 * j4;
    }

    for (int h = 0; h < H; ++h) {
        const char* rows_bh = rows_b + (int64_t)h * rs.h * sizeof(T);
        const T* p_h = p + (((int64_t)b * H + h) * N + i0) * M;
        F32x4 d[2][CB];
#pragma unroll
        for (int cs = 0; cs < 2; ++cs) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) d[cs][cb] = F32x4{0.f, 0.f, 0.f, 0.f};
        }
        for (int base = 0, pass = 0; base < total_rows; base += S::UROWS, ++pass) {
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
            // the weights of the pass by union row, 4 at a time from the token's p row; zero where a token does not
            // hold the run
            typename QuadIO::raw pq[NTASK];
            bool have[NTASK];
#pragma unroll
            for (int k = 0; k < NTASK; ++k) {
                have[k] = false;
                if (t_tok[k] >= 0 && t_tok[k] < nt && 2 * pass + t_w[k] < U) {
                    const int run = inv[t_tok[k] * S::U_MAX + 2 * pass + t_w[k]];
                    if (run != 255) {
                        have[k] = true;
                        pq[k] = *reinterpret_cast<const typename QuadIO::raw*>(p_h + t_src[k] + run * L);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < NTASK; ++k) {
                if (t_tok[k] >= 0) {
                    float x[4] = {0.f, 0.f, 0.f, 0.f};
                    if (have[k]) QuadIO::unpack(pq[k], x);
                    *reinterpret_cast<F32x4*>(weights + t_cell[k]) = F32x4{x[0], x[1], x[2], x[3]};
                }
            }
            lds_sync_vm<0>();
            // D[token][c] += W[token][row] * G[row][c]: k index kq of step s is row 12*kq + s of the pass, so that a
            // lane's weights are 12 consecutive floats; lane n16 holds channels n16*CB .. +CB-1 of a row
            F32x4 w4[2][3];
#pragma unroll
            for (int cs = 0; cs < 2; ++cs) {
                const int tok = min(16 * cs + n16, kTile24 - 1);
#pragma unroll
                for (int q = 0; q < 3; ++q) w4[cs][q] = *reinterpret_cast<const F32x4*>(weights + tok * S::SROW + 12 * kq + 4 * q);
            }
#pragma unroll
            for (int sstep = 0; sstep < S::UROWS / 4; ++sstep) {
                const int grow = 12 * kq + sstep;
                const bool alive = grow < rows_here;
                constexpr int CH_B = CB * (int)sizeof(T);                 // bytes of the lane's channels
                const int byte = n16 * CH_B;
                const typename VecIO<T, CB>::raw graw = *reinterpret_cast<const typename VecIO<T, CB>::raw*>(
                    stage + grow * S::RB + (((byte / 16) ^ S::swz(grow)) * 16) + byte % 16);
                float g[CB];
                VecIO<T, CB>::unpack(graw, g);
#pragma unroll
                for (int cs = 0; cs < 2; ++cs) {
                    const float wa = alive ? w4[cs][sstep / 4][sstep % 4] : 0.f;
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) d[cs][cb] = mfma_16x16x4(wa, alive ? g[cb] : 0.f, d[cs][cb]);
                }
            }
        }
        // lane (n16, kq): tokens 16*cs + 4*kq .. +3 of channels n16*CB + cb -> row-major chunk -> stores
        lds_sync();
#pragma unroll
        for (int cs = 0; cs < 2; ++cs) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int tok = 16 * cs + 4 * kq + j;
                if (tok < kTile24) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) chunk[tok * C + n16 * CB + cb] = d[cs][cb][j];
                }
            }
        }
        lds_sync();
        T* out_h = out + (int64_t)b * os.b + (int64_t)h * os.h + (int64_t)i0 * os.n;
#pragma unroll
        for (int q0 = 0; q0 < kTile24 * C / 4; q0 += kWave) {
            const int q = q0 + lane;
            const int tok = q / (C / 4), c4 = q - tok * (C / 4);
            if (q < kTile24 * C / 4 && tok < nt) {
                const F32x4 o = *reinterpret_cast<const F32x4*>(chunk + tok * C + 4 * c4);
                const float v[4] = {o[0], o[1], o[2], o[3]};
                store_streaming(reinterpret_cast<typename QuadIO::raw*>(out_h + (int64_t)tok * os.n + 4 * c4), QuadIO::pack(v));
            }
        }
    }
}

// ---- launch ----------------------------------------------------------------------------------------------------------

template <typename T, int C>
int launch_gather_sum_runs24_c(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                               clusten_strides os, const clusten_attn_shape& s, hipStream_t stream, const int32_t* cid) {
    const int tiles_per_batch = (s.N + kTile24 - 1) / kTile24;
    const int total = s.B * tiles_per_batch;
    hipLaunchKernelGGL((gather_sum_runs24_kernel<T, C>), dim3(xcd_grid(total)), dim3(kWave), 0, stream,
                       static_cast<const T*>(p), static_cast<const T*>(rows), idx, cid, static_cast<T*>(out), s.H, s.N, s.M, rs,
                       os, tiles_per_batch, total);
    return launch_status();
}

template <typename T>
int launch_gather_sum_runs24(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                             clusten_strides os, const clusten_attn_shape& s, hipStream_t stream,
                             const int32_t* cid = nullptr) {
    if constexpr (sizeof(T) == 4) {
        if (s.C == 16) return launch_gather_sum_runs24_c<T, 16>(p, rows, rs, idx, out, os, s, stream, cid);
    }
    if (s.C == 32) return launch_gather_sum_runs24_c<T, 32>(p, rows, rs, idx, out, os, s, stream, cid);
    return launch_gather_sum_runs24_c<T, 64>(p, rows, rs, idx, out, os, s, stream, cid);
}

}  // namespace clusten
