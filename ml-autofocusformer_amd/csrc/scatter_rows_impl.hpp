// scatter_rows: out[b,h,idx[b,i,j],c] += p[b,h,i,j] * x[b,h,i,c]
//
// This is the d_key half of the CLUSTEN QK backward (p = d_attn, x = query; reference kernel
// clusten/src/clustenqk_cuda_kernel.cu:91-132, the fastAtomicAdd line) and the d_value kernel of
// the AV backward (p = attn, x = d_feat; clusten/src/clustenav_cuda_kernel.cu:93-127).
//
// Work decomposition: as in gather_sum — one wave per tile of 8 consecutive tokens, lanes are 64
// consecutive (head, channel) pairs, the p-rows are read through DPP row broadcasts.
//
//   shared-list path — all tokens of the tile carry the same list: the 8 products that go to one
//     destination row are summed in registers and leave the wave as ONE fp32 atomic per (slot,
//     channel): 8x fewer atomics than one per product, and each wave-wide atomic instruction adds
//     to whole contiguous rows.  (Lists of at most 64 slots: such tiles are taken beforehand by
//     scatter_rows_window.hip, which sums many tiles in LDS first, and are skipped here.)
//   union path — lists that differ but are made of runs of 8 slots of which the tile's tokens share most (the
//     neighbourhoods of a cluster-ordered sequence: a run is the 8 members of one cluster; a tile of the model's own
//     lists holds 8-12 distinct runs): the runs are numbered by distinct value as in the forward kernels, p is laid
//     out in LDS by distinct run and member (zero where a token does not hold the run), and the sums over the tile's
//     tokens are one small matrix product per head,  D[run member][c] = P^T (members x 8 tokens) * X (8 tokens x C),
//     on the matrix cores.  One atomic per (distinct run member, channel): 80-100 per lane instead of 384.
//   per-token path — one atomic per product, for any other tile.
//
// The destination is accumulated in fp32: directly in `out` for fp32, in a caller-provided fp32
// workspace that is rounded once at the end for fp16/bf16.  fp64, head dims other than 16/32/64
// and list lengths that are not a multiple of 4 take the element-per-thread kernel.
// The order in which atomics from different waves arrive is not fixed, so the last bits of the
// result can differ from run to run (as they do in the reference).
#pragma once

#include "dpp.hpp"
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {

// One tile of 8 tokens (all heads) of the atomic scatter.
template <typename T, int C, int Q, bool GUARD>
__device__ __forceinline__ void scatter_rows_tile(const T* __restrict__ p, const T* __restrict__ x,
                                                  const int64_t* __restrict__ idx, float* __restrict__ out, int H, int N,
                                                  int M, clusten_strides xs, int tiles_per_batch, int tile) {
    constexpr int HPW = kWave / C;
    constexpr int SLOTS = 16 * Q;
    static_assert(C == 16 || C == 32 || C == 64, "a row of 16 lanes must stay inside one head");
    static_assert(!GUARD || Q == 4, "guarded lists are taken 64 slots at a time");
    typedef typename Quad<T>::raw QuadRaw;
    {
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTileTokens;
    const int nt = min(kTileTokens, N - i0);
    const int lane = threadIdx.x;
    const int c = lane % C;
    const int rl = lane & 15;

    const int64_t* idx_tile = idx + ((int64_t)b * N + i0) * M;
    float* out_b = out + (int64_t)b * H * N * C;

    if ((M & 7) == 0 && M <= 64) {
        // ---- union path: lists made of runs of 8 slots, at most 16 distinct runs in the tile ----
        constexpr int U_MAX = 16;
        constexpr int PS = 9;                        // floats per row of the P^T matrix: odd, rows fall into different banks
        __shared__ float pm[U_MAX * 8 * PS];
        __shared__ int ulist[U_MAX * 8];
        const int R = M >> 3;                        // runs per token
        const int nruns = nt * R;                    // <= 64: lane rho owns run rho = token * R + run
        int v[8];
        {
            const int64_t* run = idx_tile + (int64_t)min(lane, nruns - 1) * 8;
#pragma unroll
            for (int t = 0; t < 8; ++t) v[t] = (int)run[t];
        }
        // 8 consecutive rows, or the short last cluster of the sequence followed by the row 0 its pad slots hold:
        // either way the first row tells the other seven
        const int own = ((N & 7) != 0 && v[0] == N - (N & 7)) ? (N & 7) : 8;
        bool regular = true;
#pragma unroll
        for (int t = 1; t < 8; ++t) regular = regular && (v[t] == (t < own ? v[0] + t : 0));
        const int key = regular ? v[0] : ~lane;      // other runs never merge
        uint64_t remaining = nruns >= 64 ? ~0ull : ((1ull << nruns) - 1);
        bool differ = false;                         // a shared list is better served by the path below
        {
            const int k0 = __shfl(key, lane % R);
            differ = __any((lane < nruns && key != k0) ? 1 : 0) != 0;
        }
        int uslot = 0, U = 0;
        bool first = false;
        while (differ && remaining != 0 && U < U_MAX) {
            const int sl = __builtin_ctzll(remaining);
            const int ks = __builtin_amdgcn_readlane(key, sl);
            const bool hit = key == ks;
            const uint64_t match = __ballot(hit) & remaining;
            if (hit) uslot = U;
            first = first || lane == sl;
            remaining &= ~match;
            ++U;
        }
        if (differ && remaining == 0) {
            if (first) {
#pragma unroll
                for (int t = 0; t < 8; ++t) ulist[uslot * 8 + t] = v[t];
            }
            const int t8 = lane >> 3, m8 = lane & 7;     // build side: token and run member of the lane
            const int r16 = lane & 15, kq = lane >> 4;   // matrix side
            int us[8];                                   // distinct-run number of the lane's token's runs
#pragma unroll
            for (int r = 0; r < 8; ++r) us[r] = __shfl(uslot, min(t8 * R + min(r, R - 1), nruns - 1));
            const int rows_u = 8 * U;
            for (int h = 0; h < H; ++h) {
                __syncthreads();  // the previous head's operand reads are complete (and the row table is written)
                for (int z = lane; z < U_MAX * 8 * PS; z += kWave) pm[z] = 0.f;
                __syncthreads();
                if (t8 < nt) {
                    const T* prow = p + (((int64_t)b * H + h) * N + i0 + t8) * M + m8;
#pragma unroll
                    for (int r = 0; r < 8; ++r) {
                        // the lane owns column t8 of the rows of member m8: repeats of a run by one token add up
                        if (r < R) pm[(us[r] * 8 + m8) * PS + t8] += to_acc(prow[8 * r]);
                    }
                }
                // B operands: x[token 4*s + kq][channel 16*cb + r16]
                float xb[2][C / 16];
                const T* xh = x + (int64_t)b * xs.b + (int64_t)h * xs.h + (int64_t)i0 * xs.n;
#pragma unroll
                for (int sx = 0; sx < 2; ++sx) {
                    const int tok = 4 * sx + kq;
#pragma unroll
                    for (int cb = 0; cb < C / 16; ++cb) {
                        xb[sx][cb] = tok < nt ? to_acc(xh[(int64_t)tok * xs.n + 16 * cb + r16]) : 0.f;
                    }
                }
                __syncthreads();
                float* out_h = out_b + (int64_t)h * N * C;
                for (int blk = 0; blk * 16 < rows_u; ++blk) {
                    const float a0 = pm[(16 * blk + r16) * PS + kq];
                    const float a1 = pm[(16 * blk + r16) * PS + 4 + kq];
                    int drow[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) drow[e] = ulist[min(16 * blk + 4 * kq + e, rows_u - 1)];
#pragma unroll
                    for (int cb = 0; cb < C / 16; ++cb) {
                        F32x4 d = F32x4{0.f, 0.f, 0.f, 0.f};
                        d = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, xb[0][cb], d, 0, 0, 0);
                        d = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, xb[1][cb], d, 0, 0, 0);
                        // lane (r16, kq): members 16*blk + 4*kq .. +3 of channel 16*cb + r16
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (16 * blk + 4 * kq + e < rows_u) {
                                unsafeAtomicAdd(out_h + (int64_t)drow[e] * C + 16 * cb + r16, d[e]);
                            }
                        }
                    }
                }
            }
            return;
        }
    }

    for (int h0 = 0; h0 < H; h0 += HPW) {
        const int h_raw = h0 + lane / C;
        const bool head_ok = h_raw < H;
        const int h = min(h_raw, H - 1);
        const int lane_off = h * N * C + c;  // out is contiguous (B,H,N,C)
        const T* p_head = p + (((int64_t)b * H + h) * N + i0) * M;
        const T* x_lane = x + (int64_t)b * xs.b + (int64_t)h * xs.h + (int64_t)i0 * xs.n + c;

        // x-rows of the tile; tokens past the end of a partial tile contribute nothing
        float xv[kTileTokens];
#pragma unroll
        for (int t = 0; t < kTileTokens; ++t) {
            const float v = to_acc(x_lane[(int64_t)min(t, nt - 1) * xs.n]);
            xv[t] = (t < nt) ? v : 0.f;
        }

        for (int j0 = 0; j0 < M; j0 += kWave) {
            const int mc = min(kWave, M - j0);
            const int slot = min(lane, mc - 1);

            int list[kTileTokens];
            bool same = true;
            {
                int64_t wide[kTileTokens];
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) wide[t] = idx_tile[(int64_t)min(t, nt - 1) * M + j0 + slot];
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) {
                    same = same && (wide[t] == wide[0]);
                    list[t] = (int)wide[t];
                }
            }
            const bool shared_list = __all(same ? 1 : 0) != 0;

            float pv[kTileTokens][4];
            {
                const int q4 = min(4 * rl, mc - 4);
                QuadRaw raw[kTileTokens];
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) {
                    raw[t] = *reinterpret_cast<const QuadRaw*>(p_head + (int64_t)min(t, nt - 1) * M + j0 + q4);
                }
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) {
                    Quad<T>::unpack(raw[t], pv[t]);
                    if (t >= nt) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) pv[t][e] = 0.f;
                    }
                }
            }

            if (shared_list) {
                static_for<0, SLOTS>([&](auto ji) {
                    constexpr int j = decltype(ji)::value;
                    if (!GUARD || j < mc) {
                        float sum = 0.f;
                        fma4_rowlane<j / 4>(sum, pv[0][j % 4], pv[1][j % 4], pv[2][j % 4], pv[3][j % 4], xv[0], xv[1],
                                            xv[2], xv[3]);
                        fma4_rowlane<j / 4>(sum, pv[4][j % 4], pv[5][j % 4], pv[6][j % 4], pv[7][j % 4], xv[4], xv[5],
                                            xv[6], xv[7]);
                        const int row = __builtin_amdgcn_readlane(list[0], j);
                        float* dst = out_b + (int64_t)row * C;
                        if (head_ok) unsafeAtomicAdd(dst + lane_off, sum);
                    }
                });
            } else {
                static_for<0, kTileTokens>([&](auto ti) {
                    constexpr int t = decltype(ti)::value;
                    static_for<0, SLOTS>([&](auto ji) {
                        constexpr int j = decltype(ji)::value;
                        if (!GUARD || j < mc) {
                            float prod = 0.f;
                            fma1_rowlane<j / 4>(prod, pv[t][j % 4], xv[t]);
                            const int row = __builtin_amdgcn_readlane(list[t], j);
                            float* dst = out_b + (int64_t)row * C;
                            if (head_ok && t < nt) unsafeAtomicAdd(dst + lane_off, prod);
                        }
                    });
                });
            }
        }
    }
    }
}

constexpr int kScatterGroupTiles = 8;   // tiles of a workgroup when most tiles are expected to be skipped

// A workgroup takes `group` consecutive tiles: 1 when this kernel has every tile, kScatterGroupTiles when the window
// kernel ran first and left one byte per tile in `handled` (non-zero: added there).  With lists shared by the tokens of
// a tile nothing is left for this kernel, and a launch of one workgroup per tile costs 12 us at 50 000 tiles just for
// its waves to start and read their byte; a group's eight bytes are read with one load and the grid is an eighth.
template <typename T, int C, int Q, bool GUARD>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4))) void scatter_rows_tile_kernel(
    const T* __restrict__ p, const T* __restrict__ x, const int64_t* __restrict__ idx, float* __restrict__ out, int H,
    int N, int M, clusten_strides xs, int tiles_per_batch, int total_tiles, int group, int total_groups,
    const int32_t* __restrict__ only_if, const uint8_t* __restrict__ handled) {
    if (only_if != nullptr && *only_if == 0) return;   // the cluster-by-cluster kernel has these lists
    const int g = xcd_tile(blockIdx.x, total_groups);
    if (g < 0) return;
    const int tile0 = g * group;
    const int lane = threadIdx.x;
    const int mine = tile0 + lane;
    bool open = lane < group && mine < total_tiles;
    if (open && handled != nullptr) open = handled[mine] == 0;   // the window kernel has added the others
    uint64_t todo = __ballot(open);
    while (todo != 0) {
        const int k = __builtin_ctzll(todo);
        todo &= todo - 1;
        __syncthreads();   // the LDS tables of the tile before have been read
        scatter_rows_tile<T, C, Q, GUARD>(p, x, idx, out, H, N, M, xs, tiles_per_batch, tile0 + k);
    }
}

// One thread per (b,h,i,c); loops over the list with one atomic per product.  Any dtype whose
// accumulation type A has a hardware atomic add (float, double).
template <typename T, typename A>
__global__ __launch_bounds__(256) void scatter_rows_elem_kernel(const T* __restrict__ p, const T* __restrict__ x,
                                                                const int64_t* __restrict__ idx, A* __restrict__ out,
                                                                int B, int H, int N, int C, int M,
                                                                clusten_strides xs, const int32_t* __restrict__ only_if) {
    if (only_if != nullptr && *only_if == 0) return;
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
        const A xval = to_acc(x[b * xs.b + h * xs.h + i * xs.n + c]);
        A* dst = out + ((int64_t)b * H + h) * N * C + c;
        for (int j = 0; j < M; ++j) unsafeAtomicAdd(dst + list[j] * C, (A)to_acc(prow[j]) * xval);
    }
}

template <typename T, int C, int Q, bool GUARD>
int scatter_tile_q(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* out,
                   const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if, const uint8_t* handled) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int group = handled != nullptr ? kScatterGroupTiles : 1;
    const int groups = (total + group - 1) / group;
    hipLaunchKernelGGL((scatter_rows_tile_kernel<T, C, Q, GUARD>), dim3(xcd_grid(groups)), dim3(kWave), 0, stream,
                       static_cast<const T*>(p), static_cast<const T*>(x), idx, out, s.H, s.N, s.M, xs,
                       tiles_per_batch, total, group, groups, only_if, handled);
    return launch_status();
}

template <typename T, int C>
int scatter_tile(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* out,
                 const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if, const uint8_t* handled) {
    if (s.M == 48) return scatter_tile_q<T, C, 3, false>(p, x, xs, idx, out, s, stream, only_if, handled);
    return scatter_tile_q<T, C, 4, true>(p, x, xs, idx, out, s, stream, only_if, handled);
}

template <typename T, typename A>
int scatter_elem(const void* p, const void* x, clusten_strides xs, const int64_t* idx, A* out,
                 const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if = nullptr) {
    const int64_t total = (int64_t)s.B * s.H * s.N * s.C;
    const int64_t want = (total + 255) / 256;
    const int grid = (int)(want < (int64_t)1 << 20 ? want : (int64_t)1 << 20);
    hipLaunchKernelGGL((scatter_rows_elem_kernel<T, A>), dim3(grid), dim3(256), 0, stream, static_cast<const T*>(p),
                       static_cast<const T*>(x), idx, out, s.B, s.H, s.N, s.C, s.M, xs, only_if);
    return launch_status();
}

// Whether the tile kernel takes this scatter (otherwise one thread per element does).
template <typename T>
bool scatter_tiles_ok(const void* p, const clusten_attn_shape& s) {
    return s.M % 4 == 0 && (reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T))) == 0 && (s.C == 16 || s.C == 32 || s.C == 64);
}

// Accumulate into the zeroed fp32 buffer `acc32` (which is `out` itself for fp32 storage).  `handled` (may be null)
// marks the tiles that the window kernel has added already; it is read only when scatter_tiles_ok().
template <typename T>
int scatter_rows_typed(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32,
                       const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if, const uint8_t* handled) {
    if (scatter_tiles_ok<T>(p, s)) {
        switch (s.C) {
            case 16: return scatter_tile<T, 16>(p, x, xs, idx, acc32, s, stream, only_if, handled);
            case 32: return scatter_tile<T, 32>(p, x, xs, idx, acc32, s, stream, only_if, handled);
            case 64: return scatter_tile<T, 64>(p, x, xs, idx, acc32, s, stream, only_if, handled);
            default: break;
        }
    }
    return scatter_elem<T, float>(p, x, xs, idx, acc32, s, stream, only_if);
}

}  // namespace clusten
