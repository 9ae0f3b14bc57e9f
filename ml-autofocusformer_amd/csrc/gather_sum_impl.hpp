// gather_sum: out[b,h,i,c] = sum_j p[b,h,i,j] * rows[b,h,idx[b,i,j],c]
//
// This is the CLUSTEN AV forward (p = attn, rows = value; reference kernel
// clusten/src/clustenav_cuda_kernel.cu:18-50) and the d_query half of the QK backward
// (p = d_attn, rows = key; clusten/src/clustenqk_cuda_kernel.cu:91-132, the dq_update sum).
//
// Work decomposition.  One wave owns a tile of 8 consecutive tokens of one batch element.  Its 64
// lanes are 64 consecutive (head, channel) pairs, so with head dim 32 a wave covers two heads and
// a gathered row is read as one contiguous run per head.  The tile's neighbour lists are read once.
// The p-rows of the tile are loaded so that each row of 16 lanes holds 16 consecutive slots of its
// own head; the FMAs read them through DPP row broadcasts (see dpp.hpp).
//
//   shared-list path — all tokens of the tile carry the same list: every gathered element is
//     loaded once and used for the 8 tokens (8 FMAs per load).
//   per-token path — any other tile: one load per token and slot.
//
// Head dims other than 16/32/64, list lengths that are not a multiple of 4, unaligned p and fp64
// take the element-per-thread kernel at the bottom of the file.
//
// This header holds the templates; gather_sum_{f32,f16,bf16}.hip instantiate them per storage type
// so that the translation units build in parallel, gather_sum.hip holds the dtype dispatch.
#pragma once

#include "dpp.hpp"
#include "launch.hpp"

namespace clusten {

// GUARD = false: the list has exactly 16*Q slots.  GUARD = true: any list length that is a
// multiple of 4, taken 64 slots at a time (Q = 4) with every slot range-checked.
template <typename T, int C, int Q, bool GUARD>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4))) void gather_sum_tile_kernel(const T* __restrict__ p, const T* __restrict__ rows,
                                                                const int64_t* __restrict__ idx,
                                                                T* __restrict__ out, int H, int N, int M,
                                                                clusten_strides rs, clusten_strides os,
                                                                int tiles_per_batch, int total_tiles) {
    constexpr int HPW = kWave / C;  // heads covered by the wave's 64 lanes
    constexpr int SLOTS = 16 * Q;   // neighbour slots taken per chunk
    static_assert(C == 16 || C == 32 || C == 64, "a row of 16 lanes must stay inside one head");
    static_assert(!GUARD || Q == 4, "guarded lists are taken 64 slots at a time");
    typedef typename Quad<T>::raw QuadRaw;

    const int tile = xcd_tile(blockIdx.x, total_tiles);
    if (tile < 0) return;
    {
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTileTokens;
    const int nt = min(kTileTokens, N - i0);
    const int lane = threadIdx.x;
    const int c = lane % C;
    const int rl = lane & 15;  // lane inside its row of 16

    const T* rows_b = rows + (int64_t)b * rs.b;
    const int64_t* idx_tile = idx + ((int64_t)b * N + i0) * M;

    for (int h0 = 0; h0 < H; h0 += HPW) {
        const int h_raw = h0 + lane / C;
        const bool head_ok = h_raw < H;
        const int h = min(h_raw, H - 1);  // lanes past the last head repeat it; only their store is masked
        const int lane_off = h * (int)rs.h + c;
        const T* p_head = p + (((int64_t)b * H + h) * N + i0) * M;

        float acc[kTileTokens];
#pragma unroll
        for (int t = 0; t < kTileTokens; ++t) acc[t] = 0.f;

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

            // p-rows: row-lane n of every row of 16 holds slots 4n..4n+3 of the lane's head, per token
            float pv[kTileTokens][4];
            {
                const int q4 = min(4 * rl, mc - 4);
                QuadRaw raw[kTileTokens];
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) {
                    raw[t] = *reinterpret_cast<const QuadRaw*>(p_head + (int64_t)min(t, nt - 1) * M + j0 + q4);
                }
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) Quad<T>::unpack(raw[t], pv[t]);
            }

            if (shared_list) {
                float val[SLOTS];
                slot_pipeline<SLOTS, 16>(
                    [&](auto ji) {
                        constexpr int j = decltype(ji)::value;
                        const int row = __builtin_amdgcn_readlane(list[0], min(j, mc - 1));
                        const T* rowp = rows_b + (int64_t)row * rs.n;  // wave-uniform base, per-lane 32-bit offset
                        val[j] = to_acc(rowp[lane_off]);
                    },
                    [&](auto ji) {
                        constexpr int j = decltype(ji)::value;
                        if (!GUARD || j < mc) {
                            fma8_rowlane<j / 4>(acc, pv[0][j % 4], pv[1][j % 4], pv[2][j % 4], pv[3][j % 4],
                                                pv[4][j % 4], pv[5][j % 4], pv[6][j % 4], pv[7][j % 4], val[j]);
                        }
                    });
            } else {
                static_for<0, kTileTokens>([&](auto ti) {
                    constexpr int t = decltype(ti)::value;
                    float val[SLOTS];
                    slot_pipeline<SLOTS, 16>(
                        [&](auto ji) {
                            constexpr int j = decltype(ji)::value;
                            const int row = __builtin_amdgcn_readlane(list[t], min(j, mc - 1));
                            const T* rowp = rows_b + (int64_t)row * rs.n;
                            val[j] = to_acc(rowp[lane_off]);
                        },
                        [&](auto ji) {
                            constexpr int j = decltype(ji)::value;
                            if (!GUARD || j < mc) fma1_rowlane<j / 4>(acc[t], pv[t][j % 4], val[j]);
                        });
                });
            }
        }

        T* out_lane = out + (int64_t)b * os.b + (int64_t)h * os.h + (int64_t)i0 * os.n + c;
#pragma unroll
        for (int t = 0; t < kTileTokens; ++t) {
            if (head_ok && t < nt) out_lane[(int64_t)t * os.n] = from_acc<T>(acc[t]);
        }
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

template <typename T, int C, int Q, bool GUARD>
int launch_tile_q(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                  clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const int grid = xcd_grid(total);
    hipLaunchKernelGGL((gather_sum_tile_kernel<T, C, Q, GUARD>), dim3(grid), dim3(kWave), 0, stream,
                       static_cast<const T*>(p), static_cast<const T*>(rows), idx, static_cast<T*>(out), s.H, s.N,
                       s.M, rs, os, tiles_per_batch, total);
    return launch_status();
}

template <typename T, int C>
int launch_tile(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out, clusten_strides os,
                const clusten_attn_shape& s, hipStream_t stream) {
    // 48 slots is the neighbourhood size of every 224x224 model; it gets the unguarded kernel
    if (s.M == 48) return launch_tile_q<T, C, 3, false>(p, rows, rs, idx, out, os, s, stream);
    return launch_tile_q<T, C, 4, true>(p, rows, rs, idx, out, os, s, stream);
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

template <typename T>
int gather_sum_typed(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out, clusten_strides os,
                 const clusten_attn_shape& s, hipStream_t stream) {
    // the p quads are 4*sizeof(T)-byte accesses at slot offsets that are multiples of 4
    const bool quads_ok = s.M % 4 == 0 && (reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T))) == 0 &&
                          slice_fits_int32(rs, s.H, s.N, s.C);
    if (quads_ok) {
        switch (s.C) {
            case 16: return launch_tile<T, 16>(p, rows, rs, idx, out, os, s, stream);
            case 32: return launch_tile<T, 32>(p, rows, rs, idx, out, os, s, stream);
            case 64: return launch_tile<T, 64>(p, rows, rs, idx, out, os, s, stream);
            default: break;
        }
    }
    return launch_elem<T>(p, rows, rs, idx, out, os, s, stream);
}


}  // namespace clusten
