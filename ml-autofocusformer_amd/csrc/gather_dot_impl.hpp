// gather_dot: out[b,h,i,j] = sum_c a[b,h,i,c] * rows[b,h,idx[b,i,j],c]
//
// This is the CLUSTEN QK forward (a = query, rows = key; reference kernel
// clusten/src/clustenqk_cuda_kernel.cu:18-49) and the d_attn half of the AV backward
// (a = d_feat, rows = value; clusten/src/clustenav_cuda_kernel.cu:129-160).
//
// Work decomposition.  One wave owns a tile of 8 consecutive tokens of one batch element and
// walks all heads, so the int64 neighbour lists of the tile are read from HBM exactly once.
// Lane j of the wave owns neighbour slot j (slots are taken 64 at a time when M > 64).
//
//   shared-list path — all tokens of the tile carry the same list (true for every tile of a
//     cluster-ordered token sequence whose cluster shares its neighbourhood).  The M gathered rows
//     are fetched once per head with row-coalesced 16-byte accesses (consecutive lanes cover one
//     row, a wave access covers 64/pieces-per-row whole rows), turned through LDS so that lane j
//     ends up with row j in registers, and reused for the 8 tokens: 8 FMAs per gathered element.
//     The a-rows are wave-uniform and come in through the scalar data path.
//   per-token path — any other tile: lane j gathers its own row for every token.  Exact for
//     arbitrary indices (duplicates, any order), only slower.
//
// Rows whose start is not 16-byte aligned, head dims other than 16/32/64 and fp64 take the
// element-per-thread kernel at the bottom of the file.
//
// This header holds the templates; gather_dot_{f32,f16,bf16}.hip instantiate them per storage type
// so that the translation units build in parallel, gather_dot.hip holds the dtype dispatch.
#pragma once

#include "dpp.hpp"
#include "launch.hpp"

namespace clusten {

template <typename T, int C, int Q>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4))) void gather_dot_tile_kernel(const T* __restrict__ a, const T* __restrict__ rows,
                                                                const int64_t* __restrict__ idx,
                                                                T* __restrict__ out, int H, int N, int M,
                                                                clusten_strides as, clusten_strides rs,
                                                                int tiles_per_batch, int total_tiles) {
    constexpr int EPP = PieceOf<T>::kElems;          // elements per 16-byte piece
    constexpr int PPR = C / EPP;                     // pieces per row
    constexpr int RPP = kWave / PPR;                 // rows covered by one wave-wide access
    constexpr int PITCH = PPR + 1;                   // LDS row pitch in pieces: the pad keeps row-per-lane reads conflict free
    constexpr int NPASS = (16 * Q + RPP - 1) / RPP;  // wave-wide accesses that cover the 16*Q slots of a chunk
    constexpr int NA = kTileTokens * C / (16 * EPP); // pieces per lane that hold the tile's a-rows (each row of 16 lanes holds all of them)
    static_assert(C % EPP == 0 && kWave % PPR == 0, "unsupported head dim");
    static_assert((kTileTokens * C) % (16 * EPP) == 0, "the a-tile must fill whole 16-lane rows");
    static_assert(Q >= 1 && Q <= 4, "a chunk holds 16, 32, 48 or 64 neighbour slots");

    extern __shared__ Piece lds_rows[];  // [kWave][PITCH] pieces, then kWave ints
    int* lds_idx = reinterpret_cast<int*>(lds_rows + kWave * PITCH);

    const int tile = xcd_tile(blockIdx.x, total_tiles);
    if (tile < 0) return;
    const int b = tile / tiles_per_batch;
    const int i0 = (tile - b * tiles_per_batch) * kTileTokens;
    const int nt = min(kTileTokens, N - i0);
    const int lane = threadIdx.x;

    const T* a_tile = a + (int64_t)b * as.b + (int64_t)i0 * as.n;
    const T* rows_b = rows + (int64_t)b * rs.b;
    T* out_tile = out + ((int64_t)b * H * N + i0) * M;
    const int64_t* idx_tile = idx + ((int64_t)b * N + i0) * M;

    const int piece = lane % PPR;  // row-coalesced fetch: lane covers piece `piece` of row pass*RPP + sub
    const int sub = lane / PPR;

    // a-tile: flat element f = t*C + c of the tile's 8 a-rows sits in piece f / (16*EPP) of row-lane
    // (f / EPP) % 16, element f % EPP.  Tokens past the end of a partial tile repeat its last token.
    int a_off[NA];  // element offsets inside one batch element fit 32 bits (checked on the host)
#pragma unroll
    for (int m = 0; m < NA; ++m) {
        const int f0 = (16 * m + (lane & 15)) * EPP;
        a_off[m] = min(f0 / C, nt - 1) * (int)as.n + f0 % C;
    }
    auto load_a = [&](const T* a_head, Piece (&dst)[NA]) {
#pragma unroll
        for (int m = 0; m < NA; ++m) dst[m] = *reinterpret_cast<const Piece*>(a_head + a_off[m]);
    };
    // acc[t] += sum_c a[t][c] * kr[c], the a operand read across the row of 16 lanes
    auto dot_token = [&](auto ti, const Piece (&av)[NA], const float (&kr)[C], float& acc) {
        constexpr int t = decltype(ti)::value;
        float aflat[NA * EPP];
#pragma unroll
        for (int m = 0; m < NA; ++m) {
#pragma unroll
            for (int e = 0; e < EPP; ++e) aflat[m * EPP + e] = piece_get<T>(av[m], e);
        }
        static_for<0, C / 4>([&](auto gi) {
            constexpr int f = t * C + 4 * decltype(gi)::value;
            constexpr int m = f / (16 * EPP);
            constexpr int n = (f / EPP) % 16;
            constexpr int e = f % EPP;
            constexpr int c = 4 * decltype(gi)::value;
            fma4_rowlane<n>(acc, aflat[m * EPP + e], aflat[m * EPP + e + 1], aflat[m * EPP + e + 2],
                            aflat[m * EPP + e + 3], kr[c], kr[c + 1], kr[c + 2], kr[c + 3]);
        });
    };

    for (int j0 = 0; j0 < M; j0 += kWave) {
        const int mc = min(kWave, M - j0);
        const bool active = lane < mc;
        const int slot = min(lane, mc - 1);  // lanes past the list repeat its last slot; only their store is masked

        int64_t list[kTileTokens];
#pragma unroll
        for (int t = 0; t < kTileTokens; ++t) {
            list[t] = idx_tile[(int64_t)min(t, nt - 1) * M + j0 + slot];
        }
        bool same = true;
#pragma unroll
        for (int t = 1; t < kTileTokens; ++t) same = same && (list[t] == list[0]);
        const bool shared_list = __all(same ? 1 : 0) != 0;

        if (shared_list) {
            __syncthreads();  // the previous chunk's readers are done with the LDS
            lds_idx[lane] = (int)list[0];
            __syncthreads();
            int src_off[NPASS];  // element offset of this lane's piece inside one (b,h) slice, per pass
#pragma unroll
            for (int pass = 0; pass < NPASS; ++pass) {
                const int r = min(pass * RPP + sub, mc - 1);
                src_off[pass] = lds_idx[r] * (int)rs.n + piece * EPP;
            }
            Piece stage[NPASS];
            Piece a_stage[NA];
#pragma unroll
            for (int pass = 0; pass < NPASS; ++pass) {
                stage[pass] = *reinterpret_cast<const Piece*>(rows_b + src_off[pass]);
            }
            load_a(a_tile, a_stage);
            for (int h = 0; h < H; ++h) {
#pragma unroll
                for (int pass = 0; pass < NPASS; ++pass) {
                    lds_rows[(pass * RPP + sub) * PITCH + piece] = stage[pass];
                }
                Piece a_cur[NA];
#pragma unroll
                for (int m = 0; m < NA; ++m) a_cur[m] = a_stage[m];
                __syncthreads();
                if (h + 1 < H) {  // the next head's rows travel while this head is computed
                    const T* rows_next = rows_b + (int64_t)(h + 1) * rs.h;
#pragma unroll
                    for (int pass = 0; pass < NPASS; ++pass) {
                        stage[pass] = *reinterpret_cast<const Piece*>(rows_next + src_off[pass]);
                    }
                    load_a(a_tile + (int64_t)(h + 1) * as.h, a_stage);
                }
                float kr[C];
#pragma unroll
                for (int p = 0; p < PPR; ++p) {
                    const Piece pc = lds_rows[lane * PITCH + p];
#pragma unroll
                    for (int e = 0; e < EPP; ++e) kr[p * EPP + e] = piece_get<T>(pc, e);
                }
                __syncthreads();  // rows are in registers; the LDS may be refilled for the next head
                float acc[kTileTokens];
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) acc[t] = 0.f;
                static_for<0, kTileTokens>([&](auto ti) { dot_token(ti, a_cur, kr, acc[decltype(ti)::value]); });
                T* out_head = out_tile + (int64_t)h * N * M + j0 + lane;
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) {
                    if (active && t < nt) out_head[(int64_t)t * M] = from_acc<T>(acc[t]);
                }
            }
        } else {
            for (int h = 0; h < H; ++h) {
                const T* rows_bh = rows_b + (int64_t)h * rs.h;
                Piece a_cur[NA];
                load_a(a_tile + (int64_t)h * as.h, a_cur);
                float acc[kTileTokens];
                static_for<0, kTileTokens>([&](auto ti) {
                    constexpr int t = decltype(ti)::value;
                    const Piece* src = reinterpret_cast<const Piece*>(rows_bh + list[t] * rs.n);
                    float kr[C];
#pragma unroll
                    for (int p = 0; p < PPR; ++p) {
                        const Piece pc = src[p];
#pragma unroll
                        for (int e = 0; e < EPP; ++e) kr[p * EPP + e] = piece_get<T>(pc, e);
                    }
                    acc[t] = 0.f;
                    dot_token(ti, a_cur, kr, acc[t]);
                });
                T* out_head = out_tile + (int64_t)h * N * M + j0 + lane;
#pragma unroll
                for (int t = 0; t < kTileTokens; ++t) {
                    if (active && t < nt) out_head[(int64_t)t * M] = from_acc<T>(acc[t]);
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

template <typename T, int C, int Q>
int launch_tile_q(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx,
                  void* out, const clusten_attn_shape& s, hipStream_t stream) {
    constexpr int PPR = C / PieceOf<T>::kElems;
    const int tiles_per_batch = (s.N + kTileTokens - 1) / kTileTokens;
    const int total = s.B * tiles_per_batch;
    const size_t lds = (size_t)kWave * (PPR + 1) * sizeof(Piece) + kWave * sizeof(int);
    hipLaunchKernelGGL((gather_dot_tile_kernel<T, C, Q>), dim3(xcd_grid(total)), dim3(kWave), lds, stream,
                       static_cast<const T*>(a), static_cast<const T*>(rows), idx, static_cast<T*>(out), s.H, s.N,
                       s.M, as, rs, tiles_per_batch, total);
    return launch_status();
}

// Lists of up to 48 slots (the model's neighbourhood size) are one chunk of 48; anything longer goes 64 slots at a time.
template <typename T, int C>
int launch_tile(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                const clusten_attn_shape& s, hipStream_t stream) {
    if (s.M <= 48) return launch_tile_q<T, C, 3>(a, as, rows, rs, idx, out, s, stream);
    return launch_tile_q<T, C, 4>(a, as, rows, rs, idx, out, s, stream);
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

template <typename T>
int gather_dot_typed(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                 const clusten_attn_shape& s, hipStream_t stream) {
    const bool vec_ok = rows_aligned16(rows, rs, sizeof(T)) && rows_aligned16(a, as, sizeof(T)) &&
                        slice_fits_int32(rs, s.H, s.N, s.C) && slice_fits_int32(as, s.H, s.N, s.C);
    if (vec_ok) {
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
