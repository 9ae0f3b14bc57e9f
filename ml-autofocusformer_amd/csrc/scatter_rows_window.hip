// scatter_rows_window: the atomic scatter of scatter_rows (scatter_rows_impl.hpp) for tiles whose 8 tokens share one
// list, with the sums of many neighbouring tiles collected in LDS before they reach memory.
//
//   out[b,h,idx[b,i,j],c] += p[b,h,i,j] * x[b,h,i,c]      (clusten/src/clustenqk_cuda_kernel.cu:91-132,
//                                                          clusten/src/clustenav_cuda_kernel.cu:93-127)
//
// Neighbour lists name rows near their own token, so consecutive tiles add to the same few hundred rows.  A workgroup
// of 16 waves takes G consecutive tiles of one image and keeps an fp32 window of the destination rows around them in
// LDS: 128 KB of cells, at 32 channels 1024 rows for 64 tiles, [first token - 256, first token + 768).  Per head:
// every wave forms, for each of its tiles, D[slot][c] = sum_t p[t][slot] * x[t][c] on the matrix cores (operands
// straight from memory in the instruction's layout, those of the wave's next tile requested before the present one
// is used) and adds D into the window; a row outside the window is added to memory directly.  After a barrier the
// non-zero cells of the window leave as one memory atomic each and are cleared for the next head.  A row is inside
// the windows of two workgroups, so it receives two memory atomics per channel instead of one per tile that names it
// (six at 48 neighbours).
//
// The additions to the window are compare-and-swap loops on the cells' bits, not `ds_add_f32`: this device adds
// floats in LDS one lane at a time (measured: 193 clocks per 64-lane instruction, whatever the addresses; an integer
// add takes 5, a read and a write 6-10), which made the first form of this kernel 2.7 times slower than the atomics
// to memory it replaces.  Cells are read, then swapped, eight at a time per lane; a lane goes round again only when
// another wave, or another lane naming the same row, changed its cell in between.
//
// Which tiles have one list is found here and written to `handled` (one byte per tile); the tile kernel that follows
// skips those tiles and takes the rest, so the two kernels together add every product exactly once.
//
// Measured at B128 H2 N3136 C32 M48 fp32 on lists shared by each cluster of 8 tokens (+-256-token window): 320 us
// against the 471 us of one memory atomic per (tile, slot, channel).  Of the 320: finding the shared lists and
// clearing the window 60, operand loads 60, matrix products and their row numbers 70, the additions 100, the
// window's way to memory 45 - one workgroup per CU (the window fills its LDS), so these do not overlap.
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kWindowWaves = 16;
constexpr int kWindowCells = 32768;   // fp32 cells of the window, without the padding

// Tiles of a group: their tokens span half the window, and a wave has at most four tiles (their lists stay in registers)
constexpr int window_group_tiles(int C) { return kWindowCells / C / 16 < 64 ? kWindowCells / C / 16 : 64; }

template <typename T, int C>
__global__ __launch_bounds__(kWindowWaves* kWave) void scatter_rows_window_kernel(
    const T* __restrict__ p, const T* __restrict__ x, const int64_t* __restrict__ idx, float* __restrict__ out,
    uint8_t* __restrict__ handled, int H, int N, int M, clusten_strides xs, int tiles_per_image, int groups_per_image,
    int total_groups, const int32_t* __restrict__ only_if) {
    constexpr int ROWS = kWindowCells / C;
    constexpr int G = window_group_tiles(C);     // tiles of a group
    constexpr int TPW = G / kWindowWaves;        // tiles of a wave
    constexpr int STRIDE = C + 1;                // odd: the rows of one atomic instruction fall into different banks
    extern __shared__ float window[];            // ROWS * STRIDE

    if (only_if != nullptr && *only_if == 0) return;   // the cluster-by-cluster kernel has these lists
    const int unit = xcd_tile(blockIdx.x, total_groups);
    if (unit < 0) return;
    const int b = unit / groups_per_image;
    const int g = unit - b * groups_per_image;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int r16 = lane & 15, kq = lane >> 4;
    // first row of the window (may lie before the image): as many rows before the group's tokens as after them
    const int w0 = g * G * kTileTokens - (ROWS - G * kTileTokens) / 2;

    // the lists of the wave's tiles: lane j keeps slot j of a list that all tokens of the tile share
    int rows[TPW];
    uint32_t ok = 0;
#pragma unroll
    for (int k = 0; k < TPW; ++k) {
        const int tile = g * G + wave + kWindowWaves * k;
        rows[k] = 0;
        if (tile < tiles_per_image) {
            const int i0 = tile * kTileTokens;
            const int nt = min(kTileTokens, N - i0);
            const int64_t* lists = idx + ((int64_t)b * N + i0) * M + min(lane, M - 1);
            int64_t wide[kTileTokens];
#pragma unroll
            for (int t = 0; t < kTileTokens; ++t) wide[t] = lists[(int64_t)min(t, nt - 1) * M];
            bool same = true;
#pragma unroll
            for (int t = 1; t < kTileTokens; ++t) same = same && wide[t] == wide[0];
            const bool shared_list = __all(same ? 1 : 0) != 0;
            rows[k] = (int)wide[0];
            if (shared_list) ok |= 1u << k;
            if (lane == 0) handled[(int64_t)b * tiles_per_image + tile] = shared_list ? 1 : 0;
        }
    }
    for (int z = tid; z < ROWS * STRIDE; z += kWindowWaves * kWave) window[z] = 0.f;
    // nothing to add: the tile kernel has every tile of the group
    if (__syncthreads_or(ok != 0 ? 1 : 0) == 0) return;

    // Operands of one tile and head in the layout of the matrix instruction, straight from memory:
    //   A: p[token 4 s + kq][slot 16 blk + r16]        B: x[token 4 s + kq][channel 16 cb + r16]
    // Those of the wave's next tile are requested before the present tile's sums are added to the window.
    const int blocks = (M + 15) >> 4;
    struct Operands {
        T a[2][4];
        T xb[2][C / 16];
    };
    auto fetch = [&](int k, int h, Operands& o) {
        const int tile = min(g * G + wave + kWindowWaves * k, tiles_per_image - 1);   // a tile past the end: not used
        const int i0 = tile * kTileTokens;
        const int nt = min(kTileTokens, N - i0);
        const T* ph = p + (((int64_t)b * H + h) * N + i0) * M;
        const T* xh = x + (int64_t)b * xs.b + (int64_t)h * xs.h + (int64_t)i0 * xs.n;
#pragma unroll
        for (int sx = 0; sx < 2; ++sx) {
            const int tok = min(4 * sx + kq, nt - 1);
#pragma unroll
            for (int cb = 0; cb < C / 16; ++cb) o.xb[sx][cb] = xh[(uint32_t)(tok * (int)xs.n + 16 * cb + r16)];
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                if (blk < blocks) o.a[sx][blk] = ph[(uint32_t)(tok * M + min(16 * blk + r16, M - 1))];
            }
        }
    };
    uint32_t* cells = reinterpret_cast<uint32_t*>(window);
    constexpr bool AHEAD = C <= 32;    // (at 64 channels two sets of operands do not fit the registers)
    Operands cur, nxt;
    if (AHEAD) fetch(0, 0, cur);
    for (int h = 0; h < H; ++h) {
        float* out_h = out + ((int64_t)b * H + h) * N * C;
#pragma unroll 1
        for (int k = 0; k < TPW; ++k) {
            if (!AHEAD) {
                if ((ok >> k & 1u) != 0) fetch(k, h, cur);
            } else if (k + 1 < TPW) {
                fetch(k + 1, h, nxt);
            } else if (h + 1 < H) {
                fetch(0, h + 1, nxt);
            }
            const Operands now = cur;
            if (AHEAD) cur = nxt;
            if ((ok >> k & 1u) == 0) continue;
            const int nt = min(kTileTokens, N - (g * G + wave + kWindowWaves * k) * kTileTokens);
            int rows_k = rows[0];
#pragma unroll
            for (int kk = 1; kk < TPW; ++kk) rows_k = k == kk ? rows[kk] : rows_k;
            float xb[2][C / 16];
#pragma unroll
            for (int sx = 0; sx < 2; ++sx) {
#pragma unroll
                for (int cb = 0; cb < C / 16; ++cb) xb[sx][cb] = 4 * sx + kq < nt ? to_acc(now.xb[sx][cb]) : 0.f;
            }
#pragma unroll 1
            for (int blk = 0; blk < blocks; ++blk) {
                T ab[2] = {now.a[0][0], now.a[1][0]};
#pragma unroll
                for (int bb = 1; bb < 4; ++bb) {
                    ab[0] = blk == bb ? now.a[0][bb] : ab[0];
                    ab[1] = blk == bb ? now.a[1][bb] : ab[1];
                }
                const bool slot_ok = 16 * blk + r16 < M;
                const float a0 = (slot_ok && kq < nt) ? to_acc(ab[0]) : 0.f;
                const float a1 = (slot_ok && 4 + kq < nt) ? to_acc(ab[1]) : 0.f;
                // the lane's results: slots 16 blk + 4 kq .. + 3 of channel 16 cb + r16
                int drow[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) drow[e] = __shfl(rows_k, min(16 * blk + 4 * kq + e, M - 1));
                // the sums are added by compare-and-swap on the cells' bits: all cells of the block are read, then
                // swapped, and only the lanes that lost a race go round again
                // ... two blocks of 16 channels at a time
                constexpr int CB = C >= 32 ? 2 : 1;
#pragma unroll 1
                for (int c0 = 0; c0 < C / 16; c0 += CB) {
                    F32x4 d[CB];
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        float b0 = xb[0][cb], b1 = xb[1][cb];
#pragma unroll
                        for (int cc = CB; cc < C / 16; cc += CB) {
                            b0 = c0 == cc ? xb[0][cc + cb] : b0;
                            b1 = c0 == cc ? xb[1][cc + cb] : b1;
                        }
                        d[cb] = F32x4{0.f, 0.f, 0.f, 0.f};
                        d[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b0, d[cb], 0, 0, 0);
                        d[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b1, d[cb], 0, 0, 0);
                    }
                    int cell[4];
                    uint32_t seen[4][CB];
                    uint32_t open = 0;          // bit 4 cb + e: the sum still has to reach its cell
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int rel = drow[e] - w0;
                        const bool valid = 16 * blk + 4 * kq + e < M;
                        const bool inside = (uint32_t)rel < (uint32_t)ROWS;
                        cell[e] = (inside ? rel : 0) * STRIDE + 16 * c0 + r16;
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb) {
                            seen[e][cb] = 0;
                            if (valid && inside) {
                                open |= 1u << (4 * cb + e);
                                seen[e][cb] = cells[cell[e] + 16 * cb];
                            } else if (valid) {
                                unsafeAtomicAdd(out_h + (int64_t)drow[e] * C + 16 * (c0 + cb) + r16, d[cb][e]);
                            }
                        }
                    }
                    while (__any(open != 0 ? 1 : 0) != 0) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
#pragma unroll
                            for (int cb = 0; cb < CB; ++cb) {
                                if ((open >> (4 * cb + e) & 1u) != 0) {
                                    const uint32_t expect = seen[e][cb];
                                    const uint32_t sum = __float_as_uint(__uint_as_float(expect) + d[cb][e]);
                                    seen[e][cb] = atomicCAS(cells + cell[e] + 16 * cb, expect, sum);
                                    if (seen[e][cb] == expect) open &= ~(1u << (4 * cb + e));
                                }
                            }
                        }
                    }
                }
            }
        }
        __syncthreads();
        // the window's sums leave for memory, and the window is clear for the next head
        for (int cell = tid; cell < ROWS * C; cell += kWindowWaves * kWave) {
            const int r = cell / C, c = cell - r * C;
            const float v = window[r * STRIDE + c];
            if (v != 0.f) {
                window[r * STRIDE + c] = 0.f;
                unsafeAtomicAdd(out_h + (int64_t)(w0 + r) * C + c, v);
            }
        }
        __syncthreads();
    }
}

template <typename T, int C>
int launch_c(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32, uint8_t* handled,
             const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if) {
    constexpr int ROWS = kWindowCells / C;
    constexpr int G = window_group_tiles(C);
    constexpr int LDS = ROWS * (C + 1) * (int)sizeof(float);
    const int tiles = (s.N + kTileTokens - 1) / kTileTokens;
    const int groups = (tiles + G - 1) / G;
    const int64_t total = (int64_t)s.B * groups;
    if (total >= ((int64_t)1 << 30)) return CLUSTEN_ERR_BAD_DIMS;
    // more LDS than a workgroup gets without asking (a CU of this device holds 160 KB)
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(scatter_rows_window_kernel<T, C>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess) {
        (void)hipGetLastError();
        return CLUSTEN_ERR_LAUNCH;
    }
    hipLaunchKernelGGL((scatter_rows_window_kernel<T, C>), dim3(xcd_grid((int)total)), dim3(kWindowWaves * kWave), LDS,
                       stream, static_cast<const T*>(p), static_cast<const T*>(x), idx, acc32, handled, s.H, s.N, s.M, xs,
                       tiles, groups, (int)total, only_if);
    return launch_status();
}

template <typename T>
int launch_typed(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32, uint8_t* handled,
                 const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if) {
    switch (s.C) {
        case 16: return launch_c<T, 16>(p, x, xs, idx, acc32, handled, s, stream, only_if);
        case 32: return launch_c<T, 32>(p, x, xs, idx, acc32, handled, s, stream, only_if);
        case 64: return launch_c<T, 64>(p, x, xs, idx, acc32, handled, s, stream, only_if);
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
}

}  // namespace

bool scatter_rows_window_supported(const clusten_attn_shape& s, int dtype) {
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return false;
    return (s.C == 16 || s.C == 32 || s.C == 64) && s.M > 0 && s.M <= 64 && s.N > 0 &&
           (int64_t)s.N * s.C < ((int64_t)1 << 31);
}

size_t scatter_rows_window_handled_bytes(const clusten_attn_shape& s) {
    const size_t tiles = (size_t)s.B * ((s.N + kTileTokens - 1) / kTileTokens);
    return (tiles + 255) / 256 * 256;
}

int launch_scatter_rows_window(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32,
                               uint8_t* handled, const clusten_attn_shape& s, int dtype, hipStream_t stream,
                               const int32_t* only_if) {
    if (!scatter_rows_window_supported(s, dtype)) return CLUSTEN_ERR_BAD_DIMS;
    switch (dtype) {
        case CLUSTEN_F32: return launch_typed<float>(p, x, xs, idx, acc32, handled, s, stream, only_if);
        case CLUSTEN_F16: return launch_typed<f16_t>(p, x, xs, idx, acc32, handled, s, stream, only_if);
        case CLUSTEN_BF16: return launch_typed<bf16_t>(p, x, xs, idx, acc32, handled, s, stream, only_if);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
