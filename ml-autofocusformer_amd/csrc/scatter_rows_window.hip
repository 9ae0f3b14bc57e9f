// scatter_rows_window: the atomic scatter of scatter_rows (scatter_rows_impl.hpp) for tiles whose 8 tokens share one
// list, with the sums of many neighbouring tiles collected in LDS before they reach memory.
//
//   out[b,h,idx[b,i,j],c] += p[b,h,i,j] * x[b,h,i,c]      (clusten/src/clustenqk_cuda_kernel.cu:91-132,
//                                                          clusten/src/clustenav_cuda_kernel.cu:93-127)
//
// Neighbour lists name rows near their own token, so consecutive tiles add to the same few hundred rows.  A workgroup
// of 16 waves takes 64 consecutive tiles of one image (512 tokens) and 16 of the head's channels, and keeps an fp32
// window of the 1024 destination rows around those tokens, [first token - 256, first token + 768), in LDS (64 KB of
// cells; two workgroups share a CU).  Per head: every wave forms, for each of its four tiles, D[slot][c] = sum_t
// p[t][slot] * x[t][c] on the matrix cores (operands straight from memory in the instruction's layout) and adds D
// into the window; a row outside the window is added to memory directly.  After a barrier the non-zero cells of the
// window leave as one memory atomic each and are cleared for the next head.  A row is inside the windows of two
// groups of tiles, so it receives two memory atomics per channel instead of one per tile that names it (six at 48
// neighbours).
//
// The additions to the window are compare-and-swap loops on the cells' bits, not `ds_add_f32`: this device adds
// floats in LDS one lane at a time (measured: 193 clocks per 64-lane instruction, whatever the addresses; an integer
// add takes 5, a read and a write 6-10), which made the first form of this kernel 2.7 times slower than the atomics
// to memory it replaces.  The four cells of a lane are read, then swapped; a lane goes round again only when another
// wave, or another lane naming the same row, changed its cell in between.
//
// Which tiles have one list is found here and written to `handled` (one byte per tile); the tile kernel that follows
// skips those tiles and takes the rest, so the two kernels together add every product exactly once.
//
// Measured at B128 H2 N3136 C32 M48 fp32 on lists shared by each cluster of 8 tokens (+-256-token window): 255 us
// against the 471 us of one memory atomic per (tile, slot, channel).  With all 32 channels of a head in one
// workgroup (a 128 KB window, one workgroup per CU, the next tile's operands requested ahead) it took 311 us: the
// phases of a workgroup - finding the shared lists, operand loads, products, additions, the window's way to memory -
// do not overlap, and a second workgroup on the CU fills the gaps although it reads p and the lists a second time.
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kWindowWaves = 16;
constexpr int kWindowRows = 1024;                              // destination rows of the window
constexpr int kWindowTiles = 64;                               // tiles of a workgroup: half the window
constexpr int kWindowTilesPerWave = kWindowTiles / kWindowWaves;
constexpr int kWindowStride = 17;   // floats per row: odd, the rows of one access fall into different banks
constexpr int kWindowLds = kWindowRows * kWindowStride * (int)sizeof(float);

// 8 waves per SIMD: two workgroups of 16 waves on a CU
template <typename T>
__global__ __launch_bounds__(kWindowWaves* kWave) __attribute__((amdgpu_waves_per_eu(8, 8))) void scatter_rows_window_kernel(
    const T* __restrict__ p, const T* __restrict__ x, const int64_t* __restrict__ idx, float* __restrict__ out,
    uint8_t* __restrict__ handled, int H, int N, int M, int C, clusten_strides xs, int tiles_per_image,
    int groups_per_image, int total_units, const int32_t* __restrict__ only_if) {
    constexpr int ROWS = kWindowRows, G = kWindowTiles, TPW = kWindowTilesPerWave, STRIDE = kWindowStride;
    extern __shared__ float window[];            // ROWS * STRIDE

    if (only_if != nullptr && *only_if == 0) return;   // the cluster-by-cluster kernel has these lists
    const int unit = xcd_tile(blockIdx.x, total_units);
    if (unit < 0) return;
    // unit -> (image, group of tiles, block of 16 channels); the blocks of a group are neighbours in the grid, so they
    // run at the same time on one XCD and the second reads p and the lists from its L2
    const int cbn = C >> 4;
    const int cb = unit % cbn;
    const int bg = unit / cbn;
    const int b = bg / groups_per_image;
    const int g = bg - b * groups_per_image;
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
            if (lane == 0 && cb == 0) handled[(int64_t)b * tiles_per_image + tile] = shared_list ? 1 : 0;
        }
    }
    for (int z = tid; z < ROWS * STRIDE; z += kWindowWaves * kWave) window[z] = 0.f;
    // nothing to add: the tile kernel has every tile of the group
    if (__syncthreads_or(ok != 0 ? 1 : 0) == 0) return;

    const int blocks = (M + 15) >> 4;
    uint32_t* cells = reinterpret_cast<uint32_t*>(window);
    for (int h = 0; h < H; ++h) {
        float* out_h = out + ((int64_t)b * H + h) * N * C + 16 * cb;
#pragma unroll 1
        for (int k = 0; k < TPW; ++k) {
            if ((ok >> k & 1u) == 0) continue;
            const int i0 = (g * G + wave + kWindowWaves * k) * kTileTokens;
            const int nt = min(kTileTokens, N - i0);
            const T* ph = p + (((int64_t)b * H + h) * N + i0) * M;
            const T* xh = x + (int64_t)b * xs.b + (int64_t)h * xs.h + (int64_t)i0 * xs.n + 16 * cb;
            // B operands: x[token 4 s + kq][channel 16 cb + r16]
            const float x0 = to_acc(xh[(uint32_t)(min(kq, nt - 1) * (int)xs.n + r16)]);
            const float x1 = to_acc(xh[(uint32_t)(min(4 + kq, nt - 1) * (int)xs.n + r16)]);
            const float xb0 = kq < nt ? x0 : 0.f, xb1 = 4 + kq < nt ? x1 : 0.f;
            int rows_k = rows[0];
#pragma unroll
            for (int kk = 1; kk < TPW; ++kk) rows_k = k == kk ? rows[kk] : rows_k;
#pragma unroll 1
            for (int blk = 0; blk < blocks; ++blk) {
                // A operands: p[token 4 s + kq][slot 16 blk + r16]
                const int slot_a = min(16 * blk + r16, M - 1);
                const bool slot_ok = 16 * blk + r16 < M;
                const float p0 = to_acc(ph[(uint32_t)(min(kq, nt - 1) * M + slot_a)]);
                const float p1 = to_acc(ph[(uint32_t)(min(4 + kq, nt - 1) * M + slot_a)]);
                const float a0 = (slot_ok && kq < nt) ? p0 : 0.f;
                const float a1 = (slot_ok && 4 + kq < nt) ? p1 : 0.f;
                // the lane's results: slots 16 blk + 4 kq .. + 3 of channel 16 cb + r16
                int drow[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) drow[e] = __shfl(rows_k, min(16 * blk + 4 * kq + e, M - 1));
                F32x4 d = F32x4{0.f, 0.f, 0.f, 0.f};
                d = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, xb0, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, xb1, d, 0, 0, 0);
                // the sums are added by compare-and-swap on the cells' bits: the lane's four cells are read, then
                // swapped, and only the lanes that lost a race go round again
                int cell[4];
                uint32_t seen[4];
                uint32_t open = 0;          // bit e: the sum still has to reach its cell
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int rel = drow[e] - w0;
                    const bool valid = 16 * blk + 4 * kq + e < M;
                    const bool inside = (uint32_t)rel < (uint32_t)ROWS;
                    cell[e] = (inside ? rel : 0) * STRIDE + r16;
                    seen[e] = 0;
                    if (valid && inside) {
                        open |= 1u << e;
                        seen[e] = cells[cell[e]];
                    } else if (valid) {
                        unsafeAtomicAdd(out_h + (int64_t)drow[e] * C + r16, d[e]);
                    }
                }
                while (__any(open != 0 ? 1 : 0) != 0) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if ((open >> e & 1u) != 0) {
                            const uint32_t expect = seen[e];
                            const uint32_t sum = __float_as_uint(__uint_as_float(expect) + d[e]);
                            seen[e] = atomicCAS(cells + cell[e], expect, sum);
                            if (seen[e] == expect) open &= ~(1u << e);
                        }
                    }
                }
            }
        }
        __syncthreads();
        // the window's sums leave for memory, and the window is clear for the next head
        for (int cell = tid; cell < ROWS * 16; cell += kWindowWaves * kWave) {
            const int r = cell >> 4, c = cell & 15;
            const float v = window[r * STRIDE + c];
            if (v != 0.f) {
                window[r * STRIDE + c] = 0.f;
                unsafeAtomicAdd(out_h + (int64_t)(w0 + r) * C + c, v);
            }
        }
        __syncthreads();
    }
}

template <typename T>
int launch_typed(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32, uint8_t* handled,
                 const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if) {
    const int tiles = (s.N + kTileTokens - 1) / kTileTokens;
    const int groups = (tiles + kWindowTiles - 1) / kWindowTiles;
    const int64_t total = (int64_t)s.B * groups * (s.C / 16);
    if (total >= ((int64_t)1 << 30)) return CLUSTEN_ERR_BAD_DIMS;
    // more LDS than a workgroup gets without asking (a CU of this device holds 160 KB)
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(scatter_rows_window_kernel<T>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kWindowLds) != hipSuccess) {
        (void)hipGetLastError();
        return CLUSTEN_ERR_LAUNCH;
    }
    hipLaunchKernelGGL((scatter_rows_window_kernel<T>), dim3(xcd_grid((int)total)), dim3(kWindowWaves * kWave), kWindowLds,
                       stream, static_cast<const T*>(p), static_cast<const T*>(x), idx, acc32, handled, s.H, s.N, s.M, s.C,
                       xs, tiles, groups, (int)total, only_if);
    return launch_status();
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
