// Measurement kernels of libclusten_probe.so: a plain streaming copy and the stream / gather probe.  None of them
// is part of the operators' library; a benchmark loads this library to calibrate byte counters and to price the two
// kinds of memory traffic of a gather operator.
#include "../launch.hpp"
#include "../../../include/clusten_probe.h"

namespace clusten {

namespace {

constexpr int kBlock = 256;

// One 16-byte piece per thread, one short-lived workgroup per 4 KiB: on this device that streams
// 15-20 % faster than a grid-stride loop over the same bytes.
__global__ __launch_bounds__(kBlock) void copy_kernel(const Piece* __restrict__ src, Piece* __restrict__ dst,
                                                     size_t pieces) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < pieces) dst[i] = src[i];
}

// The memory instruction stream of a gather operator, reduced to its two components (see launch_stream_gather_probe):
// a wave per tile reads 5 KiB of its own (STREAM), gathers `gathers` times four random 256-byte rows of its window
// (GATHER, 12 accesses in flight) and writes 3 KiB of its own with the non-temporal hint (STREAM).
template <bool STREAM, bool GATHER>
__global__ __launch_bounds__(kWave) void stream_gather_kernel(const char* __restrict__ in, char* __restrict__ out,
                                                              const char* __restrict__ rows, int total_tiles,
                                                              int gathers, uint32_t window_rows, int tiles_per_window) {
    constexpr int U = 12;
    const int tile = xcd_tile(blockIdx.x, total_tiles);
    if (tile < 0) return;
    const uint32_t lane = threadIdx.x, sub = lane >> 4, pos = lane & 15;
    const char* window = rows + (size_t)(tile / tiles_per_window) * window_rows * 256;
    uint32_t h = (uint32_t)tile * 2654435761u + sub * 40503u;
    Piece a = Piece{0, 0, 0, 0};
    if constexpr (STREAM) {
        Piece v[5];
#pragma unroll
        for (int u = 0; u < 5; ++u) v[u] = *reinterpret_cast<const Piece*>(in + (size_t)tile * 5120 + u * 1024 + lane * 16);
#pragma unroll
        for (int u = 0; u < 5; ++u) a ^= v[u];
        h ^= a[0] & 1u;   // the gathers wait for the streamed data, as an operator's wait for its lists
    }
    if constexpr (GATHER) {
        for (int g = 0; g < gathers; g += U) {
            Piece v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                h = h * 1664525u + 1013904223u;
                v[u] = *reinterpret_cast<const Piece*>(window + (size_t)((h >> 8) % window_rows) * 256 + pos * 16);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) a ^= v[u];
        }
    }
    if constexpr (STREAM) {
#pragma unroll
        for (int u = 0; u < 3; ++u) {
            store_streaming(reinterpret_cast<Piece*>(out + (size_t)tile * 3072 + u * 1024 + lane * 16), a);
        }
    } else {
        if (a[0] == 0x12345678u && a[1] == 0x9abcdef0u) reinterpret_cast<Piece*>(out)[lane] = a;   // keeps the loads
    }
}

}  // namespace

static int launch_copy(const void* src, void* dst, size_t bytes, hipStream_t stream) {
    const size_t pieces = bytes / sizeof(Piece);
    const size_t blocks = (pieces + kBlock - 1) / kBlock;
    if (blocks >= ((size_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, static_cast<const Piece*>(src),
                       static_cast<Piece*>(dst), pieces);
    return launch_status();
}

static int launch_stream_gather_probe(const void* in, void* out, const void* rows, int tiles, int gathers, int window_rows,
                               int tiles_per_window, int mode, hipStream_t stream) {
    const char* i = static_cast<const char*>(in);
    char* o = static_cast<char*>(out);
    const char* r = static_cast<const char*>(rows);
    const dim3 grid(xcd_grid(tiles)), block(kWave);
    switch (mode) {
        case 1:
            hipLaunchKernelGGL((stream_gather_kernel<true, false>), grid, block, 0, stream, i, o, r, tiles, gathers,
                               (uint32_t)window_rows, tiles_per_window);
            break;
        case 2:
            hipLaunchKernelGGL((stream_gather_kernel<false, true>), grid, block, 0, stream, i, o, r, tiles, gathers,
                               (uint32_t)window_rows, tiles_per_window);
            break;
        case 3:
            hipLaunchKernelGGL((stream_gather_kernel<true, true>), grid, block, 0, stream, i, o, r, tiles, gathers,
                               (uint32_t)window_rows, tiles_per_window);
            break;
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
    return launch_status();
}

}  // namespace clusten

extern "C" {

int clusten_probe_abi_version(void) { return CLUSTEN_PROBE_ABI_VERSION; }

int clusten_copy_probe(const void* src, void* dst, size_t bytes, clusten_stream stream) {
    using namespace clusten;
    if (!src || !dst) return CLUSTEN_ERR_NULL_POINTER;
    if (bytes == 0 || bytes % 16 != 0) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(src) || !aligned16(dst)) return CLUSTEN_ERR_UNALIGNED;
    return launch_copy(src, dst, bytes, static_cast<hipStream_t>(stream));
}

int clusten_stream_gather_probe(const void* in, void* out, const void* rows, int tiles, int gathers, int window_rows,
                                int tiles_per_window, int mode, clusten_stream stream) {
    using namespace clusten;
    if (!in || !out || !rows) return CLUSTEN_ERR_NULL_POINTER;
    if (tiles <= 0 || gathers <= 0 || gathers % 12 != 0 || window_rows <= 0 || tiles_per_window <= 0 || mode < 1 || mode > 3) {
        return CLUSTEN_ERR_BAD_DIMS;
    }
    if (!aligned16(in) || !aligned16(out) || !aligned16(rows)) return CLUSTEN_ERR_UNALIGNED;
    return launch_stream_gather_probe(in, out, rows, tiles, gathers, window_rows, tiles_per_window, mode,
                                      static_cast<hipStream_t>(stream));
}

}  // extern "C"
