// scanline_rank: the order in which the balanced clustering of the reference model lines up the tokens of every
// image (models/point_utils.py:61-208, `space_filling_cluster`, default scan-line path with anchors): tokens are
// binned into the cells of an anchor grid walked row by row in alternating direction, and inside a cell ordered
// by the ratio of their squared distances to the previous and to the next anchor on that walk
// (point_utils.py:139-159):
//
//   cell    = floor(pos / cell_size)                     rank = position of the cell on the walk
//   ratio   = |pos - anchor(rank-1)|^2 / (|pos - anchor(rank+1)|^2 + 1e-5)
//   key     = rank * (max over the whole batch of ratio + 1) + ratio
//   ranking = stable argsort of key per image
//
// The reference spells this out as some twenty tensor operations and a sort; here two launches: one pass over the
// tokens for rank, ratio and the batch-wide maximum, and one workgroup per image that sorts (key, index) pairs in
// LDS (bitonic, at most 4096 tokens).  Every float operation is the single correctly rounded operation the tensor
// expressions perform, in their order (no fused multiply-add), so the keys are bit-identical and the ranking equal.
// It has no counterpart in the reference's extension modules.
#include "launch.hpp"

// Every product, sum and quotient below is rounded on its own, as the tensor expressions it mirrors round them:
// no fused multiply-add (the compiler's default would contract a * b + c; the rounding intrinsics of the headers
// do not help, their operations are contracted after inlining).  fp32 division is the correctly rounded sequence.
#pragma clang fp contract(off)

namespace clusten {
namespace {

constexpr int kRankBlock = 256;
// threads of the sorting workgroup: 1024 for long sequences (every step of the network touches P/2 pairs)
inline int kRankThreads(int P) { return P > 4096 ? 1024 : kRankBlock; }

struct Anchors {
    int rows, cols;
    float cell_w, cell_h;

    // centre (x, y) of the anchor at position r of the walk; positions before the first and after the last anchor
    // continue the line through the two nearest ones
    __device__ float2 centre(int r) const {
        const int ys = r / cols, xr = r - ys * cols;
        const int xs = (ys & 1) ? cols - 1 - xr : xr;
        return make_float2(((float)xs * cell_w + cell_w * 0.5f) - 0.5f, ((float)ys * cell_h + cell_h * 0.5f) - 0.5f);
    }
    __device__ float2 previous(int r) const {
        if (r > 0) return centre(r - 1);
        const float2 c0 = centre(0), c1 = centre(1);
        return make_float2(c0.x - (c1.x - c0.x), c0.y - (c1.y - c0.y));
    }
    __device__ float2 next(int r) const {
        const int last = rows * cols - 1;
        if (r < last) return centre(r + 1);
        const float2 c0 = centre(last), c1 = centre(last - 1);
        return make_float2(c0.x + (c0.x - c1.x), c0.y + (c0.y - c1.y));
    }
};

__device__ __forceinline__ float dist2(float2 p, float2 c) {
    const float dx = p.x - c.x, dy = p.y - c.y;
    return dx * dx + dy * dy;
}

// rank and ratio of every token; the largest ratio of the launch (ratios are >= 0: their bit patterns order like ints)
__global__ __launch_bounds__(kRankBlock) void rank_ratio_kernel(const float2* __restrict__ pos, int* __restrict__ rank_out,
                                                                float* __restrict__ ratio_out, int* __restrict__ max_bits,
                                                                int64_t tokens, Anchors a) {
    const int64_t e = (int64_t)blockIdx.x * kRankBlock + threadIdx.x;
    float ratio = 0.f;
    if (e < tokens) {
        const float2 p = pos[e];
        const int cells = a.rows * a.cols;
        const int cx = (int)floorf(p.x / a.cell_w), cy = (int)floorf(p.y / a.cell_h);
        const int cell = min(max(cx + cy * a.cols, 0), cells - 1);
        const int ys = cell / a.cols, xs = cell - ys * a.cols;
        const int rank = ys * a.cols + ((ys & 1) ? a.cols - 1 - xs : xs);
        ratio = dist2(p, a.previous(rank)) / (dist2(p, a.next(rank)) + 1e-5f);
        rank_out[e] = rank;
        ratio_out[e] = ratio;
    }
    float m = ratio;
#pragma unroll
    for (int s = 1; s < kWave; s <<= 1) m = fmaxf(m, __shfl_xor(m, s));
    if ((threadIdx.x & (kWave - 1)) == 0) atomicMax(max_bits, __float_as_int(m));
}

// one workgroup per image: (key bits, token index) pairs sorted in LDS; padding pairs sort last
__global__ __launch_bounds__(1024) void rank_sort_kernel(const int* __restrict__ rank, const float* __restrict__ ratio,
                                                               const int* __restrict__ max_bits,
                                                               int64_t* __restrict__ ranking, int N, int P) {
    extern __shared__ uint64_t pairs[];
    const int b = blockIdx.x;
    const float scale = __int_as_float(*max_bits) + 1.f;
    for (int i = threadIdx.x; i < P; i += blockDim.x) {
        uint64_t v = ~0ull;
        if (i < N) {
            const int64_t e = (int64_t)b * N + i;
            const float key = (float)rank[e] * scale + ratio[e];
            v = ((uint64_t)__float_as_uint(key) << 32) | (uint32_t)i;
        }
        pairs[i] = v;
    }
    __syncthreads();
    for (int k = 2; k <= P; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int t = threadIdx.x; t < P / 2; t += blockDim.x) {
                const int i = (t / j) * 2 * j + (t % j), l = i + j;
                const bool up = (i & k) == 0;
                const uint64_t x = pairs[i], y = pairs[l];
                if ((x > y) == up) {
                    pairs[i] = y;
                    pairs[l] = x;
                }
            }
            __syncthreads();
        }
    }
    for (int i = threadIdx.x; i < N; i += blockDim.x) ranking[(int64_t)b * N + i] = (int64_t)(pairs[i] & 0xffffffffu);
}

}  // namespace

size_t scanline_rank_workspace_bytes(int B, int N) { return (size_t)B * N * 8 + 16; }

int launch_scanline_rank(const float* pos, int64_t* ranking, void* workspace, int B, int N, int rows, int cols,
                         float cell_w, float cell_h, hipStream_t stream) {
    const int64_t tokens = (int64_t)B * N;
    int* max_bits = static_cast<int*>(workspace);
    int* rank = max_bits + 4;
    float* ratio = reinterpret_cast<float*>(rank + tokens);
    if (int st = launch_zero_f32(reinterpret_cast<float*>(max_bits), 4, stream)) return st;
    const Anchors a{rows, cols, cell_w, cell_h};
    hipLaunchKernelGGL(rank_ratio_kernel, dim3((unsigned)((tokens + kRankBlock - 1) / kRankBlock)), dim3(kRankBlock), 0,
                       stream, reinterpret_cast<const float2*>(pos), rank, ratio, max_bits, tokens, a);
    if (int st = launch_status()) return st;
    int P = 2;
    while (P < N) P <<= 1;
    const size_t lds = (size_t)P * 8;
    if (lds > 48 * 1024) {
        // more LDS than a workgroup gets without asking (a CU of this device holds 160 KB): 9216 tokens need 128 KB
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(rank_sort_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess) {
            (void)hipGetLastError();
            return CLUSTEN_ERR_BAD_DIMS;
        }
    }
    hipLaunchKernelGGL(rank_sort_kernel, dim3((unsigned)B), dim3(kRankThreads(P)), lds, stream, rank, ratio, max_bits,
                       ranking, N, P);
    return launch_status();
}

int scanline_rank_max_tokens() {
    int dev = 0, bytes = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) {
        (void)hipGetLastError();
        return 4096;
    }
    int P = 2;
    while ((size_t)P * 2 * 8 <= (size_t)bytes) P <<= 1;
    return P;
}

// ---- reordered positions and cluster centres --------------------------------------------------------------------

namespace {

// one thread per cluster: its members' positions in ranking order, and their mean
__global__ __launch_bounds__(256) void cluster_centres_kernel(const float2* __restrict__ pos,
                                                              const int64_t* __restrict__ ranking,
                                                              float2* __restrict__ pos_sorted, float2* __restrict__ centres,
                                                              int N, int m, int K, int64_t clusters) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= clusters) return;
    const int64_t b = e / K;
    const int g = (int)(e - b * K);
    const int first = g * m, count = min(m, N - first);
    float sx = 0.f, sy = 0.f;
    for (int t = 0; t < count; ++t) {
        const float2 p = pos[b * N + ranking[b * N + first + t]];
        if (pos_sorted != nullptr) pos_sorted[b * N + first + t] = p;
        sx += p.x;
        sy += p.y;
    }
    centres[e] = make_float2(sx / (float)count, sy / (float)count);
}

// out[b,i,:] = x[b, order[b,i], :], 16 bytes per lane
__global__ __launch_bounds__(256) void gather_rows_kernel(const Piece* __restrict__ x, const int64_t* __restrict__ order,
                                                          Piece* __restrict__ out, int N, int pieces_per_row,
                                                          int64_t order_batch_stride, int64_t total_pieces) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total_pieces) return;
    const int64_t row = e / pieces_per_row;
    const int piece = (int)(e - row * pieces_per_row);
    const int64_t b = row / N;
    const int i = (int)(row - b * N);
    const int64_t src = b * N + order[b * order_batch_stride + i];
    out[e] = x[src * pieces_per_row + piece];
}

}  // namespace

int launch_cluster_centres(const float* pos, const int64_t* ranking, float* pos_sorted, float* centres, int B, int N, int m,
                           hipStream_t stream) {
    const int K = (N + m - 1) / m;
    const int64_t clusters = (int64_t)B * K;
    hipLaunchKernelGGL(cluster_centres_kernel, dim3((unsigned)((clusters + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const float2*>(pos), ranking, reinterpret_cast<float2*>(pos_sorted),
                       reinterpret_cast<float2*>(centres), N, m, K, clusters);
    return launch_status();
}

int launch_gather_rows(const void* x, const int64_t* order, void* out, int64_t B, int N, int row_bytes, int order_shared,
                       hipStream_t stream) {
    const int ppr = row_bytes / 16;
    const int64_t total = B * N * ppr;
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const Piece*>(x), order, static_cast<Piece*>(out), N, ppr,
                       order_shared ? (int64_t)0 : (int64_t)N, total);
    return launch_status();
}

}  // namespace clusten
