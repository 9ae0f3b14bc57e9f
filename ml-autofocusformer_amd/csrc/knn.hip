// knn2d: for every query point the k nearest database points of the same batch element, nearest first.
//
// The model asks for the 6 nearest cluster centres of every token and for the distance of every token to
// its nearest other token (models/aff_transformer.py:298,476 through knn_keops, models/point_utils.py:27-58,
// which hands the search to an external library).  Positions are 2-D and a batch element holds at most a few
// thousand points, so the search is a scan: a workgroup stages the database of its batch element through LDS,
// a thread owns one query and keeps its k best (squared distance, index) pairs sorted in registers.
// Squared distances are formed as dx*dx + dy*dy from the differences (no contraction with a product of
// norms), so integer positions give exact values; equal distances keep the lower index first because the scan
// ascends and replaces only on strictly smaller.  The distance returned is the square root.
#include "launch.hpp"

// every product and sum below is rounded on its own, as the tensor expressions it mirrors round them: no fused
// multiply-add (the compiler's default would contract a * b + c)
#pragma clang fp contract(off)

namespace clusten {
namespace {

constexpr int kKnnBlock = 256;
constexpr int kKnnChunk = 1024;  // database points per LDS stage

template <int K>
__global__ __launch_bounds__(kKnnBlock) void knn2d_kernel(const float* __restrict__ query,
                                                           const float* __restrict__ database,
                                                           int64_t* __restrict__ idx_out, float* __restrict__ dist_out,
                                                           int Nq, int N, int blocks_per_batch) {
    __shared__ float2 pts[kKnnChunk];
    const int b = blockIdx.x / blocks_per_batch;
    const int q = (blockIdx.x - b * blocks_per_batch) * kKnnBlock + threadIdx.x;
    const bool live = q < Nq;
    const float2 me = live ? reinterpret_cast<const float2*>(query)[(int64_t)b * Nq + q] : make_float2(0.f, 0.f);
    const float2* db = reinterpret_cast<const float2*>(database) + (int64_t)b * N;

    float best_d[K];
    int best_i[K];
#pragma unroll
    for (int s = 0; s < K; ++s) {
        best_d[s] = INFINITY;
        best_i[s] = 0;
    }
    for (int base = 0; base < N; base += kKnnChunk) {
        const int cnt = min(kKnnChunk, N - base);
        __syncthreads();
        for (int t = threadIdx.x; t < cnt; t += kKnnBlock) pts[t] = db[base + t];
        __syncthreads();
        for (int t = 0; t < cnt; ++t) {
            const float dx = me.x - pts[t].x, dy = me.y - pts[t].y;
            const float d = __fadd_rn(__fmul_rn(dx, dx), __fmul_rn(dy, dy));
            if (d < best_d[K - 1]) {
                // insert, keeping the list ascending; entries equal to d stay in front (they came first)
                float cd = d;
                int ci = base + t;
                bool shifting = false;  // once the candidate is placed, every later entry moves down one place
#pragma unroll
                for (int s = 0; s < K; ++s) {
                    const bool take = shifting || cd < best_d[s];
                    shifting = take;
                    const float td = best_d[s];
                    const int ti = best_i[s];
                    best_d[s] = take ? cd : td;
                    best_i[s] = take ? ci : ti;
                    cd = take ? td : cd;
                    ci = take ? ti : ci;
                }
            }
        }
    }
    if (live) {
        const int64_t o = ((int64_t)b * Nq + q) * K;
#pragma unroll
        for (int s = 0; s < K; ++s) {
            idx_out[o + s] = best_i[s];
            // correctly rounded, as the tensor formulation: the fp64 root rounded once more (53 >= 2 * 24 + 2 bits)
            if (dist_out) dist_out[o + s] = (float)sqrt((double)best_d[s]);
        }
    }
}

template <int K>
int launch_k(const float* query, const float* database, int64_t* idx, float* dist, int B, int Nq, int N,
             hipStream_t stream) {
    const int blocks_per_batch = (Nq + kKnnBlock - 1) / kKnnBlock;
    hipLaunchKernelGGL((knn2d_kernel<K>), dim3((unsigned)(B * blocks_per_batch)), dim3(kKnnBlock), 0, stream, query,
                       database, idx, dist, Nq, N, blocks_per_batch);
    return launch_status();
}

}  // namespace

int launch_knn2d(const float* query, const float* database, int64_t* idx, float* dist, int B, int Nq, int N, int K,
                 hipStream_t stream) {
    switch (K) {
        case 1: return launch_k<1>(query, database, idx, dist, B, Nq, N, stream);
        case 2: return launch_k<2>(query, database, idx, dist, B, Nq, N, stream);
        case 3: return launch_k<3>(query, database, idx, dist, B, Nq, N, stream);
        case 4: return launch_k<4>(query, database, idx, dist, B, Nq, N, stream);
        case 5: return launch_k<5>(query, database, idx, dist, B, Nq, N, stream);
        case 6: return launch_k<6>(query, database, idx, dist, B, Nq, N, stream);
        case 7: return launch_k<7>(query, database, idx, dist, B, Nq, N, stream);
        case 8: return launch_k<8>(query, database, idx, dist, B, Nq, N, stream);
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
}

}  // namespace clusten
