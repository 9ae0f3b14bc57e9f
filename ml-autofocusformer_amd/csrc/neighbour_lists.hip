// neighbour_lists: the index tensors of a stage's local attention, from the nearest clusters of every token.
//
// After the balanced clustering the tokens of an image stand in cluster order (cluster g owns rows g*m .. g*m+m-1,
// the last cluster may be short), and every token attends to the members of its nnc nearest clusters, nearest
// first (models/aff_transformer.py:476-487):
//
//   row(i, j)          = m * nearest[b, i, j / m] + j % m                                   j < nnc * m
//   member_idx[b,i,j]  = row(i, j) if row(i, j) < N else 0          mask[b,i,j] = row(i, j) < N
//   pe_idx[b,i,j]      = trunc( (y' - (y - R)) * W + (x' - (x - R)) )   with (x, y) = pos[b,i], (x', y') = pos[b, member]
//   cluster_idx[b,i,r] = nearest[b,i,r] as int32
//
// which the reference spells as a gather, a comparison and some ten elementwise tensor operations.  The float
// operations are those of the tensor expressions in their order (no fused multiply-add), so pe_idx is identical also
// for positions that are not whole numbers.  It has no counterpart in the reference's extension modules.
#include "launch.hpp"

#pragma clang fp contract(off)

namespace clusten {
namespace {

__global__ __launch_bounds__(256) void neighbour_lists_kernel(const float2* __restrict__ pos,
                                                              const int64_t* __restrict__ nearest,
                                                              int64_t* __restrict__ member_idx, int64_t* __restrict__ mask,
                                                              int64_t* __restrict__ pe_idx, int32_t* __restrict__ cluster_idx,
                                                              int N, int nnc, int m, float radius, float table_width,
                                                              int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;   // (b, i, j)
    if (e >= total) return;
    const int M = nnc * m;
    const int64_t tok = e / M;              // b * N + i
    const int j = (int)(e - tok * M);
    const int r = j / m;
    const int64_t b = tok / N;
    const int64_t c = nearest[tok * nnc + r];
    const int64_t row = c * m + (j - r * m);
    const bool valid = row < N;
    const int64_t member = valid ? row : 0;
    member_idx[e] = member;
    if (mask) mask[e] = valid ? 1 : 0;
    if (cluster_idx && j == r * m) cluster_idx[tok * nnc + r] = (int32_t)c;
    const float2 p = pos[tok];
    const float2 q = pos[b * N + member];
    const float rx = q.x - (p.x - radius), ry = q.y - (p.y - radius);
    pe_idx[e] = (int64_t)(ry * table_width + rx);
}

}  // namespace

int launch_neighbour_lists(const float* pos, const int64_t* nearest, int64_t* member_idx, int64_t* mask, int64_t* pe_idx,
                           int32_t* cluster_idx, int B, int N, int nnc, int m, int radius, int table_width,
                           hipStream_t stream) {
    const int64_t total = (int64_t)B * N * nnc * m;
    hipLaunchKernelGGL(neighbour_lists_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const float2*>(pos), nearest, member_idx, mask, pe_idx, cluster_idx, N, nnc, m,
                       (float)radius, (float)table_width, total);
    return launch_status();
}

}  // namespace clusten
