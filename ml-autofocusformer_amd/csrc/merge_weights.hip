// merge_weights: the weights operand of the WF operator as the reference model builds it before a merge,
//
//   w[b,i,j,:] = table_w[pe_idx[b,i,j], :] * prob[b, nbhd_idx[b,i,j]] * mask[b,i,j]
//
// (models/aff_transformer.py:340-358: a row lookup in the position-embedding weights, a gather of the learned
// importance of each neighbour, two multiplications — each a pass over the (B,N',M,IC) tensor; prob and mask are
// optional).  Here one pass: a lane owns one (token, neighbour) pair, reads its three indices, looks up the row of
// IC = 4 weights (the table is a few hundred KB and stays in cache) and writes 16 bytes next to its neighbours'.
// It has no counterpart in the reference's extension modules.
#include "launch.hpp"

namespace clusten {
namespace {

__global__ __launch_bounds__(256) void merge_weights_kernel(const float* __restrict__ table_w,
                                                            const int64_t* __restrict__ pe_idx,
                                                            const int64_t* __restrict__ nbhd_idx,
                                                            const float* __restrict__ prob,
                                                            const int64_t* __restrict__ mask, float* __restrict__ out,
                                                            int64_t pairs, int64_t pairs_per_batch, int N) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= pairs) return;
    float4 w = *reinterpret_cast<const float4*>(table_w + pe_idx[e] * 4);
    float s = 1.f;
    if (prob) s = prob[(e / pairs_per_batch) * N + nbhd_idx[e]];
    if (mask) s *= (float)mask[e];
    w.x *= s, w.y *= s, w.z *= s, w.w *= s;
    *reinterpret_cast<float4*>(out + e * 4) = w;   // plain: the merge kernel reads it next
}

}  // namespace

int launch_merge_weights(const float* table_w, const int64_t* pe_idx, const int64_t* nbhd_idx, const float* prob,
                         const int64_t* mask, float* out, int B, int N, int Nout, int M, hipStream_t stream) {
    const int64_t per_batch = (int64_t)Nout * M;
    const int64_t pairs = per_batch * B;
    hipLaunchKernelGGL(merge_weights_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream, table_w, pe_idx,
                       nbhd_idx, prob, mask, out, pairs, per_batch, N);
    return launch_status();
}

}  // namespace clusten
