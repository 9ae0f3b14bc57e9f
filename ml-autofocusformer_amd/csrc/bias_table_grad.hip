// bias_table_grad: the gradient of the relative-position bias table of an attention layer.
//
//   d_table[pe_idx[b,i,j], h] = sum over (b,i,j) of d_logit[b,h,i,j]
//
// the backward of `pe_table.gather(index=pe_idx...)` added to the attention logits (models/aff_transformer.py:131-133).
// The framework runs it as a scatter-add of B*H*N*M values into a table of some 12 000 rows: one global atomic per
// value, all of them on the same few hundred kilobytes.  Here a workgroup takes one head and a slice of the tokens
// and sums into a copy of that head's column of the table in LDS (LDS atomics; at most 16 000 rows); what it has
// collected goes to memory with one global atomic per touched row.  d_table is fp32 and zeroed by the caller.  It has
// no counterpart in the reference's extension modules.
#include "launch.hpp"

namespace clusten {
namespace {

constexpr int kGradThreads = 256;
constexpr int kGradRowsMax = 16000;   // 64 000 bytes of LDS

template <typename T>
__global__ __launch_bounds__(kGradThreads) void bias_table_grad_kernel(const T* __restrict__ d_logit,
                                                                       const int64_t* __restrict__ pe_idx,
                                                                       float* __restrict__ d_table, int H, int rows,
                                                                       int64_t per_image, int64_t per_slice, int B) {
    __shared__ float col[kGradRowsMax];
    const int h = blockIdx.y;
    for (int r = threadIdx.x; r < rows; r += kGradThreads) col[r] = 0.f;
    __syncthreads();
    // slice blockIdx.x of every image: elements [lo, hi) of its N*M (token, neighbour) pairs
    const int64_t lo = (int64_t)blockIdx.x * per_slice, hi = min(per_image, lo + per_slice);
    for (int b = 0; b < B; ++b) {
        const int64_t* idx_b = pe_idx + (int64_t)b * per_image;
        const T* g_bh = d_logit + ((int64_t)b * H + h) * per_image;
        for (int64_t e0 = lo + threadIdx.x; e0 < hi; e0 += 4 * kGradThreads) {
            int64_t r[4];
            float g[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {   // four independent loads before the first addition
                const int64_t e = e0 + k * kGradThreads;
                r[k] = e < hi ? idx_b[e] : -1;
                g[k] = e < hi ? to_acc(g_bh[e]) : 0.f;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if ((uint64_t)r[k] < (uint64_t)rows) atomicAdd(&col[r[k]], g[k]);
            }
        }
    }
    __syncthreads();
    for (int r = threadIdx.x; r < rows; r += kGradThreads) {
        const float v = col[r];
        if (v != 0.f) unsafeAtomicAdd(d_table + (int64_t)r * H + h, v);
    }
}

}  // namespace

int launch_bias_table_grad(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int N, int M, int rows,
                           int dtype, hipStream_t stream) {
    if (rows > kGradRowsMax) return CLUSTEN_ERR_BAD_DIMS;
    const int64_t per_image = (int64_t)N * M;
    // a workgroup per head and some 16 000 values: clearing its column of the table (rows words) and flushing the rows
    // it touched stay small next to that, and the device gets thousands of workgroups to overlap their latencies
    const int64_t want = (per_image * B + 16383) / 16384;
    const int slices = (int)max((int64_t)1, min(want, min(per_image, (int64_t)8192)));
    const int64_t per_slice = (per_image + slices - 1) / slices;
    const dim3 grid((unsigned)slices, (unsigned)H);
    switch (dtype) {
        case CLUSTEN_F32:
            hipLaunchKernelGGL(bias_table_grad_kernel<float>, grid, dim3(kGradThreads), 0, stream,
                               static_cast<const float*>(d_logit), pe_idx, d_table, H, rows, per_image, per_slice, B);
            break;
        case CLUSTEN_F16:
            hipLaunchKernelGGL(bias_table_grad_kernel<f16_t>, grid, dim3(kGradThreads), 0, stream,
                               static_cast<const f16_t*>(d_logit), pe_idx, d_table, H, rows, per_image, per_slice, B);
            break;
        case CLUSTEN_BF16:
            hipLaunchKernelGGL(bias_table_grad_kernel<bf16_t>, grid, dim3(kGradThreads), 0, stream,
                               static_cast<const bf16_t*>(d_logit), pe_idx, d_table, H, rows, per_image, per_slice, B);
            break;
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace clusten
