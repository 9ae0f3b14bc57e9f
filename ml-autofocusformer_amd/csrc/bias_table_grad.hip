// bias_table_grad: the gradient of the relative-position bias table of an attention layer.
//
//   d_table[pe_idx[b,i,j], h] = sum over (b,i,j) of d_logit[b,h,i,j]
//
// the backward of `pe_table.gather(index=pe_idx...)` added to the attention logits (models/aff_transformer.py:131-133).
// The framework runs it as a scatter-add of B*H*N*M values into a table of some 12 000 rows: one global atomic per
// value, all of them on the same few hundred kilobytes.  Here a workgroup takes one head and a contiguous slice of the
// head's values (images one after the other) and sums into a copy of that head's column of the table in LDS (LDS
// atomics; at most 16 000 rows); what it has collected goes to memory with one global atomic per touched row.
// The grid is about a thousand workgroups of 512 threads: the global atomics of the flush all land on the same few
// kilobytes, so a workgroup should flush once for a long slice, and a column of 12 000 rows is 48 KB of LDS, so few
// workgroups fit a compute unit and each has to bring many waves.  A thread reads four consecutive values at a time
// (two 16-byte loads of indices, one load of gradients) and keeps four such groups in flight.  What bounds the kernel
// is the rate of the fp32 LDS atomics, about one every three cycles per compute unit whatever the rows are (38.5 M
// values: 205 us in fp32 and fp16, over 3000 or 12 321 rows, uniform or clustered; the same loop with integer atomics
// takes 73 us on fp16 values).
// d_table is fp32 and zeroed by the caller.  It has no counterpart in the reference's extension modules.
#include "launch.hpp"

namespace clusten {
namespace {

constexpr int kGradThreads = 512;
constexpr int kGradRowsMax = 16000;   // 64 000 bytes of LDS
constexpr int kGradGroups = 4;        // groups of 4 values in flight per thread

// VEC = 4: per_image % 4 == 0 and both tensors 16-byte aligned (a group never straddles two images); VEC = 1 otherwise.
template <typename T, int VEC>
__global__ __launch_bounds__(kGradThreads) void bias_table_grad_kernel(const T* __restrict__ d_logit,
                                                                       const int64_t* __restrict__ pe_idx,
                                                                       float* __restrict__ d_table, int H, int rows,
                                                                       int64_t per_image, int64_t per_slice, int B) {
    typedef VecIO<T, VEC> GIO;
    typedef typename RawBytes<VEC == 4 ? 16 : 8>::type IdxRaw;   // two indices (VEC = 4: a group is two of them) or one
    constexpr int IR = VEC == 4 ? 2 : 1;
    extern __shared__ float col[];   // rows floats
    const int h = blockIdx.y;
    for (int r = threadIdx.x; r < rows; r += kGradThreads) col[r] = 0.f;
    __syncthreads();
    // slice blockIdx.x of the head's B * per_image / VEC groups of values: the thread keeps (image, group in the image)
    // of its next group and steps it, so that no division enters the loop
    const int64_t groups_per_image = per_image / VEC;
    const int64_t total = groups_per_image * B;
    const int64_t lo = (int64_t)blockIdx.x * per_slice, hi = min(total, lo + per_slice);
    int64_t f = lo + threadIdx.x;
    int64_t b = f / groups_per_image, e = f - b * groups_per_image;
    for (; f < hi; f += kGradGroups * kGradThreads) {
        IdxRaw r[kGradGroups][IR];
        typename GIO::raw g[kGradGroups];
        bool in[kGradGroups];
#pragma unroll
        for (int k = 0; k < kGradGroups; ++k) {   // independent loads before the first addition
            in[k] = f + k * kGradThreads < hi;
            if (in[k]) {
#pragma unroll
                for (int w = 0; w < IR; ++w) {
                    r[k][w] = *reinterpret_cast<const IdxRaw*>(pe_idx + (b * groups_per_image + e) * VEC + 2 * w);
                }
                g[k] = *reinterpret_cast<const typename GIO::raw*>(d_logit + ((b * H + h) * groups_per_image + e) * VEC);
            }
            e += kGradThreads;
            while (e >= groups_per_image) {   // (at most once unless an image holds fewer groups than there are threads)
                e -= groups_per_image;
                b = min(b + 1, (int64_t)B - 1);
            }
        }
#pragma unroll
        for (int k = 0; k < kGradGroups; ++k) {
            if (in[k]) {
                float x[VEC];
                GIO::unpack(g[k], x);
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    // the index as two 32-bit words: a row is below 2^31
                    const uint32_t lo32 = raw_word(r[k][v / 2], 2 * (v % 2)), hi32 = raw_word(r[k][v / 2], 2 * (v % 2) + 1);
                    if (hi32 == 0u && lo32 < (uint32_t)rows) atomicAdd(&col[lo32], x[v]);
                }
            }
        }
    }
    __syncthreads();
    for (int r = threadIdx.x; r < rows; r += kGradThreads) {
        const float v = col[r];
        if (v != 0.f) unsafeAtomicAdd(d_table + (int64_t)r * H + h, v);
    }
}

template <typename T>
void launch_typed(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int rows, int64_t per_image,
                  hipStream_t stream) {
    const bool wide = per_image % 4 == 0 && aligned16(d_logit) && aligned16(pe_idx);
    const int vec = wide ? 4 : 1;
    // about 1024 workgroups in all, and no slice shorter than 16 000 values
    const int64_t total = per_image / vec * B;
    const int64_t want = (total * vec + 16383) / 16384;
    const int64_t cap = max(1, 1024 / H);
    const int slices = (int)max((int64_t)1, min(want, cap));
    const int64_t per_slice = (total + slices - 1) / slices;
    const dim3 grid((unsigned)slices, (unsigned)H);
    const size_t lds = (size_t)rows * sizeof(float);
    if (wide) {
        hipLaunchKernelGGL((bias_table_grad_kernel<T, 4>), grid, dim3(kGradThreads), lds, stream,
                           static_cast<const T*>(d_logit), pe_idx, d_table, H, rows, per_image, per_slice, B);
    } else {
        hipLaunchKernelGGL((bias_table_grad_kernel<T, 1>), grid, dim3(kGradThreads), lds, stream,
                           static_cast<const T*>(d_logit), pe_idx, d_table, H, rows, per_image, per_slice, B);
    }
}

}  // namespace

int launch_bias_table_grad(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int N, int M, int rows,
                           int dtype, hipStream_t stream) {
    if (rows > kGradRowsMax) return CLUSTEN_ERR_BAD_DIMS;
    const int64_t per_image = (int64_t)N * M;
    switch (dtype) {
        case CLUSTEN_F32: launch_typed<float>(d_logit, pe_idx, d_table, B, H, rows, per_image, stream); break;
        case CLUSTEN_F16: launch_typed<f16_t>(d_logit, pe_idx, d_table, B, H, rows, per_image, stream); break;
        case CLUSTEN_BF16: launch_typed<bf16_t>(d_logit, pe_idx, d_table, B, H, rows, per_image, stream); break;
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace clusten
