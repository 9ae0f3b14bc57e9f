// bias_table_grad: the gradient of the relative-position bias table of an attention layer.
//
//   d_table[pe_idx[b,i,j], h] = sum over (b,i,j) of d_logit[b,h,i,j]
//
// the backward of `pe_table.gather(index=pe_idx...)` added to the attention logits (models/aff_transformer.py:131-133).
// The framework runs it as a scatter-add of B*H*N*M values into a table of some 12 000 rows: one global atomic per
// value, all of them on the same few hundred kilobytes.  Here a workgroup takes one head and a contiguous slice of the
// head's values (images one after the other) and sums into a copy of that head's column of the table in LDS (LDS
// atomics; at most 16 000 rows); what it has collected goes to memory with one global atomic per touched row.
// The grid is one round of workgroups of 512 threads (768 to 1024 of them): the global atomics of the flush all land
// on the same few kilobytes, so a workgroup should flush once for a long slice, and a column of 12 000 rows is 48 KB
// of LDS, so few workgroups fit a compute unit and each has to bring many waves.  A thread reads four consecutive values at a time
// (two 16-byte loads of indices, one load of gradients) and keeps four such groups in flight.
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
    uint32_t* cells = reinterpret_cast<uint32_t*>(col);
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
            // The values are added by compare-and-swap on the cells' bits (an fp32 LDS atomic add takes some 190 cycles
            // per wave instruction here, a compare-and-swap a few): the group's cells are read, then swapped, and only
            // the lanes that lost a race go round again.
            float x[VEC];
            uint32_t cell[VEC], seen[VEC];
            uint32_t open = 0;          // bit v: the value still has to reach its cell
            if (in[k]) {
                GIO::unpack(g[k], x);
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    // the index as two 32-bit words: a row is below 2^31
                    const uint32_t lo32 = raw_word(r[k][v / 2], 2 * (v % 2)), hi32 = raw_word(r[k][v / 2], 2 * (v % 2) + 1);
                    const bool ok = hi32 == 0u && lo32 < (uint32_t)rows;
                    cell[v] = ok ? lo32 : 0u;
                    seen[v] = ok ? cells[cell[v]] : 0u;
                    open |= ok ? 1u << v : 0u;
                }
            }
            while (open != 0) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    if ((open >> v & 1u) != 0) {
                        const uint32_t expect = seen[v];
                        const uint32_t sum = __float_as_uint(__uint_as_float(expect) + x[v]);
                        seen[v] = atomicCAS(cells + cell[v], expect, sum);
                        if (seen[v] == expect) open &= ~(1u << v);
                    }
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
    // one round of workgroups: as many as fit the 256 compute units at once (4 of 512 threads each, fewer when the
    // column takes more than a quarter of a unit's 160 KB of LDS), and no slice shorter than 16 000 values
    const size_t lds_bytes = (size_t)rows * sizeof(float);
    const int per_unit = (int)max((size_t)1, min((size_t)4, (size_t)(160 * 1024) / max(lds_bytes, (size_t)1)));
    const int64_t total = per_image / vec * B;
    const int64_t want = (total * vec + 16383) / 16384;
    const int64_t cap = max(1, 256 * per_unit / H);
    const int slices = (int)max((int64_t)1, min(want, cap));
    const int64_t per_slice = (total + slices - 1) / slices;
    const dim3 grid((unsigned)slices, (unsigned)H);
    const size_t lds = lds_bytes;
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
