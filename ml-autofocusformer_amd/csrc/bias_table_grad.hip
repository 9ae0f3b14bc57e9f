// bias_table_grad: the gradient of the relative-position bias table of an attention layer.
//
//   d_table[pe_idx[b,i,j], h] = sum over (b,i,j) of d_logit[b,h,i,j]
//
// the backward of `pe_table.gather(index=pe_idx...)` added to the attention logits (models/aff_transformer.py:131-133).
// The framework runs it as a scatter-add of B*H*N*M values into a table of some 12 000 rows: one global atomic per
// value, all of them on the same few hundred kilobytes.  Here a workgroup takes one head and a contiguous slice of the
// head's values (images one after the other) and sums into a copy of that head's column of the table in LDS; what it
// has collected goes to memory with one global atomic per touched row.
// The position indices of a model are offsets between neighbouring tokens: a few hundred cells around the table's
// centre take all the additions (on such indices a loop of compare-and-swap additions of floats spends its time on
// lost races, 420 us against 90 us on indices spread over the table).  So a cell is a 64-bit integer: a value enters
// as a multiple of 2^-40 of the power of two above the slice's largest magnitude, the additions are LDS integer
// atomics, which the hardware serialises without a retry, and the sum of a slice is exact whatever the order.  fp16
// values need no look at the slice (all are multiples of 2^-24 below 2^16: every sum is exact); for fp32 and bf16 the
// workgroup first sweeps its slice for the largest magnitude.
// The LDS copy holds 20 000 cells (160 KB): the whole column of a table of up to 20 000 rows, else the 20 000 rows
// around the table's centre (the offset zero of a (2r+1)^2 table is its middle row); values for rows outside that
// window go to the table with a global atomic each.
// The grid is one round of workgroups of 512 threads: the global atomics of the flush all land on the same few
// kilobytes, so a workgroup should flush once for a long slice.  A thread reads four consecutive values at a time
// (two 16-byte loads of indices, one load of gradients) and keeps four such groups in flight.
// d_table is fp32 and zeroed by the caller.  It has no counterpart in the reference's extension modules.
#include <type_traits>

#include "launch.hpp"

namespace clusten {
namespace {

constexpr int kGradThreads = 512;
constexpr int kGradWindow = 20000;         // 64-bit cells of the LDS copy: 160 000 bytes
constexpr int kGradGroups = 4;             // groups of 4 values in flight per thread
constexpr int kFixedBits = 40;             // a value of the slice's top binade has 41 bits; 2^21 of them fit a cell
constexpr int64_t kFixedSliceMax = 1 << 21;   // values of a slice
constexpr int kHalfTop = 142;              // fp32 exponent field of the binade [2^15, 2^16): no fp16 value lies above it

// x in units of 2^(e_top - 127 - kFixedBits), truncated towards zero; |x| < 2^(e_top - 126) gives |result| < 2^41.
__device__ __forceinline__ long long to_fixed(float x, int e_top) {
    const uint32_t bits = __float_as_uint(x);
    const int e = (int)(bits >> 23) & 0xff;
    const uint32_t mant = (bits & 0x7fffffu) | (e != 0 ? 0x800000u : 0u);
    // x = mant * 2^(max(e,1) - 150); the unit is 2^(e_top - 127 - 40)
    const int sh = max(e, 1) - e_top + (kFixedBits - 23);
    const unsigned long long mag = sh >= 0 ? (unsigned long long)mant << min(sh, kFixedBits - 23)
                                           : (unsigned long long)(mant >> min(-sh, 31));
    return (bits >> 31) != 0 ? -(long long)mag : (long long)mag;
}

// The position (image, group in the image) of a thread's next group of VEC values inside the head's slice, stepped
// without a division.
struct SliceWalk {
    int64_t f, b, e;
    __device__ __forceinline__ void start(int64_t lo, int64_t groups_per_image) {
        f = lo + threadIdx.x;
        b = f / groups_per_image;
        e = f - b * groups_per_image;
    }
    __device__ __forceinline__ void step(int64_t groups_per_image, int B) {
        e += kGradThreads;
        while (e >= groups_per_image) {   // (at most once unless an image holds fewer groups than there are threads)
            e -= groups_per_image;
            b = min(b + 1, (int64_t)B - 1);
        }
    }
};

// VEC = 4: per_image % 4 == 0 and both tensors 16-byte aligned (a group never straddles two images); VEC = 1 otherwise.
// The LDS copy covers the rows [win_lo, win_lo + win_cells) of the table (win_cells * 8 + 16 bytes of dynamic LDS).
template <typename T, int VEC>
__global__ __launch_bounds__(kGradThreads) void bias_table_grad_kernel(const T* __restrict__ d_logit,
                                                                       const int64_t* __restrict__ pe_idx,
                                                                       float* __restrict__ d_table, int H, int rows,
                                                                       int win_lo, int win_cells, int64_t per_image,
                                                                       int64_t per_slice, int B) {
    typedef VecIO<T, VEC> GIO;
    typedef typename RawBytes<VEC == 4 ? 16 : 8>::type IdxRaw;   // two indices (VEC = 4: a group is two of them) or one
    constexpr int IR = VEC == 4 ? 2 : 1;
    // win_cells 64-bit sums and behind them the bits of the slice's largest finite magnitude; no other LDS variable,
    // so that the array starts at offset 0 (64-bit LDS atomics fault on an address that is not 8-byte aligned)
    extern __shared__ __attribute__((aligned(16))) unsigned long long sums[];
    uint32_t* slice_top = reinterpret_cast<uint32_t*>(sums + win_cells);
    const int h = blockIdx.y;
    for (int r = threadIdx.x; r < win_cells; r += kGradThreads) sums[r] = 0ull;
    if (threadIdx.x == 0) *slice_top = 0u;
    __syncthreads();
    // slice blockIdx.x of the head's B * per_image / VEC groups of values
    const int64_t groups_per_image = per_image / VEC;
    const int64_t total = groups_per_image * B;
    const int64_t lo = (int64_t)blockIdx.x * per_slice, hi = min(total, lo + per_slice);
    int e_top = kHalfTop;
    if constexpr (!std::is_same<T, f16_t>::value) {
        // first sweep: the largest finite magnitude of the slice names the binade the cells' unit hangs on
        uint32_t top = 0u;
        SliceWalk w;
        w.start(lo, groups_per_image);
        for (; w.f < hi; w.f += kGradGroups * kGradThreads) {
            typename GIO::raw g[kGradGroups];
            bool in[kGradGroups];
#pragma unroll
            for (int k = 0; k < kGradGroups; ++k) {
                in[k] = w.f + k * kGradThreads < hi;
                if (in[k]) g[k] = *reinterpret_cast<const typename GIO::raw*>(d_logit + ((w.b * H + h) * groups_per_image + w.e) * VEC);
                w.step(groups_per_image, B);
            }
#pragma unroll
            for (int k = 0; k < kGradGroups; ++k) {
                if (in[k]) {
                    float x[VEC];
                    GIO::unpack(g[k], x);
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        const uint32_t m = __float_as_uint(x[v]) & 0x7fffffffu;
                        top = m < 0x7f800000u ? max(top, m) : top;
                    }
                }
            }
        }
        atomicMax(slice_top, top);
        __syncthreads();
        e_top = max(1, (int)(*slice_top >> 23));
    }
    SliceWalk w;
    w.start(lo, groups_per_image);
    for (; w.f < hi; w.f += kGradGroups * kGradThreads) {
        IdxRaw r[kGradGroups][IR];
        typename GIO::raw g[kGradGroups];
        bool in[kGradGroups];
#pragma unroll
        for (int k = 0; k < kGradGroups; ++k) {   // independent loads before the first addition
            in[k] = w.f + k * kGradThreads < hi;
            if (in[k]) {
#pragma unroll
                for (int q = 0; q < IR; ++q) {
                    r[k][q] = *reinterpret_cast<const IdxRaw*>(pe_idx + (w.b * groups_per_image + w.e) * VEC + 2 * q);
                }
                g[k] = *reinterpret_cast<const typename GIO::raw*>(d_logit + ((w.b * H + h) * groups_per_image + w.e) * VEC);
            }
            w.step(groups_per_image, B);
        }
#pragma unroll
        for (int k = 0; k < kGradGroups; ++k) {
            if (in[k]) {
                float x[VEC];
                GIO::unpack(g[k], x);
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    // the index as two 32-bit words: a row is below 2^31; entries outside the table are skipped
                    const uint32_t lo32 = raw_word(r[k][v / 2], 2 * (v % 2)), hi32 = raw_word(r[k][v / 2], 2 * (v % 2) + 1);
                    if (hi32 == 0u && lo32 < (uint32_t)rows) {
                        const uint32_t cell = lo32 - (uint32_t)win_lo;
                        const bool finite = (__float_as_uint(x[v]) & 0x7f800000u) != 0x7f800000u;
                        if (cell < (uint32_t)win_cells && finite) {
                            atomicAdd(sums + cell, (unsigned long long)to_fixed(x[v], e_top));
                        } else {
                            // a row outside the window, or an infinity / a NaN, which has no integer: to the table as it is
                            unsafeAtomicAdd(d_table + (int64_t)lo32 * H + h, x[v]);
                        }
                    }
                }
            }
        }
    }
    __syncthreads();
    for (int r = threadIdx.x; r < win_cells; r += kGradThreads) {
        const long long v = (long long)sums[r];
        if (v != 0) unsafeAtomicAdd(d_table + (int64_t)(win_lo + r) * H + h, (float)ldexp((double)v, e_top - 127 - kFixedBits));
    }
}

template <typename T>
int launch_typed(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int rows, int64_t per_image,
                 hipStream_t stream) {
    const bool wide = per_image % 4 == 0 && aligned16(d_logit) && aligned16(pe_idx);
    const int vec = wide ? 4 : 1;
    const int win_cells = min(rows, kGradWindow), win_lo = (rows - win_cells) / 2;
    // one round of workgroups: as many as fit the 256 compute units at once (4 of 512 threads each, fewer when the
    // copy takes more than a quarter of a unit's 160 KB of LDS), no slice shorter than 16 000 values and none longer
    // than 2^21 (41 bits a value, 62 bits a sum)
    const size_t lds = (size_t)win_cells * sizeof(long long) + 16;
    const int per_unit = (int)max((size_t)1, min((size_t)4, (size_t)(160 * 1024) / lds));
    const int64_t total = per_image / vec * B;
    const int64_t want = (total * vec + 16383) / 16384;
    const int64_t cap = max(1, 256 * per_unit / H);
    int64_t slices = max((int64_t)1, min(want, cap));
    slices = max(slices, (total * vec + kFixedSliceMax - 1) / kFixedSliceMax);
    const int64_t per_slice = (total + slices - 1) / slices;
    const dim3 grid((unsigned)slices, (unsigned)H);
    const void* fn = wide ? reinterpret_cast<const void*>(bias_table_grad_kernel<T, 4>)
                          : reinterpret_cast<const void*>(bias_table_grad_kernel<T, 1>);
    if (lds > 48 * 1024) {   // more LDS than a workgroup gets without asking
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kGradWindow * (int)sizeof(long long) + 16) !=
            hipSuccess) {
            (void)hipGetLastError();
            return CLUSTEN_ERR_LAUNCH;
        }
    }
    if (wide) {
        hipLaunchKernelGGL((bias_table_grad_kernel<T, 4>), grid, dim3(kGradThreads), lds, stream,
                           static_cast<const T*>(d_logit), pe_idx, d_table, H, rows, win_lo, win_cells, per_image, per_slice, B);
    } else {
        hipLaunchKernelGGL((bias_table_grad_kernel<T, 1>), grid, dim3(kGradThreads), lds, stream,
                           static_cast<const T*>(d_logit), pe_idx, d_table, H, rows, win_lo, win_cells, per_image, per_slice, B);
    }
    return CLUSTEN_OK;
}

}  // namespace

int launch_bias_table_grad(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int N, int M, int rows,
                           int dtype, hipStream_t stream) {
    if (rows <= 0 || B <= 0 || H <= 0 || H > 65535) return CLUSTEN_ERR_BAD_DIMS;
    const int64_t per_image = (int64_t)N * M;
    int rc;
    switch (dtype) {
        case CLUSTEN_F32: rc = launch_typed<float>(d_logit, pe_idx, d_table, B, H, rows, per_image, stream); break;
        case CLUSTEN_F16: rc = launch_typed<f16_t>(d_logit, pe_idx, d_table, B, H, rows, per_image, stream); break;
        case CLUSTEN_BF16: rc = launch_typed<bf16_t>(d_logit, pe_idx, d_table, B, H, rows, per_image, stream); break;
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
    return rc != CLUSTEN_OK ? rc : launch_status();
}

}  // namespace clusten
