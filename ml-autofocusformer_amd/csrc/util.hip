// Small streaming kernels: zero fill, fp32 -> fp16/bf16 rounding.
#include "launch.hpp"

namespace clusten {

namespace {

constexpr int kBlock = 256;
constexpr int kMaxGrid = 256 * 64;  // 64 workgroups of 4 waves per CU: enough to keep every CU's queues full

// `only_if` (may be null): a device flag; the kernel does nothing when it points to zero.
template <typename W>
__global__ __launch_bounds__(kBlock) void zero_kernel(W* __restrict__ dst, size_t count, const int32_t* only_if) {
    if (only_if != nullptr && *only_if == 0) return;
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < count; i += stride) dst[i] = W(0);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void round_kernel(const float* __restrict__ src, T* __restrict__ dst,
                                                      size_t count, const int32_t* only_if) {
    if (only_if != nullptr && *only_if == 0) return;
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < count; i += stride) dst[i] = from_acc<T>(src[i]);
}

inline int grid_for(size_t items) {
    const size_t want = (items + kBlock - 1) / kBlock;
    return (int)(want < (size_t)kMaxGrid ? (want ? want : 1) : (size_t)kMaxGrid);
}

}  // namespace

int launch_zero_f32(float* dst, size_t count, hipStream_t stream, const int32_t* only_if) {
    // whole 16-byte pieces when the buffer allows it
    if (aligned16(dst) && count % 4 == 0) {
        hipLaunchKernelGGL((zero_kernel<Piece>), dim3(grid_for(count / 4)), dim3(kBlock), 0, stream,
                           reinterpret_cast<Piece*>(dst), count / 4, only_if);
    } else {
        hipLaunchKernelGGL((zero_kernel<float>), dim3(grid_for(count)), dim3(kBlock), 0, stream, dst, count, only_if);
    }
    return launch_status();
}

int launch_zero_f64(double* dst, size_t count, hipStream_t stream) {
    hipLaunchKernelGGL((zero_kernel<double>), dim3(grid_for(count)), dim3(kBlock), 0, stream, dst, count,
                       static_cast<const int32_t*>(nullptr));
    return launch_status();
}

int launch_round_from_f32(const float* src, void* dst, size_t count, int dtype, hipStream_t stream,
                          const int32_t* only_if) {
    if (dtype == CLUSTEN_F16) {
        hipLaunchKernelGGL((round_kernel<f16_t>), dim3(grid_for(count)), dim3(kBlock), 0, stream, src,
                           static_cast<f16_t*>(dst), count, only_if);
    } else if (dtype == CLUSTEN_BF16) {
        hipLaunchKernelGGL((round_kernel<bf16_t>), dim3(grid_for(count)), dim3(kBlock), 0, stream, src,
                           static_cast<bf16_t*>(dst), count, only_if);
    } else {
        return CLUSTEN_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace clusten
