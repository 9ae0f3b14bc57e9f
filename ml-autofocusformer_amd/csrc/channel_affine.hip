// channel_affine_gelu: y = GELU(x * scale[c] + shift[c]) over an (B, C, H, W) tensor of 16-bit data.
//
// The patch embedding of the reference model runs convolution, BatchNorm and GELU one after the other
// (models/aff_transformer.py:542: `self.act1(self.bn(self.proj1(x)))`).  In inference BatchNorm is an affine map
// per channel, so the convolution's bias, the normalisation and the activation are one pass over the convolution's
// output: scale = gamma / sqrt(running_var + eps), shift = (conv_bias - running_mean) * scale + beta, prepared by
// the caller.  Arithmetic in fp32, one rounding to the storage type.  It has no counterpart in the reference's
// extension modules.
#include "gelu.hpp"
#include "launch.hpp"

namespace clusten {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void channel_affine_gelu_kernel(const T* __restrict__ x, const float* __restrict__ scale,
                                                                  const float* __restrict__ shift, T* __restrict__ y, int C,
                                                                  int pieces_per_plane) {
    // blockIdx.y: the (image, channel) plane; a thread owns 16-byte pieces (8 elements) of it
    const int c = blockIdx.y % C;
    const float a = scale[c], b = shift[c];
    const int64_t plane = (int64_t)blockIdx.y * pieces_per_plane;
    for (int p = blockIdx.x * 256 + threadIdx.x; p < pieces_per_plane; p += gridDim.x * 256) {
        float v[8];
        VecIO<T, 8>::unpack(*reinterpret_cast<const Piece*>(x + (plane + p) * 8), v);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = gelu_erf(v[e] * a + b);
        *reinterpret_cast<Piece*>(y + (plane + p) * 8) = VecIO<T, 8>::pack(v);
    }
}

}  // namespace

int launch_channel_affine_gelu(const void* x, const float* scale, const float* shift, void* y, int64_t B, int C, int HW,
                               int dtype, hipStream_t stream) {
    const int pieces = HW / 8;
    const int64_t planes = B * C;
    if (planes >= 65536) return CLUSTEN_ERR_BAD_DIMS;
    const dim3 grid((unsigned)min((pieces + 255) / 256, 64), (unsigned)planes);
    if (dtype == CLUSTEN_F16) {
        hipLaunchKernelGGL(channel_affine_gelu_kernel<f16_t>, grid, dim3(256), 0, stream, static_cast<const f16_t*>(x), scale,
                           shift, static_cast<f16_t*>(y), C, pieces);
    } else if (dtype == CLUSTEN_BF16) {
        hipLaunchKernelGGL(channel_affine_gelu_kernel<bf16_t>, grid, dim3(256), 0, stream, static_cast<const bf16_t*>(x),
                           scale, shift, static_cast<bf16_t*>(y), C, pieces);
    } else {
        return CLUSTEN_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace clusten
