// skinny_linear: y = act(x W^T + b) for a tall activation matrix and a small weight matrix, 16-bit data.
//
//   y[m,n] = act( sum_k x[m,k] * W[n,k] + b[n] ),   x (M,K), W (NOUT,K), b (NOUT), y (M,NOUT);  act = identity or GELU
//
// The Linear layers around the first-stage attention of the reference model (`nn.Linear` q, kv, proj at
// models/aff_transformer.py:60-68, the MLP at :181-196) have K and NOUT of 64 to 192 and some 400 000 rows: they
// move memory, not flops (100-200 MB against 3-10 GFLOP), and what matters is that x is read once, y written once
// and nothing else happens.  The whole weight matrix lives in the registers of every wave as the A operand of the
// matrix instructions (K * NOUT <= 12288 elements: 96 registers), a wave walks blocks of 16 rows with the next
// block's rows requested before the current one is multiplied, and the product is taken transposed
// (y^T = W x^T) with the weight rows dealt to the instruction's rows such that every lane ends up with 8
// consecutive output channels of one row: one 16-byte store.  Sums are fp32; with GELU the sum is rounded to the
// storage type first, as the separate activation kernel of the framework sees it.  It has no counterpart in the
// reference's extension modules.
#include "gelu.hpp"
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kLinearWaves = 4;        // waves per workgroup
constexpr int kLinearGroups = 512;     // workgroups at most: 8 waves per compute unit

template <typename T, int K, int NOUT, int ACT>
__global__ __launch_bounds__(64 * kLinearWaves, 2) void skinny_linear_kernel(const T* __restrict__ x, int64_t ldx,
                                                                         const T* __restrict__ w,
                                                                         const T* __restrict__ bias, T* __restrict__ y,
                                                                         int64_t M, int64_t blocks) {
    constexpr int KS = K / 32;       // k steps of the 16x16x32 instruction
    constexpr int CB = NOUT / 16;    // 16-channel blocks
    constexpr int D = K <= 64 ? 4 : 2;  // row blocks a wave has requested ahead (2 KB to 6 KB each)
    static_assert(K % 32 == 0 && NOUT % 32 == 0, "whole k steps, pairs of channel blocks");
    __shared__ __attribute__((aligned(16))) float bias_lds[NOUT];
    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15, kq = lane >> 4;

    for (int n = threadIdx.x; n < NOUT; n += 64 * kLinearWaves) bias_lds[n] = bias ? to_acc(bias[n]) : 0.f;

    // Weight operand.  Row i = 4*q + j of channel block 2p+u is output channel 32p + 8q + 4u + j, so that the lane
    // holding result rows 4*kq .. 4*kq+3 of blocks 2p and 2p+1 holds channels 32p + 8*kq .. +7.
    Piece wreg[CB][KS];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        const int ch = 32 * (cb >> 1) + 8 * (r16 >> 2) + 4 * (cb & 1) + (r16 & 3);
#pragma unroll
        for (int s = 0; s < KS; ++s) wreg[cb][s] = *reinterpret_cast<const Piece*>(w + ch * K + 32 * s + 8 * kq);
    }
    __syncthreads();

    const int64_t wave = (int64_t)blockIdx.x * kLinearWaves + (threadIdx.x >> 6);
    const int64_t waves = (int64_t)gridDim.x * kLinearWaves;
    const uint32_t pitch = (uint32_t)ldx * 2;

    auto load_rows = [&](int64_t rb, Piece (&xa)[KS]) {
        const int64_t row0 = rb * 16;
        const int rows_here = (int)min((int64_t)16, M - row0);
        const char* xb = reinterpret_cast<const char*>(x + row0 * ldx);
        const uint32_t off = (uint32_t)min(r16, rows_here - 1) * pitch + (uint32_t)kq * 16;
#pragma unroll
        for (int s = 0; s < KS; ++s) xa[s] = *reinterpret_cast<const Piece*>(xb + lane_offset(off + 64 * s));
    };

    Piece xq[D][KS];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        if (wave + d * waves < blocks) load_rows(wave + d * waves, xq[d]);
    }
    for (int64_t rb0 = wave; rb0 < blocks; rb0 += D * waves) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int64_t rb = rb0 + d * waves;
            if (rb < blocks) {
                F32x4 acc[CB];
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    acc[cb] = F32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < KS; ++s) acc[cb] = tile_mfma<T>(wreg[cb][s], xq[d][s], acc[cb]);
                }
                // the operands are consumed: their registers take the rows of D blocks further on
                if (rb + D * waves < blocks) load_rows(rb + D * waves, xq[d]);
                const int64_t row = rb * 16 + r16;
                if (row < M) {
                    T* yrow = y + row * NOUT + 8 * kq;
#pragma unroll
                    for (int p = 0; p < CB / 2; ++p) {
                        const F32x4 b0 = *reinterpret_cast<const F32x4*>(bias_lds + 32 * p + 8 * kq);
                        const F32x4 b1 = *reinterpret_cast<const F32x4*>(bias_lds + 32 * p + 8 * kq + 4);
                        float v[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            v[e] = acc[2 * p + (e >> 2)][e & 3] + (e < 4 ? b0[e & 3] : b1[e & 3]);
                            if (ACT == 1) v[e] = gelu_erf(to_acc(from_acc<T>(v[e])));
                        }
                        *reinterpret_cast<Piece*>(yrow + 32 * p) = VecIO<T, 8>::pack(v);
                    }
                }
            }
        }
    }
}

template <typename T, int K, int NOUT, int ACT>
int launch_kn(const void* x, int64_t ldx, const void* w, const void* bias, void* y, int64_t M, hipStream_t stream) {
    const int64_t blocks = (M + 15) / 16;
    const int64_t groups = min((blocks + kLinearWaves - 1) / kLinearWaves, (int64_t)kLinearGroups);
    hipLaunchKernelGGL((skinny_linear_kernel<T, K, NOUT, ACT>), dim3((unsigned)groups), dim3(64 * kLinearWaves), 0, stream,
                       static_cast<const T*>(x), ldx, static_cast<const T*>(w), static_cast<const T*>(bias),
                       static_cast<T*>(y), M, blocks);
    return launch_status();
}

template <typename T>
int launch_typed(const void* x, int64_t ldx, const void* w, const void* bias, void* y, int64_t M, int K, int NOUT, int act,
                 hipStream_t stream) {
    if (act == 0) {
        if (K == 64 && NOUT == 64) return launch_kn<T, 64, 64, 0>(x, ldx, w, bias, y, M, stream);
        if (K == 64 && NOUT == 128) return launch_kn<T, 64, 128, 0>(x, ldx, w, bias, y, M, stream);
        if (K == 64 && NOUT == 192) return launch_kn<T, 64, 192, 0>(x, ldx, w, bias, y, M, stream);
        if (K == 192 && NOUT == 64) return launch_kn<T, 192, 64, 0>(x, ldx, w, bias, y, M, stream);
        if (K == 128 && NOUT == 64) return launch_kn<T, 128, 64, 0>(x, ldx, w, bias, y, M, stream);
    } else {
        if (K == 64 && NOUT == 64) return launch_kn<T, 64, 64, 1>(x, ldx, w, bias, y, M, stream);
        if (K == 64 && NOUT == 128) return launch_kn<T, 64, 128, 1>(x, ldx, w, bias, y, M, stream);
        if (K == 64 && NOUT == 192) return launch_kn<T, 64, 192, 1>(x, ldx, w, bias, y, M, stream);
    }
    return CLUSTEN_ERR_BAD_DIMS;
}

}  // namespace

bool skinny_linear_supported(int K, int NOUT, int act) {
    if (act == 0) return (K == 64 && (NOUT == 64 || NOUT == 128 || NOUT == 192)) || ((K == 192 || K == 128) && NOUT == 64);
    return act == 1 && K == 64 && (NOUT == 64 || NOUT == 128 || NOUT == 192);
}

int launch_skinny_linear(const void* x, int64_t ldx, const void* w, const void* bias, void* y, int64_t M, int K, int NOUT,
                         int act, int dtype, hipStream_t stream) {
    if (dtype == CLUSTEN_F16) return launch_typed<f16_t>(x, ldx, w, bias, y, M, K, NOUT, act, stream);
    if (dtype == CLUSTEN_BF16) return launch_typed<bf16_t>(x, ldx, w, bias, y, M, K, NOUT, act, stream);
    return CLUSTEN_ERR_BAD_DTYPE;
}

}  // namespace clusten
