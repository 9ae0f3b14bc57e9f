// layer_norm: y = (x - mean(x)) * rsqrt(var(x) + eps) * weight + bias over the last axis of an fp32, fp16 or bf16
// tensor, computed in fp32 and written as fp32, fp16 or bf16.
//
// The reference model normalises the token features before every attention and MLP block, before each merge
// projection and at the end (`nn.LayerNorm`, models/aff_transformer.py:220, 231, 362, 546, 663); under mixed
// precision the normalisation runs in fp32 (a 16-bit input is widened first) and the Linear layer that follows
// rounds its input to 16 bits.  This kernel does all of that in one pass over the rows (64 to 1024 channels: a row
// is a few hundred bytes, which the framework's general kernel handles at a fraction of the memory bandwidth).  A
// second form takes the residual addition ahead of the norm along (`x = x + drop_path(branch)` followed by
// `norm(x)`: models/aff_transformer.py:230-231, and :232 with the next block's :219): it writes the sum, rounded as the
// framework's addition leaves it, and the normalised row in one pass.  A third form reads the rows of every image
// in a given order and adds a per-channel bias first: the norm at the end of the patch embedding
// (models/aff_transformer.py:542-546), with the second convolution's bias and the reordering of the tokens into
// cluster order (:465-466, the first stage) taken along.  None has a counterpart in the reference's extension
// modules.
//
// A row is held by L lanes, W consecutive channels per lane and step (W = 8 when a 16-bit tensor is among the
// operands, so that their accesses are 16 bytes per lane, else 4), C / (W L) steps; mean and variance are two reductions over registers (the
// variance from the centred values, as a two-pass computation gives it), across the lanes of the row with xor
// shuffles.  All arithmetic is fp32.
#include <type_traits>

#include "launch.hpp"

namespace clusten {
namespace {

template <int L>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
    for (int m = 1; m < L; m <<= 1) v += __shfl_xor(v, m);
    return v;
}

// W consecutive elements of a row (4 or 8) between memory and fp32 registers, in 16-byte accesses where W elements
// fill them.
template <typename T, int W>
__device__ __forceinline__ void load_run(const T* p, float (&x)[W]) {
    if constexpr (W == 4) {
        Quad<T>::unpack(*reinterpret_cast<const typename Quad<T>::raw*>(p), x);
    } else if constexpr (sizeof(T) == 2) {
        VecIO<T, 8>::unpack(*reinterpret_cast<const typename VecIO<T, 8>::raw*>(p), x);
    } else {
        float lo[4], hi[4];
        Quad<T>::unpack(*reinterpret_cast<const typename Quad<T>::raw*>(p), lo);
        Quad<T>::unpack(*reinterpret_cast<const typename Quad<T>::raw*>(p + 4), hi);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = lo[e], x[4 + e] = hi[e];
    }
}
template <typename T, int W>
__device__ __forceinline__ void store_run(T* p, const float (&x)[W]) {
    if constexpr (W == 4) {
        *reinterpret_cast<typename Quad<T>::raw*>(p) = Quad<T>::pack(x);
    } else if constexpr (sizeof(T) == 2) {
        *reinterpret_cast<typename VecIO<T, 8>::raw*>(p) = VecIO<T, 8>::pack(x);
    } else {
        const float lo[4] = {x[0], x[1], x[2], x[3]}, hi[4] = {x[4], x[5], x[6], x[7]};
        *reinterpret_cast<typename Quad<T>::raw*>(p) = Quad<T>::pack(lo);
        *reinterpret_cast<typename Quad<T>::raw*>(p + 4) = Quad<T>::pack(hi);
    }
}

// ResT = void: plain layer norm of x.  Otherwise the row normalised is x + branch (the residual connection ahead of
// the norm), rounded to x's type as the framework's addition would leave it and also written to `sum_out`.
// A row is held by L lanes, W consecutive channels per lane and step, V steps: C = W * L * V.
template <typename InT, typename ResT, typename OutT, int L, int V, int W>
__global__ __launch_bounds__(256) void layer_norm_kernel(const InT* __restrict__ x, const ResT* __restrict__ branch,
                                                         InT* __restrict__ sum_out, const float* __restrict__ weight,
                                                         const float* __restrict__ bias, OutT* __restrict__ out,
                                                         int64_t rows, float eps, const int64_t* __restrict__ order,
                                                         int group, const InT* __restrict__ pre_bias) {
    constexpr int C = W * L * V;
    constexpr int ROWS_PER_WG = 256 / L;
    const int sub = threadIdx.x % L;
    const int64_t row_raw = (int64_t)blockIdx.x * ROWS_PER_WG + threadIdx.x / L;
    const bool live = row_raw < rows;
    const int64_t row = live ? row_raw : rows - 1;  // every lane stays in the shuffles
    // with `order`: output row g * group + i is the norm of input row g * group + order[i] (the rows of every group
    // of `group` rows, an image's tokens, permuted the same way)
    const int64_t src = order ? row - row % group + order[row % group] : row;
    const InT* xr = x + src * C;
    float v[V][W];
#pragma unroll
    for (int s = 0; s < V; ++s) {
        const int c = W * (s * L + sub);
        load_run<InT, W>(xr + c, v[s]);
        if (pre_bias) {  // a per-channel bias the producer left out, added as its own addition would have: rounded
            float pb[W];
            load_run<InT, W>(pre_bias + c, pb);
#pragma unroll
            for (int e = 0; e < W; ++e) v[s][e] = to_acc(from_acc<InT>(v[s][e] + pb[e]));
        }
        if constexpr (!std::is_void<ResT>::value) {
            float br[W];
            load_run<ResT, W>(branch + row * C + c, br);
#pragma unroll
            for (int e = 0; e < W; ++e) v[s][e] = to_acc(from_acc<InT>(v[s][e] + br[e]));
            if (live) store_run<InT, W>(sum_out + row * C + c, v[s]);
        }
    }
    // sums in the order ((a + b) + (c + d)) per group of four, groups in channel order
    float sum = 0.f;
#pragma unroll
    for (int s = 0; s < V; ++s) {
#pragma unroll
        for (int e = 0; e < W; e += 4) sum += (v[s][e] + v[s][e + 1]) + (v[s][e + 2] + v[s][e + 3]);
    }
    const float mean = row_sum<L>(sum) * (1.f / C);
    float sq = 0.f;
#pragma unroll
    for (int s = 0; s < V; ++s) {
#pragma unroll
        for (int e = 0; e < W; ++e) v[s][e] -= mean;
#pragma unroll
        for (int e = 0; e < W; e += 4) {
            sq += (v[s][e] * v[s][e] + v[s][e + 1] * v[s][e + 1]) + (v[s][e + 2] * v[s][e + 2] + v[s][e + 3] * v[s][e + 3]);
        }
    }
    const float rstd = rsqrtf(row_sum<L>(sq) * (1.f / C) + eps);
    if (!live) return;
    OutT* orow = out + row * C;
#pragma unroll
    for (int s = 0; s < V; ++s) {
        const int c = W * (s * L + sub);
        float y[W];
#pragma unroll
        for (int e = 0; e < W; e += 4) {
            const float4 w = *reinterpret_cast<const float4*>(weight + c + e);
            const float4 b = *reinterpret_cast<const float4*>(bias + c + e);
            y[e] = v[s][e] * rstd * w.x + b.x;
            y[e + 1] = v[s][e + 1] * rstd * w.y + b.y;
            y[e + 2] = v[s][e + 2] * rstd * w.z + b.z;
            y[e + 3] = v[s][e + 3] * rstd * w.w + b.w;
        }
        store_run<OutT, W>(orow + c, y);
    }
}

template <typename InT, typename ResT, typename OutT, int L, int V, int W = 4>
int launch_lv(const void* x, const void* branch, void* sum_out, const float* weight, const float* bias, void* out,
              int64_t rows, float eps, hipStream_t stream, const int64_t* order = nullptr, int group = 1,
              const void* pre_bias = nullptr) {
    constexpr int ROWS_PER_WG = 256 / L;
    const int64_t blocks = (rows + ROWS_PER_WG - 1) / ROWS_PER_WG;
    hipLaunchKernelGGL((layer_norm_kernel<InT, ResT, OutT, L, V, W>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const InT*>(x), static_cast<const ResT*>(branch), static_cast<InT*>(sum_out), weight,
                       bias, static_cast<OutT*>(out), rows, eps, order, group, static_cast<const InT*>(pre_bias));
    return launch_status();
}

template <typename InT, typename ResT, typename OutT>
int launch_typed(const void* x, const void* branch, void* sum_out, const float* weight, const float* bias, void* out,
                 int64_t rows, int C, float eps, hipStream_t stream, const int64_t* order = nullptr, int group = 1,
                 const void* pre_bias = nullptr) {
    // eight channels per lane (16-byte accesses to 16-bit rows) when a 16-bit tensor is among the operands
    constexpr bool wide = sizeof(InT) == 2 || sizeof(OutT) == 2;
#define CLUSTEN_LN_ARGS x, branch, sum_out, weight, bias, out, rows, eps, stream, order, group, pre_bias
    if constexpr (wide) {
        switch (C) {
            case 64: return launch_lv<InT, ResT, OutT, 8, 1, 8>(CLUSTEN_LN_ARGS);
            case 128: return launch_lv<InT, ResT, OutT, 16, 1, 8>(CLUSTEN_LN_ARGS);
            case 256: return launch_lv<InT, ResT, OutT, 32, 1, 8>(CLUSTEN_LN_ARGS);
            case 384: return launch_lv<InT, ResT, OutT, 16, 3, 8>(CLUSTEN_LN_ARGS);
            case 512: return launch_lv<InT, ResT, OutT, 64, 1, 8>(CLUSTEN_LN_ARGS);
            case 768: return launch_lv<InT, ResT, OutT, 32, 3, 8>(CLUSTEN_LN_ARGS);
            case 1024: return launch_lv<InT, ResT, OutT, 64, 2, 8>(CLUSTEN_LN_ARGS);
            default: return CLUSTEN_ERR_BAD_DIMS;
        }
    }
    switch (C) {
        case 64: return launch_lv<InT, ResT, OutT, 16, 1>(CLUSTEN_LN_ARGS);
        case 128: return launch_lv<InT, ResT, OutT, 32, 1>(CLUSTEN_LN_ARGS);
        case 256: return launch_lv<InT, ResT, OutT, 64, 1>(CLUSTEN_LN_ARGS);
        case 384: return launch_lv<InT, ResT, OutT, 32, 3>(CLUSTEN_LN_ARGS);
        case 512: return launch_lv<InT, ResT, OutT, 64, 2>(CLUSTEN_LN_ARGS);
        case 768: return launch_lv<InT, ResT, OutT, 64, 3>(CLUSTEN_LN_ARGS);
        case 1024: return launch_lv<InT, ResT, OutT, 64, 4>(CLUSTEN_LN_ARGS);
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
#undef CLUSTEN_LN_ARGS
}

template <typename InT>
int launch_in(const void* x, const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
              int out_dtype, hipStream_t stream, const int64_t* order = nullptr, int group = 1,
              const void* pre_bias = nullptr) {
    switch (out_dtype) {
        case CLUSTEN_F32:
            return launch_typed<InT, void, float>(x, nullptr, nullptr, weight, bias, out, rows, C, eps, stream, order, group,
                                                  pre_bias);
        case CLUSTEN_F16:
            return launch_typed<InT, void, f16_t>(x, nullptr, nullptr, weight, bias, out, rows, C, eps, stream, order, group,
                                                  pre_bias);
        case CLUSTEN_BF16:
            return launch_typed<InT, void, bf16_t>(x, nullptr, nullptr, weight, bias, out, rows, C, eps, stream, order,
                                                   group, pre_bias);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

// x + branch, then the norm, written in the 16-bit type T of the branch: x is fp32 or T
template <typename T>
int launch_add(const void* x, int x_dtype, const void* branch, void* sum_out, const float* weight, const float* bias,
               void* out, int64_t rows, int C, float eps, int t_code, hipStream_t stream) {
    if (x_dtype == CLUSTEN_F32) return launch_typed<float, T, T>(x, branch, sum_out, weight, bias, out, rows, C, eps, stream);
    if (x_dtype == t_code) return launch_typed<T, T, T>(x, branch, sum_out, weight, bias, out, rows, C, eps, stream);
    return CLUSTEN_ERR_BAD_DTYPE;
}

}  // namespace

int launch_layer_norm(const void* x, int in_dtype, const float* weight, const float* bias, void* out, int64_t rows, int C,
                      float eps, int out_dtype, hipStream_t stream) {
    switch (in_dtype) {
        case CLUSTEN_F32: return launch_in<float>(x, weight, bias, out, rows, C, eps, out_dtype, stream);
        case CLUSTEN_F16: return launch_in<f16_t>(x, weight, bias, out, rows, C, eps, out_dtype, stream);
        case CLUSTEN_BF16: return launch_in<bf16_t>(x, weight, bias, out, rows, C, eps, out_dtype, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int launch_layer_norm_rows(const void* x, int in_dtype, const int64_t* order, int group, const void* pre_bias,
                           const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
                           int out_dtype, hipStream_t stream) {
    switch (in_dtype) {
        case CLUSTEN_F32:
            return launch_in<float>(x, weight, bias, out, rows, C, eps, out_dtype, stream, order, group, pre_bias);
        case CLUSTEN_F16:
            return launch_in<f16_t>(x, weight, bias, out, rows, C, eps, out_dtype, stream, order, group, pre_bias);
        case CLUSTEN_BF16:
            return launch_in<bf16_t>(x, weight, bias, out, rows, C, eps, out_dtype, stream, order, group, pre_bias);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int launch_add_layer_norm(const void* x, int x_dtype, const void* branch, int branch_dtype, void* sum_out,
                          const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
                          hipStream_t stream) {
    if (branch_dtype == CLUSTEN_F16) {
        return launch_add<f16_t>(x, x_dtype, branch, sum_out, weight, bias, out, rows, C, eps, CLUSTEN_F16, stream);
    }
    if (branch_dtype == CLUSTEN_BF16) {
        return launch_add<bf16_t>(x, x_dtype, branch, sum_out, weight, bias, out, rows, C, eps, CLUSTEN_BF16, stream);
    }
    return CLUSTEN_ERR_BAD_DTYPE;
}

}  // namespace clusten
