// add_row_score: the importance score of every token, with the residual addition ahead of it taken along.
//
//   sum[r,:]  = x[r,:] + branch[r,:]                        (optional; rounded to x's type, written to sum_out)
//   score[r]  = sigmoid( <sum[r,:] rounded to T, w> + b )   (T the 16-bit type of w; the product rounded to T
//                                                            before the sigmoid, as a Linear layer leaves it)
//
// The reference model scores the tokens of a stage before it merges them (`self.prob_net(feat).sigmoid()`,
// models/aff_transformer.py:498, a Linear layer with one output), right after the last block's residual addition
// (:232).  Under mixed precision the framework spends an addition, a cast of the token tensor, a matrix product with
// one column and an activation on it; here it is one pass over the rows.  A row is held by L lanes, four channels
// each per step, as in the layer-norm kernel.  It has no counterpart in the reference's extension modules.
#include <type_traits>

#include "launch.hpp"

namespace clusten {
namespace {

template <typename InT, typename ResT, typename T, int L, int V>
__global__ __launch_bounds__(256) void add_row_score_kernel(const InT* __restrict__ x, const ResT* __restrict__ branch,
                                                            InT* __restrict__ sum_out, const T* __restrict__ w,
                                                            const T* __restrict__ b, T* __restrict__ score, int64_t rows) {
    constexpr int C = 4 * L * V;
    constexpr int ROWS_PER_WG = 256 / L;
    const int sub = threadIdx.x % L;
    const int64_t row_raw = (int64_t)blockIdx.x * ROWS_PER_WG + threadIdx.x / L;
    const bool live = row_raw < rows;
    const int64_t row = live ? row_raw : rows - 1;  // every lane stays in the shuffles
    float dot = 0.f;
#pragma unroll
    for (int s = 0; s < V; ++s) {
        const int c = 4 * (s * L + sub);
        float in[4], wv[4];
        Quad<InT>::unpack(*reinterpret_cast<const typename Quad<InT>::raw*>(x + row * C + c), in);
        if constexpr (!std::is_void<ResT>::value) {
            float br[4];
            Quad<ResT>::unpack(*reinterpret_cast<const typename Quad<ResT>::raw*>(branch + row * C + c), br);
#pragma unroll
            for (int e = 0; e < 4; ++e) in[e] = to_acc(from_acc<InT>(in[e] + br[e]));
            if (live) *reinterpret_cast<typename Quad<InT>::raw*>(sum_out + row * C + c) = Quad<InT>::pack(in);
        }
        Quad<T>::unpack(*reinterpret_cast<const typename Quad<T>::raw*>(w + c), wv);
#pragma unroll
        for (int e = 0; e < 4; ++e) dot += to_acc(from_acc<T>(in[e])) * wv[e];
    }
#pragma unroll
    for (int m = 1; m < L; m <<= 1) dot += __shfl_xor(dot, m);
    if (live && sub == 0) {
        const float y = to_acc(from_acc<T>(dot + (b ? to_acc(*b) : 0.f)));
        score[row] = from_acc<T>(1.f / (1.f + __expf(-y)));
    }
}

template <typename InT, typename ResT, typename T>
int launch_c(const void* x, const void* branch, void* sum_out, const void* w, const void* b, void* score, int64_t rows,
             int C, hipStream_t stream) {
#define CLUSTEN_ROW_SCORE(LL, VV)                                                                                        \
    {                                                                                                                    \
        constexpr int per = 256 / LL;                                                                                    \
        hipLaunchKernelGGL((add_row_score_kernel<InT, ResT, T, LL, VV>), dim3((unsigned)((rows + per - 1) / per)),      \
                           dim3(256), 0, stream, static_cast<const InT*>(x), static_cast<const ResT*>(branch),          \
                           static_cast<InT*>(sum_out), static_cast<const T*>(w), static_cast<const T*>(b),               \
                           static_cast<T*>(score), rows);                                                                \
        return launch_status();                                                                                          \
    }
    switch (C) {
        case 64: CLUSTEN_ROW_SCORE(16, 1)
        case 128: CLUSTEN_ROW_SCORE(32, 1)
        case 256: CLUSTEN_ROW_SCORE(64, 1)
        case 512: CLUSTEN_ROW_SCORE(64, 2)
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
#undef CLUSTEN_ROW_SCORE
}

template <typename T>
int launch_t(const void* x, int x_dtype, const void* branch, void* sum_out, const void* w, const void* b, void* score,
             int64_t rows, int C, int t_code, hipStream_t stream) {
    if (x_dtype == CLUSTEN_F32) {
        if (branch) return launch_c<float, T, T>(x, branch, sum_out, w, b, score, rows, C, stream);
        return launch_c<float, void, T>(x, nullptr, nullptr, w, b, score, rows, C, stream);
    }
    if (x_dtype == t_code) {
        if (branch) return launch_c<T, T, T>(x, branch, sum_out, w, b, score, rows, C, stream);
        return launch_c<T, void, T>(x, nullptr, nullptr, w, b, score, rows, C, stream);
    }
    return CLUSTEN_ERR_BAD_DTYPE;
}

}  // namespace

int launch_add_row_score(const void* x, int x_dtype, const void* branch, void* sum_out, const void* w, const void* b,
                         void* score, int64_t rows, int C, int dtype, hipStream_t stream) {
    if (dtype == CLUSTEN_F16) return launch_t<f16_t>(x, x_dtype, branch, sum_out, w, b, score, rows, C, CLUSTEN_F16, stream);
    if (dtype == CLUSTEN_BF16) {
        return launch_t<bf16_t>(x, x_dtype, branch, sum_out, w, b, score, rows, C, CLUSTEN_BF16, stream);
    }
    return CLUSTEN_ERR_BAD_DTYPE;
}

}  // namespace clusten
