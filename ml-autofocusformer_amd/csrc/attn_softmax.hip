// attn_softmax: the arithmetic between the QK and AV operators of local attention, in one pass.
//
//   logits[b,h,i,j] = attn[b,h,i,j] + table[pe_idx[b,i,j], h] - 100 * (1 - mask[b,i,j])      j < M
//   logits[b,h,i,M] = blank[b,h,i]   or   sum_c q[b,h,i,c] * blank_k[h,c]                     (blank token)
//   probs[b,h,i,:M], blank_prob[b,h,i] = softmax(logits[b,h,i,:M+1])
//
// The reference model spells this out as tensor expressions (models/aff_transformer.py:122-147: a gather of the
// position-bias table, two additions, a concatenation, a softmax and two slices), each a full pass over
// (B,H,N,M).  Here a token's M logits are read once and its probabilities written once; pe_idx and mask,
// which the heads share, are read once per token.
//
// LPT = 16 lanes per token (M <= 64) or a whole wave (M <= 256: the 144 neighbours of the 384 x 384 models), 4
// consecutive neighbours per lane (M % 4 == 0); a 256-thread workgroup takes 256 / LPT tokens.  Row maxima and sums
// are reduced inside the LPT-lane rows with xor shuffles.  All arithmetic is fp32.
#include "launch.hpp"

namespace clusten {
namespace {

template <int LPT>
__device__ __forceinline__ float row_max(float v) {
#pragma unroll
    for (int m = 1; m < LPT; m <<= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}
template <int LPT>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
    for (int m = 1; m < LPT; m <<= 1) v += __shfl_xor(v, m);
    return v;
}

template <typename T, int LPT>
__global__ __launch_bounds__(256) void attn_softmax_kernel(const T* __restrict__ attn, const T* __restrict__ table,
                                                           const int64_t* __restrict__ pe_idx,
                                                           const int64_t* __restrict__ mask,
                                                           const float* __restrict__ blank, const T* __restrict__ q,
                                                           clusten_strides qs, const float* __restrict__ blank_k,
                                                           int C, float* __restrict__ probs,
                                                           float* __restrict__ blank_prob, int H, int N, int M,
                                                           int64_t tokens) {
    typedef Quad<T> Q4;
    const int64_t tok_raw = (int64_t)blockIdx.x * (256 / LPT) + threadIdx.x / LPT;
    const bool tok_live = tok_raw < tokens;
    const int64_t tok = tok_live ? tok_raw : tokens - 1;  // every lane stays in the shuffles
    const int sub = threadIdx.x % LPT;
    const int j0 = sub * 4;
    const bool live = j0 < M;
    const int jc = live ? j0 : 0;
    const int64_t b = tok / N;
    const int64_t i = tok - b * N;

    int64_t pe[4];
    float off[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        pe[e] = pe_idx[tok * M + jc + e];
        off[e] = mask ? (float)(1 - mask[tok * M + jc + e]) * -100.f : 0.f;
    }
    for (int h = 0; h < H; ++h) {
        const int64_t row = (b * H + h) * N + i;
        float x[4];
        Q4::unpack(*reinterpret_cast<const typename Q4::raw*>(attn + row * M + jc), x);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[e] = live ? x[e] + (float)to_acc(table[pe[e] * H + h]) + off[e] : -INFINITY;
        }
        float bl;
        if (q) {  // the blank token's logit: this token's query against the blank key of the head
            const T* qrow = q + b * qs.b + h * qs.h + i * qs.n;
            float part = 0.f;
            for (int c = sub; c < C; c += LPT) part += to_acc(qrow[c]) * blank_k[h * C + c];
            bl = row_sum<LPT>(part);
        } else {
            bl = blank[row];
        }
        const float mx = fmaxf(row_max<LPT>(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]))), bl);
        float ex[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) ex[e] = live ? expf(v[e] - mx) : 0.f;
        const float eb = expf(bl - mx);
        const float inv = 1.f / (row_sum<LPT>((ex[0] + ex[1]) + (ex[2] + ex[3])) + eb);
        if (tok_live && live) {
            float4 o = make_float4(ex[0] * inv, ex[1] * inv, ex[2] * inv, ex[3] * inv);
            *reinterpret_cast<float4*>(probs + row * M + j0) = o;
        }
        if (tok_live && sub == 0) blank_prob[row] = eb * inv;
    }
}

template <typename T>
int launch_typed(const void* attn, const void* table, const int64_t* pe_idx, const int64_t* mask, const float* blank,
                 const void* q, clusten_strides qs, const float* blank_k, float* probs, float* blank_prob,
                 const clusten_attn_shape& s, hipStream_t stream) {
    const int64_t tokens = (int64_t)s.B * s.N;
    if (s.M <= 64) {
        hipLaunchKernelGGL((attn_softmax_kernel<T, 16>), dim3((unsigned)((tokens + 15) / 16)), dim3(256), 0, stream,
                           static_cast<const T*>(attn), static_cast<const T*>(table), pe_idx, mask, blank,
                           static_cast<const T*>(q), qs, blank_k, s.C, probs, blank_prob, s.H, s.N, s.M, tokens);
    } else {
        hipLaunchKernelGGL((attn_softmax_kernel<T, 64>), dim3((unsigned)((tokens + 3) / 4)), dim3(256), 0, stream,
                           static_cast<const T*>(attn), static_cast<const T*>(table), pe_idx, mask, blank,
                           static_cast<const T*>(q), qs, blank_k, s.C, probs, blank_prob, s.H, s.N, s.M, tokens);
    }
    return launch_status();
}

}  // namespace

int launch_attn_softmax(const void* attn, const void* table, const int64_t* pe_idx, const int64_t* mask,
                        const float* blank, const void* q, clusten_strides qs, const float* blank_k, float* probs,
                        float* blank_prob, clusten_attn_shape s, int dtype, hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return launch_typed<float>(attn, table, pe_idx, mask, blank, q, qs, blank_k, probs, blank_prob, s, stream);
        case CLUSTEN_F16: return launch_typed<f16_t>(attn, table, pe_idx, mask, blank, q, qs, blank_k, probs, blank_prob, s, stream);
        case CLUSTEN_BF16: return launch_typed<bf16_t>(attn, table, pe_idx, mask, blank, q, qs, blank_k, probs, blank_prob, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

// Backward of the softmax over the M neighbours and the blank token:
//   s = sum_j p_j dp_j + p_blank dp_blank;   d_logit_j = p_j (dp_j - s);   d_blank_logit = p_blank (dp_blank - s)
// (the bias, the mask and the logits enter the softmax as a sum, so d_logit is the gradient of each of them).
// One row per 16 lanes (M <= 64) or per wave (M <= 256), four consecutive neighbours per lane; probs, d_probs fp32,
// d_logit of the logits' type.
namespace {

template <typename T, int LPT>
__global__ __launch_bounds__(256) void attn_softmax_backward_kernel(const float* __restrict__ probs,
                                                                    const float* __restrict__ blank_prob,
                                                                    const float* __restrict__ d_probs,
                                                                    const float* __restrict__ d_blank_prob,
                                                                    T* __restrict__ d_logit, float* __restrict__ d_blank_logit,
                                                                    int64_t rows, int M) {
    const int sub = threadIdx.x % LPT;
    const int64_t row_raw = (int64_t)blockIdx.x * (256 / LPT) + threadIdx.x / LPT;
    const bool live = row_raw < rows;
    const int64_t row = live ? row_raw : rows - 1;  // every lane stays in the shuffles
    const bool mine = 4 * sub < M;
    float4 p = make_float4(0.f, 0.f, 0.f, 0.f), dp = p;
    if (mine) {
        p = *reinterpret_cast<const float4*>(probs + row * M + 4 * sub);
        dp = *reinterpret_cast<const float4*>(d_probs + row * M + 4 * sub);
    }
    const float pb = blank_prob[row], dpb = d_blank_prob[row];
    float s = (p.x * dp.x + p.y * dp.y) + (p.z * dp.z + p.w * dp.w);
    s = row_sum<LPT>(s);
    s += pb * dpb;
    if (!live) return;
    if (mine) {
        float v[4] = {p.x * (dp.x - s), p.y * (dp.y - s), p.z * (dp.z - s), p.w * (dp.w - s)};
        *reinterpret_cast<typename Quad<T>::raw*>(d_logit + row * M + 4 * sub) = Quad<T>::pack(v);
    }
    if (sub == 0) d_blank_logit[row] = pb * (dpb - s);
}

}  // namespace

int launch_attn_softmax_backward(const float* probs, const float* blank_prob, const float* d_probs,
                                 const float* d_blank_prob, void* d_logit, float* d_blank_logit, int64_t rows, int M,
                                 int dtype, hipStream_t stream) {
    auto launch = [&](auto tag) {
        typedef decltype(tag) T;
        if (M <= 64) {
            hipLaunchKernelGGL((attn_softmax_backward_kernel<T, 16>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream,
                               probs, blank_prob, d_probs, d_blank_prob, static_cast<T*>(d_logit), d_blank_logit, rows, M);
        } else {
            hipLaunchKernelGGL((attn_softmax_backward_kernel<T, 64>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream,
                               probs, blank_prob, d_probs, d_blank_prob, static_cast<T*>(d_logit), d_blank_logit, rows, M);
        }
    };
    switch (dtype) {
        case CLUSTEN_F32: launch(float()); break;
        case CLUSTEN_F16: launch(f16_t()); break;
        case CLUSTEN_BF16: launch(bf16_t()); break;
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace clusten
