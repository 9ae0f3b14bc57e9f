// WF (adaptive down-sampling) kernels.
//
//   forward   out[b,i,ic,c]  = sum_j w[b,i,j,ic] * feat[b,idx[b,i,j],c]
//             (reference kernel clusten/src/clustenwf_cuda_kernel.cu:18-53)
//   d_weights d_w[b,i,j,ic]  = sum_c feat[b,idx[b,i,j],c] * d_out[b,i,ic,c]
//             (clustenwf_cuda_kernel.cu:137-169)
//   d_feat    d_feat[b,idx[b,i,j],c] += sum_ic d_out[b,i,ic,c] * w[b,i,j,ic]
//             (clustenwf_cuda_kernel.cu:96-135)
//
// Forward.  A gathered feature row is C*sizeof(T) bytes; LPT = that / 16 lanes cover it with one
// 16-byte access each, so a wave serves 64/LPT output tokens at once (4 tokens of 64 fp32 channels)
// and every gather instruction moves whole rows, 1 KiB per wave access.  Each row is read once for
// all IC inner channels (the reference re-gathers it IC times).  What the lanes of one token share —
// the token's weights w[b,i,:,:] and its neighbour list — is held spread over the rows of 16 lanes
// that belong to the token and read through DPP row broadcasts (see dpp.hpp): no LDS, no scalar
// loads.  Rows wider than 64 lanes are taken in 1 KiB column blocks.
// Rows that are not a multiple of 256 bytes, inner channel counts other than 1, 2 and 4, and M*IC
// not a multiple of 4 take the element-per-thread kernel.
//
// Backward: plain kernels (one thread per d_w element; one wave-row per token for d_feat with one
// fp32 atomic per (slot, channel)).
//
// This header holds the templates; wf_{f32,f16,bf16}.hip instantiate them per storage type so that
// the translation units build in parallel, wf.hip holds the dtype dispatch.
#pragma once

#include "dpp.hpp"
#include "launch.hpp"

namespace clusten {

// LPT = lanes per token (16, 32 or 64).  GUARD = false: the list has exactly 16*Q slots;
// GUARD = true: any length, taken 64 slots at a time (Q = 4) with every slot range-checked.
template <typename T, int LPT, int IC, int Q, bool GUARD>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4))) void wf_forward_row_kernel(
    const T* __restrict__ w, const T* __restrict__ feat, const int64_t* __restrict__ idx, T* __restrict__ out, int N,
    int Nout, int C, int M, int total_tokens, int total_groups) {
    constexpr int TPW = kWave / LPT;               // output tokens per wave
    constexpr int VEC = 16 / (int)sizeof(T);       // channels per lane and column block
    constexpr int SLOTS = 16 * Q;
    constexpr int NW = (SLOTS * IC + 63) / 64;     // registers that hold one chunk of a token's weights
    constexpr int NL = Q;                          // registers that hold one chunk of a token's list
    constexpr int GS = 4;                          // gather accesses per pipeline group (two groups in flight)
    static_assert(LPT == 16 || LPT == 32 || LPT == 64, "a row of 16 lanes must belong to one token");
    static_assert(!GUARD || Q == 4, "guarded lists are taken 64 slots at a time");
    static_assert(IC == 1 || IC == 2 || IC == 4, "inner channels of one slot must stay inside one quad");
    typedef typename Quad<T>::raw QuadRaw;

    const int group = xcd_tile(blockIdx.x, total_groups);
    if (group < 0) return;
    const int lane = threadIdx.x;
    const int rl = lane & 15;
    // the lane's token (waves past the end repeat the last token; their stores are masked)
    const int token_raw = group * TPW + lane / LPT;
    const bool token_ok = token_raw < total_tokens;
    const int token = min(token_raw, total_tokens - 1);
    const int b = token / Nout;
    const int col = (lane % LPT) * VEC;  // first channel of the lane inside a column block

    const int64_t* list_p = idx + (int64_t)token * M;
    const T* w_tok = w + (int64_t)token * M * IC;
    const char* feat_b = reinterpret_cast<const char*>(feat + (int64_t)b * N * C);
    T* out_tok = out + (int64_t)token * IC * C;
    const uint32_t row_bytes = (uint32_t)C * sizeof(T);

    for (int c0 = 0; c0 < C; c0 += LPT * VEC) {
        float acc[IC][VEC];
#pragma unroll
        for (int ic = 0; ic < IC; ++ic) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[ic][v] = 0.f;
        }
        const uint32_t lane_bytes = (uint32_t)(c0 + col) * sizeof(T);

        for (int j0 = 0; j0 < M; j0 += kWave) {
            const int mc = min(kWave, M - j0);

            // list: slot 16*k + rl of the token in register k of its row(s) of 16 lanes
            int lst[NL];
#pragma unroll
            for (int k = 0; k < NL; ++k) lst[k] = (int)list_p[j0 + min(16 * k + rl, mc - 1)];
            // weights: flat element f = j*IC + ic of the chunk sits in register f/64 of row-lane (f%64)/4, element f%4
            float wv[NW][4];
            {
                QuadRaw raw[NW];
#pragma unroll
                for (int m = 0; m < NW; ++m) {
                    const int f0 = min(64 * m + 4 * rl, mc * IC - 4);
                    raw[m] = *reinterpret_cast<const QuadRaw*>(w_tok + (int64_t)j0 * IC + f0);
                }
#pragma unroll
                for (int m = 0; m < NW; ++m) Quad<T>::unpack(raw[m], wv[m]);
            }

            Piece fv[SLOTS];
            slot_pipeline<SLOTS, GS>(
                [&](auto ji) {
                    constexpr int j = decltype(ji)::value;
                    // row index of slot j: lane j % 16 of list register j / 16, broadcast inside each row of 16
                    const int row = rowlane_bcast<j % 16>(lst[j / 16]);
                    const uint32_t off = (uint32_t)((GUARD && j >= mc) ? 0 : row) * row_bytes + lane_bytes;
                    fv[j] = *reinterpret_cast<const Piece*>(feat_b + off);
                },
                [&](auto ji) {
                    constexpr int j = decltype(ji)::value;
                    if (!GUARD || j < mc) {
                        float x[VEC];
                        VecIO<T, VEC>::unpack(fv[j], x);
                        static_for<0, IC>([&](auto ici) {
                            constexpr int ic = decltype(ici)::value;
                            constexpr int f = j * IC + ic;
                            fma_vec_rowlane<(f % 64) / 4, VEC>(acc[ic], wv[f / 64][f % 4], x);
                        });
                    }
                });
        }

        if (token_ok) {
#pragma unroll
            for (int ic = 0; ic < IC; ++ic) {
                *reinterpret_cast<Piece*>(out_tok + (int64_t)ic * C + c0 + col) = VecIO<T, VEC>::pack(acc[ic]);
            }
        }
    }
}

// One thread per output element; any dtype and shape.
template <typename T>
__global__ __launch_bounds__(256) void wf_forward_elem_kernel(const T* __restrict__ w, const T* __restrict__ feat,
                                                              const int64_t* __restrict__ idx, T* __restrict__ out,
                                                              int B, int N, int Nout, int C, int M, int IC) {
    const int64_t total = (int64_t)B * Nout * IC * C;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(o % C);
        const int64_t q1 = o / C;
        const int ic = (int)(q1 % IC);
        const int64_t token = q1 / IC;  // b*Nout + i
        const int b = (int)(token / Nout);
        const int64_t* list = idx + token * M;
        const T* wrow = w + token * M * IC + ic;
        const T* base = feat + (int64_t)b * N * C + c;
        typename Acc<T>::type acc = 0;
        for (int j = 0; j < M; ++j) acc += to_acc(wrow[(int64_t)j * IC]) * to_acc(base[list[j] * C]);
        out[o] = from_acc<T>(acc);
    }
}

// d_w: one thread per (b,i,j,ic) element, a serial dot product over the C channels.
template <typename T>
__global__ __launch_bounds__(256) void wf_dweights_kernel(const T* __restrict__ d_out, const T* __restrict__ feat,
                                                          const int64_t* __restrict__ idx, T* __restrict__ d_w, int B,
                                                          int N, int Nout, int C, int M, int IC) {
    const int64_t total = (int64_t)B * Nout * M * IC;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
        const int ic = (int)(o % IC);
        const int64_t q1 = o / IC;  // token*M + j
        const int64_t token = q1 / M;
        const int b = (int)(token / Nout);
        const T* frow = feat + ((int64_t)b * N + idx[q1]) * C;
        const T* grow = d_out + (token * IC + ic) * C;
        typename Acc<T>::type acc = 0;
        for (int c = 0; c < C; ++c) acc += to_acc(frow[c]) * to_acc(grow[c]);
        d_w[o] = from_acc<T>(acc);
    }
}

// d_feat: one workgroup per output token, threads over channels; per slot the IC products are
// summed in registers and leave as one atomic per channel onto a contiguous destination row.
template <typename T, typename A>
__global__ __launch_bounds__(256) void wf_dfeat_kernel(const T* __restrict__ d_out, const T* __restrict__ w,
                                                       const int64_t* __restrict__ idx, A* __restrict__ d_feat, int N,
                                                       int Nout, int C, int M, int IC, int total_tokens) {
    const int token = xcd_tile(blockIdx.x, total_tokens);
    if (token < 0) return;
    {
    const int b = token / Nout;
    const int64_t* list = idx + (int64_t)token * M;
    const T* wtok = w + (int64_t)token * M * IC;
    const T* gtok = d_out + (int64_t)token * IC * C;
    A* dst_b = d_feat + (int64_t)b * N * C;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        for (int j = 0; j < M; ++j) {
            A sum = 0;
            for (int ic = 0; ic < IC; ++ic) sum += (A)to_acc(gtok[(int64_t)ic * C + c]) * (A)to_acc(wtok[j * IC + ic]);
            unsafeAtomicAdd(dst_b + list[j] * C + c, sum);
        }
    }
    }
}

inline int elem_grid(int64_t total) {
    const int64_t want = (total + 255) / 256;
    return (int)(want < (int64_t)1 << 20 ? want : (int64_t)1 << 20);
}

template <typename T, int LPT, int IC>
int wf_forward_row(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    const int total = s.B * s.Nout;
    const int groups = (total + kWave / LPT - 1) / (kWave / LPT);
    if (s.M == 48) {
        hipLaunchKernelGGL((wf_forward_row_kernel<T, LPT, IC, 3, false>), dim3(xcd_grid(groups)), dim3(kWave), 0,
                           stream, static_cast<const T*>(w), static_cast<const T*>(feat), idx, static_cast<T*>(out),
                           s.N, s.Nout, s.C, s.M, total, groups);
    } else {
        hipLaunchKernelGGL((wf_forward_row_kernel<T, LPT, IC, 4, true>), dim3(xcd_grid(groups)), dim3(kWave), 0,
                           stream, static_cast<const T*>(w), static_cast<const T*>(feat), idx, static_cast<T*>(out),
                           s.N, s.Nout, s.C, s.M, total, groups);
    }
    return launch_status();
}

template <typename T, int IC>
int wf_forward_vec(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    // lanes per token: the widest of 64, 32, 16 whose 16-byte accesses tile the row
    const int row_bytes = s.C * (int)sizeof(T);
    if (row_bytes % 1024 == 0) return wf_forward_row<T, 64, IC>(w, feat, idx, out, s, stream);
    if (row_bytes % 512 == 0) return wf_forward_row<T, 32, IC>(w, feat, idx, out, s, stream);
    return wf_forward_row<T, 16, IC>(w, feat, idx, out, s, stream);
}

template <typename T>
int wf_forward_elem(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                    hipStream_t stream) {
    const int64_t total = (int64_t)s.B * s.Nout * s.IC * s.C;
    hipLaunchKernelGGL((wf_forward_elem_kernel<T>), dim3(elem_grid(total)), dim3(256), 0, stream,
                       static_cast<const T*>(w), static_cast<const T*>(feat), idx, static_cast<T*>(out), s.B, s.N,
                       s.Nout, s.C, s.M, s.IC);
    return launch_status();
}

template <typename T>
int wf_forward_typed(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                     hipStream_t stream) {
    // whole 256-byte rows, and 32-bit byte offsets inside one batch element of feat
    const bool rows_ok = (s.C * (int)sizeof(T)) % 256 == 0 && aligned16(feat) && aligned16(out) &&
                         (int64_t)s.N * s.C * (int64_t)sizeof(T) < ((int64_t)1 << 31);
    const bool quads_ok = (s.M * s.IC) % 4 == 0 && (reinterpret_cast<uintptr_t>(w) % (4 * sizeof(T))) == 0;
    if (rows_ok && quads_ok) {
        if (s.IC == 4) return wf_forward_vec<T, 4>(w, feat, idx, out, s, stream);
        if (s.IC == 2) return wf_forward_vec<T, 2>(w, feat, idx, out, s, stream);
        if (s.IC == 1) return wf_forward_vec<T, 1>(w, feat, idx, out, s, stream);
    }
    return wf_forward_elem<T>(w, feat, idx, out, s, stream);
}

template <typename T>
int wf_dweights_typed(const void* d_out, const void* feat, const int64_t* idx, void* d_w, const clusten_wf_shape& s,
                      hipStream_t stream) {
    const int64_t total = (int64_t)s.B * s.Nout * s.M * s.IC;
    hipLaunchKernelGGL((wf_dweights_kernel<T>), dim3(elem_grid(total)), dim3(256), 0, stream,
                       static_cast<const T*>(d_out), static_cast<const T*>(feat), idx, static_cast<T*>(d_w), s.B, s.N,
                       s.Nout, s.C, s.M, s.IC);
    return launch_status();
}

template <typename T, typename A>
int wf_dfeat_typed(const void* d_out, const void* w, const int64_t* idx, A* acc, const clusten_wf_shape& s,
                   hipStream_t stream) {
    const int total = s.B * s.Nout;
    const int threads = s.C >= 256 ? 256 : (s.C > 64 ? 128 : 64);
    hipLaunchKernelGGL((wf_dfeat_kernel<T, A>), dim3(xcd_grid(total)), dim3(threads), 0, stream,
                       static_cast<const T*>(d_out), static_cast<const T*>(w), idx, acc, s.N, s.Nout, s.C, s.M, s.IC,
                       total);
    return launch_status();
}

}  // namespace clusten
