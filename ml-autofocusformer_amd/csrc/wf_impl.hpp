// WF (adaptive down-sampling) kernels.
//
//   forward   out[b,i,ic,c]  = sum_j w[b,i,j,ic] * feat[b,idx[b,i,j],c]
//             (reference kernel clusten/src/clustenwf_cuda_kernel.cu:18-53)
//   d_weights d_w[b,i,j,ic]  = sum_c feat[b,idx[b,i,j],c] * d_out[b,i,ic,c]
//             (clustenwf_cuda_kernel.cu:137-169)
//   d_feat    d_feat[b,idx[b,i,j],c] += sum_ic d_out[b,i,ic,c] * w[b,i,j,ic]
//             (clustenwf_cuda_kernel.cu:96-135)
//
// Forward: one wave per output token.  The 64 lanes cover 64*VEC consecutive channels with one
// VEC-element access each, so every gathered row is read as one contiguous run, once, for all IC
// inner channels (the reference re-gathers it IC times).  The token's weights w[b,i,:,:] — M*IC
// values shared by all lanes — are loaded so that each row of 16 lanes holds 64 consecutive values
// per register and are read through DPP row broadcasts (see dpp.hpp).  The neighbour list is read
// once per token.  Channel counts that are not a multiple of 64, inner channel counts other than
// 1 and 4, and M*IC not a multiple of 4 take the element-per-thread kernel.
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

template <typename T, int VEC, int IC, int Q, bool GUARD>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4))) void wf_forward_row_kernel(
    const T* __restrict__ w, const T* __restrict__ feat, const int64_t* __restrict__ idx, T* __restrict__ out, int N,
    int Nout, int C, int M, int total_tokens) {
    constexpr int SLOTS = 16 * Q;
    constexpr int NW = (SLOTS * IC + 63) / 64;  // registers that hold one chunk of the token's weights
    static_assert(!GUARD || Q == 4, "guarded lists are taken 64 slots at a time");
    static_assert(IC == 1 || IC == 2 || IC == 4, "inner channels of one slot must stay inside one quad");
    typedef typename Quad<T>::raw QuadRaw;
    typedef typename VecIO<T, VEC>::raw VecRaw;
    constexpr int GS = VEC >= 4 ? 4 : 16 / VEC;  // slots per pipeline group: 16 registers of row data per group

    const int token = xcd_tile(blockIdx.x, total_tokens);
    if (token < 0) return;
    {
    const int b = token / Nout;
    const int lane = threadIdx.x;
    const int rl = lane & 15;

    const int64_t* list_p = idx + (int64_t)token * M;
    const T* w_tok = w + (int64_t)token * M * IC;
    const T* feat_b = feat + (int64_t)b * N * C;
    T* out_tok = out + (int64_t)token * IC * C;

    for (int c0 = 0; c0 < C; c0 += kWave * VEC) {
        const int c = c0 + lane * VEC;
        float acc[IC][VEC];
#pragma unroll
        for (int ic = 0; ic < IC; ++ic) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[ic][v] = 0.f;
        }

        for (int j0 = 0; j0 < M; j0 += kWave) {
            const int mc = min(kWave, M - j0);
            const int list = (int)list_p[j0 + min(lane, mc - 1)];

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

            VecRaw fv[SLOTS];
            slot_pipeline<SLOTS, GS>(
                [&](auto ji) {
                    constexpr int j = decltype(ji)::value;
                    const int row = __builtin_amdgcn_readlane(list, min(j, mc - 1));
                    const T* rowp = feat_b + (int64_t)row * C;  // wave-uniform base, per-lane 32-bit offset
                    fv[j] = *reinterpret_cast<const VecRaw*>(rowp + c);
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

#pragma unroll
        for (int ic = 0; ic < IC; ++ic) {
            *reinterpret_cast<VecRaw*>(out_tok + (int64_t)ic * C + c) = VecIO<T, VEC>::pack(acc[ic]);
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

template <typename T, int VEC, int IC>
int wf_forward_row(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    const int total = s.B * s.Nout;
    if (s.M == 48) {
        const int grid = xcd_grid(total);
        hipLaunchKernelGGL((wf_forward_row_kernel<T, VEC, IC, 3, false>), dim3(grid), dim3(kWave), 0,
                           stream, static_cast<const T*>(w), static_cast<const T*>(feat), idx, static_cast<T*>(out),
                           s.N, s.Nout, s.C, s.M, total);
    } else {
        const int grid = xcd_grid(total);
        hipLaunchKernelGGL((wf_forward_row_kernel<T, VEC, IC, 4, true>), dim3(grid), dim3(kWave), 0, stream,
                           static_cast<const T*>(w), static_cast<const T*>(feat), idx, static_cast<T*>(out), s.N,
                           s.Nout, s.C, s.M, total);
    }
    return launch_status();
}

template <typename T, int IC>
int wf_forward_vec(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    // widest access of at most 16 bytes per lane that tiles the channel count
    if constexpr (sizeof(T) == 2) {
        if (s.C % (kWave * 8) == 0) return wf_forward_row<T, 8, IC>(w, feat, idx, out, s, stream);
    }
    if (s.C % (kWave * 4) == 0) return wf_forward_row<T, 4, IC>(w, feat, idx, out, s, stream);
    if (s.C % (kWave * 2) == 0) return wf_forward_row<T, 2, IC>(w, feat, idx, out, s, stream);
    return wf_forward_row<T, 1, IC>(w, feat, idx, out, s, stream);
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
    const bool rows_ok = s.C % kWave == 0 && aligned16(feat) && aligned16(out);
    const bool quads_ok = (s.M * s.IC) % 4 == 0 && (reinterpret_cast<uintptr_t>(w) % (4 * sizeof(T))) == 0;
    if (rows_ok && quads_ok) {
        if (s.IC == 4) return wf_forward_vec<T, 4>(w, feat, idx, out, s, stream);
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
