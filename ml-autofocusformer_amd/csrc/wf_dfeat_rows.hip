// wf_dfeat_rows: the feature gradient of the WF operator for any neighbour list, as a gather (no atomics).
//
//   d_feat[b, idx[b,i,j], c] += sum_ic d_out[b,i,ic,c] * w[b,i,j,ic]          (clusten/src/clustenwf_cuda_kernel.cu:96-135)
//
// The reference issues one atomic per (i, j, c); its sums arrive in whatever order the hardware serves them.  Here
// the list entries (i, j) of every image are sorted by the row they name (cluster_pairs.hip: a stable counting sort on
// the device, entries of a row in ascending order), and one wave per destination row walks its entries:
//
//   d_feat[b, n, :] = sum over the entries (i, j) with idx[b,i,j] = n, in ascending (i, j), of
//                     sum_ic w[b,i,j,ic] * d_out[b,i,ic,:]
//
// lane (ic, c4) takes four channels of inner channel ic of the entry's output token (the four rows of an entry are one
// contiguous piece of d_out), four entries are requested together, and the inner channels are added up across the
// lanes at the end.  Every row is written exactly once from an fp32 sum in a fixed order: no atomics, no zero-fill, no
// fp32 workspace for 16-bit data, results that repeat bit for bit.  Lists made of whole clusters have a faster kernel
// (wf_dfeat_by_cluster.hip); this one takes all the others.  It has no counterpart in the reference's extension modules.
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

template <typename T>
__global__ __launch_bounds__(kWave) void wf_dfeat_rows_kernel(const T* __restrict__ d_out, const T* __restrict__ w,
                                                              const int32_t* __restrict__ starts,
                                                              const int32_t* __restrict__ ends,
                                                              const int32_t* __restrict__ entries,
                                                              const int32_t* __restrict__ only_if, T* __restrict__ d_feat,
                                                              int N, int Nout, int C, int M, int IC, int total_rows) {
    typedef VecIO<T, 4> Quad4;
    const int row = xcd_tile(blockIdx.x, total_rows);
    if (row < 0) return;
    // the flag and the bounds of the row's entries are requested together (one trip to memory, not two); the bounds
    // mean nothing when the other kernel has the lists, and are not used then
    const int wanted = only_if != nullptr ? *only_if : 1;
    const int first = starts[row];
    const int last = ends[row];
    if (wanted == 0) return;   // lists made of whole clusters: the other kernel has them
    const int b = row / N;
    const int lane = threadIdx.x;
    const int ic = lane >> 4, c4 = lane & 15;
    const bool ic_ok = ic < IC;
    const int count = last - first;
    const T* d_out_b = d_out + (int64_t)b * Nout * IC * C;
    const T* w_b = w + (int64_t)b * Nout * M * IC;
    T* dst = d_feat + (int64_t)row * C;
    constexpr int GS = 8;   // entries requested together
    for (int c0 = 0; c0 < C; c0 += 64) {
        const int c = c0 + 4 * c4;
        const bool live = ic_ok && c < C;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int e0 = 0; e0 < count; e0 += GS) {
            typename Quad4::raw raw[GS];
            float wv[GS];
#pragma unroll
            for (int u = 0; u < GS; ++u) {
                const int e = entries[first + min(e0 + u, count - 1)];      // the same for every lane: i * M + j
                const int i = e / M;
                raw[u] = typename Quad4::raw(0);
                wv[u] = 0.f;
                if (live && e0 + u < count) {
                    raw[u] = *reinterpret_cast<const typename Quad4::raw*>(d_out_b + ((int64_t)i * IC + ic) * C + c);
                    wv[u] = to_acc(w_b[(int64_t)e * IC + ic]);
                }
            }
#pragma unroll
            for (int u = 0; u < GS; ++u) {
                float x[4];
                Quad4::unpack(raw[u], x);
#pragma unroll
                for (int k = 0; k < 4; ++k) acc[k] += wv[u] * x[k];
            }
        }
        // the four inner channels sit in the four rows of 16 lanes: add them up (in the order ic = 0, 1, 2, 3)
        float total[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float a0 = __shfl(acc[k], c4), a1 = __shfl(acc[k], 16 + c4), a2 = __shfl(acc[k], 32 + c4),
                        a3 = __shfl(acc[k], 48 + c4);
            total[k] = ((a0 + a1) + a2) + a3;
        }
        if (ic == 0 && c < C) *reinterpret_cast<typename Quad4::raw*>(dst + c) = Quad4::pack(total);
    }
}

template <typename T>
int launch_typed(const void* d_out, const void* w, const int32_t* starts, const int32_t* ends, const int32_t* entries,
                 const int32_t* only_if, void* d_feat, const clusten_wf_shape& s, hipStream_t stream) {
    const int64_t total = (int64_t)s.B * s.N;
    if (total >= ((int64_t)1 << 30)) return CLUSTEN_ERR_BAD_DIMS;
    hipLaunchKernelGGL((wf_dfeat_rows_kernel<T>), dim3(xcd_grid((int)total)), dim3(kWave), 0, stream,
                       static_cast<const T*>(d_out), static_cast<const T*>(w), starts, ends, entries, only_if,
                       static_cast<T*>(d_feat), s.N, s.Nout, s.C, s.M, s.IC, (int)total);
    return launch_status();
}

}  // namespace

bool wf_dfeat_rows_supported(const void* d_out, const void* d_feat, const clusten_wf_shape& s, int dtype) {
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return false;
    if (s.IC > 4 || s.C % 4 != 0) return false;
    const size_t eb = dtype_size(dtype);
    const bool quads = dtype == CLUSTEN_F32 ? (aligned16(d_out) && aligned16(d_feat))
                                            : ((reinterpret_cast<uintptr_t>(d_out) & 7u) == 0 &&
                                               (reinterpret_cast<uintptr_t>(d_feat) & 7u) == 0);
    return quads && (int64_t)s.Nout * s.M * s.IC < ((int64_t)1 << 31) && (int64_t)s.Nout * s.IC * s.C * (int64_t)eb < ((int64_t)1 << 40);
}

int launch_wf_dfeat_rows(const void* d_out, const void* w, const int32_t* starts, const int32_t* ends,
                         const int32_t* entries, const int32_t* only_if, void* d_feat, clusten_wf_shape s, int dtype,
                         hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return launch_typed<float>(d_out, w, starts, ends, entries, only_if, d_feat, s, stream);
        case CLUSTEN_F16: return launch_typed<f16_t>(d_out, w, starts, ends, entries, only_if, d_feat, s, stream);
        case CLUSTEN_BF16: return launch_typed<bf16_t>(d_out, w, starts, ends, entries, only_if, d_feat, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
