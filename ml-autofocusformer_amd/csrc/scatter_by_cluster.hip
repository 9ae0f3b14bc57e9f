// scatter_by_cluster: the scatter of the attention backward passes, turned into a gather (no atomics).
//
//   y[b,h, idx[b,i,j], :] += p[b,h,i,j] * x[b,h,i,:]          (d_key with p = d_attn, x = query;
//                                                              d_value with p = attn, x = d_out:
//                                                              clusten/src/clustenqk_cuda_kernel.cu:96-133,
//                                                              clustenav_cuda_kernel.cu:96-131)
//
// for neighbour lists made of whole clusters: idx[b,i,8r+t] = 8 c(b,i,r) + t, the lists the reference model
// builds (models/aff_transformer.py:476-480).  Then the 8 rows of cluster g receive
//
//   y[b,h, 8g + t, :] = sum over the pairs (i, r) with c(b,i,r) = g of  p[b,h,i,8r+t] * x[b,h,i,:]
//
// and, with the pairs of every cluster listed once (cluster_pairs.hip: a counting sort of the cluster numbers on the
// device, shared by the heads), each cluster is an independent small matrix product
// Y_g (8 x C) = P_g^T (8 x pairs) X_g (pairs x C): one wave per cluster walks the heads, the x rows and the 8-element
// pieces of p of 32 pairs at a time travel to LDS by LDS-direct loads, and the product runs on
// `v_mfma_f32_16x16x4_f32` (16-bit data is widened when the operands are read from LDS; rows 8-15 of the instruction
// are idle).  Every row of y is written exactly once, from fp32 sums over all its pairs: no atomics, no zero-fill, no
// fp32 workspace for 16-bit data, and the sums do not depend on the order in which workgroups run.
// A sequence whose length is not a multiple of 8 ends in a short cluster, and the lists that name it hold row 0 in
// the slots past its rows (models/point_utils.py pads member lists with index 0): those slots add to row 0, so
// such a pair is listed a second time, flagged, under cluster 0, where the sum of its pad slots feeds row 0.
// It has no counterpart in the reference's extension modules.
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kPass = 32;        // pairs per pass
constexpr int kListMax = 256;    // pairs of a cluster held in LDS at a time
constexpr int kPadEntry = 1 << 30;   // list entry flag: the pair names the short last cluster; here, for its pad slots
constexpr int kEntryMask = kPadEntry - 1;

template <typename T, int C>
__global__ __launch_bounds__(kWave) void scatter_by_cluster_kernel(const T* __restrict__ p, const T* __restrict__ x,
                                                                   clusten_strides xs, const int32_t* __restrict__ starts,
                                                                   const int32_t* __restrict__ ends,
                                                                   const int32_t* __restrict__ pairs,
                                                                   const int32_t* __restrict__ not_whole, T* __restrict__ y,
                                                                   int H, int N, int M, int clusters_per_image,
                                                                   int total_clusters) {
    constexpr int EB = (int)sizeof(T);
    constexpr int ROW_B = C * EB;                    // bytes of an x row
    constexpr int PIECE_B = 8 * EB;                  // bytes of the 8 elements of p a pair contributes
    constexpr int X_BYTES = kPass * ROW_B;
    constexpr int X_DMA = X_BYTES / 1024;            // LDS-direct loads per pass for the x rows
    constexpr int ROWS_PER_DMA = 1024 / ROW_B;
    constexpr int LANES_PER_ROW = ROW_B / 16;
    constexpr int CB = C / 16;                       // 16-channel blocks of a row
    constexpr int X_BASE = 0;
    constexpr int P_BASE = X_BASE + X_BYTES;
    constexpr int O_BASE = P_BASE + 1024;
    constexpr int L_BASE = O_BASE + 8 * C * 4;
    constexpr int LDS_BYTES = L_BASE + kListMax * 4;
    static_assert(X_BYTES % 1024 == 0 && 1024 % ROW_B == 0, "whole LDS-direct loads, whole rows per load");
    __shared__ __attribute__((aligned(1024))) char stage[LDS_BYTES];

    const int unit = xcd_tile(blockIdx.x, total_clusters);
    if (unit < 0) return;
    // the flag and the bounds of the cluster's list are requested together (one trip to memory, not two); the bounds
    // mean nothing when the flag is set, and are not used then
    const int flagged = not_whole != nullptr ? *not_whole : 0;
    const int first = starts[unit];
    const int last = ends[unit];
    if (flagged != 0) return;   // not lists of whole clusters: the atomic kernels run instead
    const int b = unit / clusters_per_image;
    const int g = unit - b * clusters_per_image;
    const int lane = threadIdx.x;
    const int r16 = lane & 15, kq = lane >> 4;
    const int count = last - first;
    int* list = reinterpret_cast<int*>(stage + L_BASE);
    const int rows_here = min(8, N - 8 * g);   // the last cluster of a sequence may be short
    const int pad_from = N & 7;                // ... and the lists that name it hold row 0 in slots pad_from .. 7

    // a cluster listed by more than kListMax pairs is taken in segments, every head walking all of them before it
    // writes its rows; the usual cluster's list is read once for all heads
    const bool one_segment = count <= kListMax;
    if (one_segment) {
        for (int e = lane; e < count; e += kWave) list[e] = pairs[first + e];
    }
    for (int h = 0; h < H; ++h) {
        const char* x_bh = reinterpret_cast<const char*>(x + (int64_t)b * xs.b + (int64_t)h * xs.h);
        const char* p_bh = reinterpret_cast<const char*>(p + ((int64_t)b * H + h) * N * M);
        F32x4 acc[CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[cb] = F32x4{0.f, 0.f, 0.f, 0.f};
        for (int seg = 0; seg < count; seg += kListMax) {
            const int n = min(kListMax, count - seg);
            if (!one_segment) {
                lds_sync();
                for (int e = lane; e < n; e += kWave) list[e] = pairs[first + seg + e];
            }
            for (int base = 0; base < n; base += kPass) {
                const int here = min(kPass, n - base);
                lds_sync();  // the previous pass has been read (and the list is in place)
#pragma unroll
                for (int a = 0; a < X_DMA; ++a) {
                    const int e = list[base + min(ROWS_PER_DMA * a + lane / LANES_PER_ROW, here - 1)] & kEntryMask;
                    CLUSTEN_LDS_DMA16(x_bh + lane_offset((uint32_t)(e >> kPairRunBits) * (uint32_t)xs.n * EB +
                                                         (uint32_t)(lane % LANES_PER_ROW) * 16),
                                      stage + X_BASE + a * 1024);
                }
                {
                    // 32 pieces of PIECE_B bytes: 16 bytes per lane
                    constexpr int LANES_PER_PIECE = PIECE_B / 16;
                    if (lane < kPass * LANES_PER_PIECE) {
                        const int e = list[base + min(lane / LANES_PER_PIECE, here - 1)] & kEntryMask;
                        CLUSTEN_LDS_DMA16(p_bh + lane_offset(((uint32_t)(e >> kPairRunBits) * (uint32_t)M + (uint32_t)(e & kPairRunMask) * 8) * EB +
                                                             (uint32_t)(lane % LANES_PER_PIECE) * 16),
                                          stage + P_BASE);
                    }
                }
                lds_sync_vm<0>();
#pragma unroll
                for (int s = 0; s < kPass / 4; ++s) {
                    if (4 * s < here) {
                        const int pr = 4 * s + kq;
                        const T* pp = reinterpret_cast<const T*>(stage + P_BASE + pr * PIECE_B);
                        float a = 0.f;
                        if (pr < here) {
                            if ((list[base + pr] & kPadEntry) == 0) {
                                if (r16 < rows_here) a = to_acc(pp[r16]);
                            } else if (r16 == 0) {
                                // a pair that names the short last cluster: its pad slots hold row 0, this cluster's first
                                for (int t = pad_from; t < 8; ++t) a += to_acc(pp[t]);
                            }
                        }
                        const T* xp = reinterpret_cast<const T*>(stage + X_BASE + pr * ROW_B) + r16;
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb) {
                            acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, to_acc(xp[16 * cb]), acc[cb], 0, 0, 0);
                        }
                    }
                }
            }
        }
        // rows 4*kq + j of the result (kq < 2: the cluster's 8 rows), channels 16*cb + r16
        T* y_rows = y + (((int64_t)b * H + h) * N + (int64_t)g * 8) * C;
        lds_sync();
        if (kq < 2) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    reinterpret_cast<float*>(stage + O_BASE)[(4 * kq + j) * C + 16 * cb + r16] = acc[cb][j];
                }
            }
        }
        lds_sync();
        // 8 rows x C channels, four consecutive channels per lane: 8*C/4 quads
#pragma unroll
        for (int q0 = 0; q0 < 8 * C / 4; q0 += kWave) {
            const int q = q0 + lane;
            if (q < 8 * C / 4 && q / (C / 4) < rows_here) {
                const F32x4 o = *reinterpret_cast<const F32x4*>(stage + O_BASE + q * 16);
                const float v[4] = {o[0], o[1], o[2], o[3]};
                *reinterpret_cast<typename Quad<T>::raw*>(y_rows + q * 4) = Quad<T>::pack(v);
            }
        }
    }
}

template <typename T, int C>
int launch_typed_c(const void* p, const void* x, clusten_strides xs, const int32_t* starts, const int32_t* ends,
                   const int32_t* pairs, const int32_t* not_whole, void* y, const clusten_attn_shape& s,
                   hipStream_t stream) {
    const int per_image = (s.N + 7) / 8;
    const int64_t total = (int64_t)s.B * per_image;
    if (total >= ((int64_t)1 << 30)) return CLUSTEN_ERR_BAD_DIMS;
    hipLaunchKernelGGL((scatter_by_cluster_kernel<T, C>), dim3(xcd_grid((int)total)), dim3(kWave), 0, stream,
                       static_cast<const T*>(p), static_cast<const T*>(x), xs, starts, ends, pairs, not_whole,
                       static_cast<T*>(y), s.H, s.N, s.M, per_image, (int)total);
    return launch_status();
}

template <typename T>
int launch_typed(const void* p, const void* x, clusten_strides xs, const int32_t* starts, const int32_t* ends,
                 const int32_t* pairs, const int32_t* not_whole, void* y, const clusten_attn_shape& s,
                 hipStream_t stream) {
    switch (s.C) {
        case 16: return launch_typed_c<T, 16>(p, x, xs, starts, ends, pairs, not_whole, y, s, stream);
        case 32: return launch_typed_c<T, 32>(p, x, xs, starts, ends, pairs, not_whole, y, s, stream);
        case 64: return launch_typed_c<T, 64>(p, x, xs, starts, ends, pairs, not_whole, y, s, stream);
        default: return CLUSTEN_ERR_BAD_DIMS;
    }
}

}  // namespace

bool scatter_by_cluster_supported(const void* p, const void* x, clusten_strides xs, const void* y,
                                  const clusten_attn_shape& s, int dtype) {
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return false;
    if ((s.C != 16 && s.C != 32 && s.C != 64) || s.N < 8 || s.M % 8 != 0 || s.M > kPairMaxSlots || s.M <= 0) return false;
    const size_t eb = dtype_size(dtype);
    return rows_aligned16(x, xs, (int)eb) && aligned16(p) && aligned16(y) && slice_fits_int32(xs, s.H, s.N, s.C) &&
           (int64_t)s.N * s.M * (int64_t)eb < ((int64_t)1 << 31);
}

int launch_scatter_by_cluster(const void* p, const void* x, clusten_strides xs, const int32_t* starts, const int32_t* ends,
                              const int32_t* pairs, const int32_t* not_whole, void* y, clusten_attn_shape s, int dtype,
                              hipStream_t stream) {
    if ((s.C != 16 && s.C != 32 && s.C != 64) || s.N < 8 || s.M % 8 != 0 || s.M > kPairMaxSlots || s.M == 0) return CLUSTEN_ERR_BAD_DIMS;
    if (!scatter_by_cluster_supported(p, x, xs, y, s, dtype)) return CLUSTEN_ERR_UNALIGNED;
    switch (dtype) {
        case CLUSTEN_F32: return launch_typed<float>(p, x, xs, starts, ends, pairs, not_whole, y, s, stream);
        case CLUSTEN_F16: return launch_typed<f16_t>(p, x, xs, starts, ends, pairs, not_whole, y, s, stream);
        case CLUSTEN_BF16: return launch_typed<bf16_t>(p, x, xs, starts, ends, pairs, not_whole, y, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
