// wf_dfeat_by_cluster: the feature gradient of the WF operator as a gather (no atomics).
//
//   d_feat[b, idx[b,i,j], c] += sum_ic d_out[b,i,ic,c] * w[b,i,j,ic]          (clusten/src/clustenwf_cuda_kernel.cu:96-135)
//
// for neighbour lists made of whole clusters (idx[b,i,8r+t] = 8 c(b,i,r) + t: the lists a merge of the reference
// model reads, models/aff_transformer.py:476-480 gathered at :336).  The 8 rows of cluster g of the finer sequence
// receive
//
//   d_feat[b, 8g + t, :] = sum over the pairs (i, r) with c(b,i,r) = g of  sum_ic w[b,i,8r+t,ic] * d_out[b,i,ic,:]
//
// With the pairs of every cluster listed once (cluster_pairs.hip: the same sorted pair lists) a pair is one
// `v_mfma_f32_16x16x4_f32` per 16 channels: A = the pair's 8 x 4 block of weights (32 contiguous elements), B = the
// four d_out rows of its output token, k = the inner channel.  One wave per cluster takes the channels 32 at a time;
// d_out rows and weight blocks of 8 pairs at a time travel to LDS by LDS-direct loads (16-bit data is widened when the
// operands are read).  Every row of d_feat is written exactly once, from fp32 sums over all its pairs: no atomics, no
// zero-fill, no fp32 workspace.  It has no counterpart in the reference's extension modules.
#include "launch.hpp"
#include "mfma.hpp"

namespace clusten {
namespace {

constexpr int kChunk = 32;       // channels per pass over the pairs
constexpr int kPass = 8;         // pairs per pass
constexpr int kListMax = 256;    // pairs of a cluster held in LDS at a time
constexpr int kIC = 4;           // inner channels: the k of the matrix instruction
constexpr int kPadEntry = 1 << 30;   // list entry flag: see scatter_by_cluster.hip
constexpr int kEntryMask = kPadEntry - 1;

template <typename T>
__global__ __launch_bounds__(kWave) void wf_dfeat_by_cluster_kernel(const T* __restrict__ d_out, const T* __restrict__ w,
                                                                    const int32_t* __restrict__ starts,
                                                                    const int32_t* __restrict__ ends,
                                                                    const int32_t* __restrict__ pairs,
                                                                    const int32_t* __restrict__ not_whole,
                                                                    T* __restrict__ d_feat, int N, int Nout, int C, int M,
                                                                    int clusters_per_image, int total_clusters) {
    constexpr int EB = (int)sizeof(T);
    constexpr int ROW_B = kChunk * EB;                 // bytes of a d_out row inside the chunk
    constexpr int PAIR_B = kIC * ROW_B;                // the four rows of a pair
    constexpr int X_BYTES = kPass * PAIR_B;
    constexpr int X_DMA = X_BYTES / 1024;
    constexpr int LANES_PER_ROW = ROW_B / 16;
    constexpr int LANES_PER_PAIR = PAIR_B / 16;
    constexpr int W_B = 8 * kIC * EB;                  // a pair's block of weights
    constexpr int LANES_PER_W = W_B / 16;
    constexpr int X_BASE = 0;
    constexpr int W_BASE = X_BASE + X_BYTES;
    constexpr int O_BASE = W_BASE + 1024;
    constexpr int L_BASE = O_BASE + 8 * kChunk * 4;
    constexpr int LDS_BYTES = L_BASE + kListMax * 4;
    __shared__ __attribute__((aligned(1024))) char stage[LDS_BYTES];

    const int unit = xcd_tile(blockIdx.x, total_clusters);
    if (unit < 0) return;
    // the flag and the bounds of the cluster's list are requested together (one trip to memory, not two); the bounds
    // mean nothing when the flag is set, and are not used then
    const int flagged = not_whole != nullptr ? *not_whole : 0;
    const int first = starts[unit];
    const int last = ends[unit];
    if (flagged != 0) return;   // not lists of whole clusters: the atomic kernel runs instead
    const int b = unit / clusters_per_image;
    const int g = unit - b * clusters_per_image;
    const int lane = threadIdx.x;
    const int r16 = lane & 15, kq = lane >> 4;
    const int count = last - first;
    int* list = reinterpret_cast<int*>(stage + L_BASE);
    const char* d_out_b = reinterpret_cast<const char*>(d_out + (int64_t)b * Nout * kIC * C);
    const char* w_b = reinterpret_cast<const char*>(w + (int64_t)b * Nout * M * kIC);
    T* rows_out = d_feat + ((int64_t)b * N + (int64_t)g * 8) * C;
    const int rows_here = min(8, N - 8 * g);   // the last cluster of a sequence may be short
    const int pad_from = N & 7;                // ... and the lists that name it hold row 0 in slots pad_from .. 7

    // a cluster listed by more than kListMax pairs is taken in segments, every channel chunk walking all of them
    // before it writes its rows; the usual cluster's list is read once for all chunks
    const bool one_segment = count <= kListMax;
    if (one_segment) {
        for (int e = lane; e < count; e += kWave) list[e] = pairs[first + e];
    }
    for (int c0 = 0; c0 < C; c0 += kChunk) {
        F32x4 acc[2] = {F32x4{0.f, 0.f, 0.f, 0.f}, F32x4{0.f, 0.f, 0.f, 0.f}};
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
                    // lane -> (pair, inner channel, 16-byte piece of the row)
                    const int slot = a * 64 + lane;
                    const int e = list[base + min(slot / LANES_PER_PAIR, here - 1)] & kEntryMask;
                    const int ic = (slot / LANES_PER_ROW) % kIC;
                    CLUSTEN_LDS_DMA16(d_out_b + lane_offset((((uint32_t)(e >> kPairRunBits) * kIC + (uint32_t)ic) * (uint32_t)C +
                                                             (uint32_t)c0) * EB + (uint32_t)(lane % LANES_PER_ROW) * 16),
                                      stage + X_BASE + a * 1024);
                }
                if (lane < kPass * LANES_PER_W) {
                    const int e = list[base + min(lane / LANES_PER_W, here - 1)] & kEntryMask;
                    CLUSTEN_LDS_DMA16(w_b + lane_offset(((uint32_t)(e >> kPairRunBits) * (uint32_t)M + (uint32_t)(e & kPairRunMask) * 8) * (kIC * EB) +
                                                        (uint32_t)(lane % LANES_PER_W) * 16),
                                      stage + W_BASE);
                }
                lds_sync_vm<0>();
#pragma unroll
                for (int pr = 0; pr < kPass; ++pr) {
                    if (pr < here) {
                        // A[t][ic] = w[i, 8r + t, ic]; B[ic][c] = d_out[i, ic, c0 + c]
                        const T* wp = reinterpret_cast<const T*>(stage + W_BASE + pr * W_B) + kq;
                        float a = 0.f;
                        if ((list[base + pr] & kPadEntry) == 0) {
                            if (r16 < rows_here) a = to_acc(wp[r16 * kIC]);
                        } else if (r16 == 0) {
                            // a pair that names the short last cluster: its pad slots hold row 0, this cluster's first
                            for (int t = pad_from; t < 8; ++t) a += to_acc(wp[t * kIC]);
                        }
                        const T* xp = reinterpret_cast<const T*>(stage + X_BASE + pr * PAIR_B + kq * ROW_B) + r16;
                        acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, to_acc(xp[0]), acc[0], 0, 0, 0);
                        acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, to_acc(xp[16]), acc[1], 0, 0, 0);
                    }
                }
            }
        }
        // rows 4*kq + j of the result (kq < 2: the cluster's 8 rows), channels c0 + 16*cb + r16
        lds_sync();
        if (kq < 2) {
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    reinterpret_cast<float*>(stage + O_BASE)[(4 * kq + j) * kChunk + 16 * cb + r16] = acc[cb][j];
                }
            }
        }
        lds_sync();
        {
            // 8 rows x 32 channels: four consecutive channels per lane
            const F32x4 o = *reinterpret_cast<const F32x4*>(stage + O_BASE + lane * 16);
            const float v[4] = {o[0], o[1], o[2], o[3]};
            T* dst = rows_out + (int64_t)(lane >> 3) * C + c0 + (lane & 7) * 4;
            if ((lane >> 3) < rows_here) *reinterpret_cast<typename Quad<T>::raw*>(dst) = Quad<T>::pack(v);
        }
    }
}

template <typename T>
int launch_typed(const void* d_out, const void* w, const int32_t* starts, const int32_t* ends, const int32_t* pairs,
                 const int32_t* not_whole, void* d_feat, const clusten_wf_shape& s, hipStream_t stream) {
    const int per_image = (s.N + 7) / 8;
    const int64_t total = (int64_t)s.B * per_image;
    if (total >= ((int64_t)1 << 30)) return CLUSTEN_ERR_BAD_DIMS;
    hipLaunchKernelGGL((wf_dfeat_by_cluster_kernel<T>), dim3(xcd_grid((int)total)), dim3(kWave), 0, stream,
                       static_cast<const T*>(d_out), static_cast<const T*>(w), starts, ends, pairs, not_whole,
                       static_cast<T*>(d_feat), s.N,
                       s.Nout, s.C, s.M, per_image, (int)total);
    return launch_status();
}

}  // namespace

bool wf_dfeat_by_cluster_supported(const void* d_out, const void* w, const void* d_feat, const clusten_wf_shape& s,
                                   int dtype) {
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return false;
    if (s.IC != kIC || s.C % kChunk != 0 || s.N < 8 || s.M % 8 != 0 || s.M > kPairMaxSlots || s.M <= 0) return false;
    const int64_t eb = (int64_t)dtype_size(dtype);
    if ((int64_t)s.Nout * kIC * s.C * eb >= ((int64_t)1 << 31) || (int64_t)s.Nout * s.M * kIC * eb >= ((int64_t)1 << 31)) {
        return false;
    }
    return aligned16(d_out) && aligned16(w) && aligned16(d_feat);
}

int launch_wf_dfeat_by_cluster(const void* d_out, const void* w, const int32_t* starts, const int32_t* ends,
                               const int32_t* pairs, const int32_t* not_whole, void* d_feat, clusten_wf_shape s, int dtype,
                               hipStream_t stream) {
    if (s.IC != kIC || s.C % kChunk != 0 || s.N < 8 || s.M % 8 != 0 || s.M > kPairMaxSlots || s.M == 0) return CLUSTEN_ERR_BAD_DIMS;
    if (!wf_dfeat_by_cluster_supported(d_out, w, d_feat, s, dtype)) return CLUSTEN_ERR_UNALIGNED;
    switch (dtype) {
        case CLUSTEN_F32: return launch_typed<float>(d_out, w, starts, ends, pairs, not_whole, d_feat, s, stream);
        case CLUSTEN_F16: return launch_typed<f16_t>(d_out, w, starts, ends, pairs, not_whole, d_feat, s, stream);
        case CLUSTEN_BF16: return launch_typed<bf16_t>(d_out, w, starts, ends, pairs, not_whole, d_feat, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
