// merge_centres: which tokens the adaptive down-sampling of the reference model keeps as merge centres
// (models/aff_transformer.py:296-334, `ClusterMerging.forward`), and the rows of the per-token tensors that go
// with them (:336-346).  The reference spells the selection out as some fifteen tensor operations and a top-k:
//
//   prior    = 1 where the token lies on the (adaptive) grid, else 0                         (:296-303)
//   score    = prior + learned_prob * alpha  [+ (-100) on the reserved coarse grid]          (:305-317)
//   sampled  = the keep - reserve_num tokens of highest score                                (:320)
//   centres  = sampled, then the reserved tokens in ascending index order                    (:322-326)
//
// here one workgroup per image: scores as order-preserving 32-bit keys in LDS, the k-th largest key by a radix
// select over its four bytes, then the selected indices written in a fixed order (`topk(sorted=False)` leaves the
// order open): first the tokens above the k-th score by ascending index, then as many of those equal to it as are
// still needed, by ascending index.  Every float operation is the single rounded operation the tensor expressions
// perform, in their order.  The second kernel gathers the rows of up to four tensors at the centres in one launch.
// Neither has a counterpart in the reference's extension modules.
#include "launch.hpp"

#pragma clang fp contract(off)

namespace clusten {
namespace {

constexpr int kMergeThreads = 1024;

// python's `%` on floats for a positive divisor (torch.remainder): the result has the sign of the divisor
__device__ __forceinline__ float py_mod(float a, float m) {
    float r = fmodf(a, m);
    if (r != 0.f && (r < 0.f)) r += m;
    return r;
}

// what `.long()` does to a float on this device for the values that occur here (truncation)
__device__ __forceinline__ long long as_long(float v) { return (long long)v; }

__device__ __forceinline__ long long py_mod_long(long long a, long long m) {
    long long r = a % m;
    if (r != 0 && ((r < 0) != (m < 0))) r += m;
    return r;
}

template <typename T>
__device__ __forceinline__ float score_of(const float2 p, const float* __restrict__ min_dist, const T* __restrict__ prob,
                                          int64_t e, float alpha, int stride, int reserve_on, bool* reserved) {
    float prior;
    if (min_dist == nullptr) {
        prior = (py_mod(p.x, (float)stride) + py_mod(p.y, (float)stride)) == 0.f ? 1.f : 0.f;
    } else {
        // spacing = 2 ** (ceil(log2(distance to the nearest other token)) + 1)
        const float spacing = exp2f(ceilf(log2f(min_dist[e])) + 1.f);
        const long long s = as_long(spacing);
        prior = 0.f;
        if (s != 0) prior = (py_mod_long(as_long(p.x), s) + py_mod_long(as_long(p.y), s)) == 0 ? 1.f : 0.f;
    }
    float score = prior;
    if (prob != nullptr) {
        // the product is rounded to the type of the probabilities before it is widened for the sum
        const T lp = from_acc<T>(to_acc(prob[e]) * alpha);
        score = score + to_acc(lp);
    }
    *reserved = false;
    if (reserve_on) {
        const float coarse = (float)(stride * 2);
        *reserved = (py_mod(p.x, coarse) + py_mod(p.y, coarse)) == 0.f;
        score = score + (*reserved ? 1.f : 0.f) * -100.f;
    }
    return score;
}

// keys order like the scores: larger score, larger key; -0 and +0 share a key
__device__ __forceinline__ uint32_t key_of_score(float s) {
    if (s == 0.f) s = 0.f;
    const uint32_t u = __float_as_uint(s);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// exclusive prefix over the workgroup's threads and the total
__device__ __forceinline__ int scan_threads(int v, int* scratch, int* total) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, W = blockDim.x >> 6;
    int inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(inc, d);
        if (lane >= d) inc += up;
    }
    __syncthreads();
    if (lane == 63) scratch[w] = inc;
    __syncthreads();
    int before = 0, all = 0;
    for (int k = 0; k < W; ++k) {
        const int t = scratch[k];
        if (k < w) before += t;
        all += t;
    }
    *total = all;
    return before + inc - v;
}

// one workgroup per image; thread t owns the tokens t*chunk .. t*chunk+chunk-1, so that prefix sums over the threads
// are prefix sums over the token indices
template <typename T>
__global__ __launch_bounds__(kMergeThreads) void merge_centres_kernel(const float2* __restrict__ pos,
                                                                      const float* __restrict__ min_dist,
                                                                      const T* __restrict__ prob,
                                                                      int64_t* __restrict__ centre, int N, int sample_num,
                                                                      int reserve_num, int reserve_on, float alpha,
                                                                      int stride) {
    extern __shared__ uint32_t keys[];          // N keys, then 256 bins, 16 wave totals, 4 words of state
    uint32_t* hist = keys + N;
    int* scratch = reinterpret_cast<int*>(hist + 256);
    uint32_t* state = reinterpret_cast<uint32_t*>(scratch + 16);     // [0] prefix, [1] still to find
    const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int chunk = (N + kMergeThreads - 1) / kMergeThreads;
    const int lo = min(tid * chunk, N), hi = min(lo + chunk, N);
    const int out_n = sample_num + (reserve_on ? reserve_num : 0);

    uint64_t reserved_bits = 0;                 // bit c: token lo + c is reserved (chunk <= 64)
    for (int i = lo; i < hi; ++i) {
        const int64_t e = (int64_t)b * N + i;
        bool r;
        keys[i] = key_of_score(score_of<T>(pos[e], min_dist, prob, e, alpha, stride, reserve_on, &r));
        if (r) reserved_bits |= 1ull << (i - lo);
    }
    if (tid == 0) {
        state[0] = 0;
        state[1] = (uint32_t)sample_num;
    }
    // the sample_num-th largest key, one byte at a time from the top
    uint32_t known = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        const uint32_t prefix = state[0];
        for (int i = lo; i < hi; ++i) {
            const uint32_t k = keys[i];
            if ((k & known) == prefix) atomicAdd(&hist[(k >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (tid < 64) {
            // lane l holds the bins 255-4l .. 252-4l, highest first
            const uint32_t want = state[1];
            uint32_t c[4], mine = 0;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                c[u] = hist[255 - 4 * lane - u];
                mine += c[u];
            }
            uint32_t inc = mine;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(inc, d);
                if (lane >= d) inc += up;
            }
            const uint64_t reached = __ballot(inc >= want);
            const int first = __ffsll((unsigned long long)reached) - 1;      // some lane reaches it: want <= matching keys
            if (lane == first) {
                uint32_t above = inc - mine;
                int u = 0;
                while (u < 3 && above + c[u] < want) above += c[u++];
                state[0] = prefix | ((uint32_t)(255 - 4 * lane - u) << shift);
                state[1] = want - above;
            }
        }
        known |= 255u << shift;
        __syncthreads();
    }
    const uint32_t kth = state[0];
    const int ties = (int)state[1];             // how many of the keys equal to kth are taken
    const int above_total = sample_num - ties;

    int n_above = 0, n_equal = 0, n_res = 0;
    for (int i = lo; i < hi; ++i) {
        const uint32_t k = keys[i];
        n_above += k > kth;
        n_equal += k == kth;
    }
    n_res = __popcll(reserved_bits);
    int total;
    int at_above = scan_threads(n_above, scratch, &total);
    int at_equal = scan_threads(n_equal, scratch, &total);
    int at_res = scan_threads(n_res, scratch, &total);
    int64_t* out = centre + (int64_t)b * out_n;
    // an image with fewer reserved tokens than reserve_num (the reference's reshape raises there,
    // models/aff_transformer.py:323): the slots nobody fills hold -1, which the caller can test for and which
    // merge_rows_kernel reads as row 0
    if (reserve_on) {
        for (int s = total + (int)threadIdx.x; s < reserve_num; s += (int)blockDim.x) out[sample_num + s] = -1;
    }
    for (int i = lo; i < hi; ++i) {
        const uint32_t k = keys[i];
        if (k > kth) {
            out[at_above++] = i;
        } else if (k == kth) {
            if (at_equal < ties) out[above_total + at_equal] = i;
            ++at_equal;
        }
        if (reserve_on && ((reserved_bits >> (i - lo)) & 1)) {
            if (at_res < reserve_num) out[sample_num + at_res] = i;
            ++at_res;
        }
    }
}

struct MergeRows {
    const uint64_t* src[4];
    uint64_t* dst[4];
    int words[4];       // 8-byte words per row
    int first[5];       // first[t] = words of the tensors before t; first[count] = all
    int count;
};

// rows of up to four (B,N,.) tensors at the centres: dst_t[b,i,:] = src_t[b, centre[b,i], :]; one thread per 8 bytes
__global__ __launch_bounds__(256) void merge_rows_kernel(MergeRows r, const int64_t* __restrict__ centre, int N, int n_out,
                                                         int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const int W = r.first[r.count];
    const int64_t row = e / W;
    const int w = (int)(e - row * W);
    const int64_t b = row / n_out;
    const int64_t c = centre[row];
    const int64_t from = b * N + ((uint64_t)c < (uint64_t)N ? c : 0);   // an index outside [0,N) reads row 0
    int t = 0;
#pragma unroll
    for (int u = 1; u < 4; ++u) t += (u < r.count && w >= r.first[u]);
    const int at = w - r.first[t];
    r.dst[t][row * r.words[t] + at] = r.src[t][from * r.words[t] + at];
}

template <typename T>
int launch_typed(const float* pos, const float* min_dist, const void* prob, int64_t* centre, int B, int N, int sample_num,
                 int reserve_num, int reserve_on, float alpha, int stride, hipStream_t stream) {
    const size_t lds = ((size_t)N + 256 + 16 + 4) * 4;
    if (lds > 48 * 1024) {
        // more LDS than a workgroup gets without asking (a CU of this device holds 160 KB)
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(merge_centres_kernel<T>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
            (void)hipGetLastError();
            return CLUSTEN_ERR_BAD_DIMS;
        }
    }
    hipLaunchKernelGGL(merge_centres_kernel<T>, dim3((unsigned)B), dim3(kMergeThreads), lds, stream,
                       reinterpret_cast<const float2*>(pos), min_dist, static_cast<const T*>(prob), centre, N, sample_num,
                       reserve_num, reserve_on, alpha, stride);
    return launch_status();
}

}  // namespace

// The longest sequence whose keys the selecting workgroup holds in LDS; a thread owns at most 64 tokens (the
// reserved-token bits of its share are one 64-bit word).
int merge_centres_max_tokens() {
    int dev = 0, bytes = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) {
        (void)hipGetLastError();
        bytes = 48 * 1024;
    }
    const int by_lds = (bytes - (256 + 16 + 4) * 4) / 4;
    return by_lds < 64 * kMergeThreads ? by_lds : 64 * kMergeThreads;
}

int launch_merge_centres(const float* pos, const float* min_dist, const void* prob, int prob_dtype, int64_t* centre, int B,
                         int N, int sample_num, int reserve_num, int reserve_on, float alpha, int stride,
                         hipStream_t stream) {
    if (B <= 0 || N <= 0 || N > merge_centres_max_tokens() || sample_num <= 0 || sample_num > N || stride <= 0 ||
        reserve_num < 0 || sample_num + (reserve_on ? reserve_num : 0) > N)
        return CLUSTEN_ERR_BAD_DIMS;
    switch (prob_dtype) {
        case CLUSTEN_F32: return launch_typed<float>(pos, min_dist, prob, centre, B, N, sample_num, reserve_num, reserve_on, alpha, stride, stream);
        case CLUSTEN_F16: return launch_typed<f16_t>(pos, min_dist, prob, centre, B, N, sample_num, reserve_num, reserve_on, alpha, stride, stream);
        case CLUSTEN_BF16: return launch_typed<bf16_t>(pos, min_dist, prob, centre, B, N, sample_num, reserve_num, reserve_on, alpha, stride, stream);
    }
    return CLUSTEN_ERR_BAD_DTYPE;
}

int launch_merge_rows(const void* const* src, void* const* dst, const int* row_bytes, int count, const int64_t* centre,
                      int64_t B, int N, int n_out, hipStream_t stream) {
    if (count < 1 || count > 4 || B <= 0 || N <= 0 || n_out <= 0) return CLUSTEN_ERR_BAD_DIMS;
    MergeRows r{};
    r.count = count;
    int W = 0;
    for (int t = 0; t < count; ++t) {
        if (src[t] == nullptr || dst[t] == nullptr) return CLUSTEN_ERR_NULL_POINTER;
        if (row_bytes[t] <= 0 || row_bytes[t] % 8 != 0) return CLUSTEN_ERR_BAD_DIMS;
        if (reinterpret_cast<uintptr_t>(src[t]) % 8 != 0 || reinterpret_cast<uintptr_t>(dst[t]) % 8 != 0)
            return CLUSTEN_ERR_UNALIGNED;
        r.src[t] = static_cast<const uint64_t*>(src[t]);
        r.dst[t] = static_cast<uint64_t*>(dst[t]);
        r.words[t] = row_bytes[t] / 8;
        r.first[t] = W;
        W += r.words[t];
    }
    for (int t = count; t <= 4; ++t) r.first[t] = W;
    const int64_t total = B * n_out * W;
    hipLaunchKernelGGL(merge_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, r, centre, N, n_out,
                       total);
    return launch_status();
}

}  // namespace clusten
