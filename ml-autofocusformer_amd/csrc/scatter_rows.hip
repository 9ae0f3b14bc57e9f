// Storage-type dispatch for scatter_rows (see scatter_rows_impl.hpp).  Two sets of kernels are enqueued and a device
// flag decides which of them works: the pair lists and the cluster-by-cluster gather (cluster_pairs.hip,
// scatter_by_cluster.hip) for lists made of whole clusters, the zero-fill, atomic scatter (tiles with one list through
// an LDS window, scatter_rows_window.hip; the others tile by tile) and rounding to fp16/bf16 for any other list.  The
// host never learns which: nothing is read back.
#include "scatter_rows_impl.hpp"

namespace clusten {

int scatter_rows_f32(const void*, const void*, clusten_strides, const int64_t*, float*, const clusten_attn_shape&, hipStream_t,
                     const int32_t*, const uint8_t*);
int scatter_rows_f16(const void*, const void*, clusten_strides, const int64_t*, float*, const clusten_attn_shape&, hipStream_t,
                     const int32_t*, const uint8_t*);
int scatter_rows_bf16(const void*, const void*, clusten_strides, const int64_t*, float*, const clusten_attn_shape&, hipStream_t,
                      const int32_t*, const uint8_t*);
// scatter_rows_window.hip
bool scatter_rows_window_supported(const clusten_attn_shape& s, int dtype);
size_t scatter_rows_window_handled_bytes(const clusten_attn_shape& s);
int launch_scatter_rows_window(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32,
                               uint8_t* handled, const clusten_attn_shape& s, int dtype, hipStream_t stream,
                               const int32_t* only_if);

namespace {

// Workspace of one scatter: the pair lists of the cluster-by-cluster kernel when the shape admits it (whether the
// lists are made of whole clusters is found out on the device), one byte per tile for the window kernel's account of
// the tiles it has added, then the fp32 sums of 16-bit data for the atomic kernels.
struct ScatterPlan {
    bool by_cluster;
    bool window;
    ClusterPairsLayout pairs;
    size_t handled; // offset of the tile bytes
    size_t acc32;   // offset of the fp32 buffer
    size_t bytes;
};

ScatterPlan scatter_plan(const clusten_attn_shape& s, int dtype) {
    ScatterPlan plan;
    plan.by_cluster = dtype != CLUSTEN_F64 && (s.C == 16 || s.C == 32 || s.C == 64) &&
                      cluster_pairs_supported(s.B, s.N, s.M, s.N);
    plan.pairs = plan.by_cluster ? cluster_pairs_layout(s.B, s.N, s.M, s.N) : ClusterPairsLayout{};
    plan.window = s.M % 4 == 0 && scatter_rows_window_supported(s, dtype);
    plan.handled = plan.by_cluster ? plan.pairs.bytes : 0;
    plan.acc32 = plan.handled + (plan.window ? scatter_rows_window_handled_bytes(s) : 0);
    const bool narrow = dtype == CLUSTEN_F16 || dtype == CLUSTEN_BF16;
    plan.bytes = plan.acc32 + (narrow ? (size_t)s.B * s.H * s.N * s.C * sizeof(float) : 0);
    return plan;
}

}  // namespace

size_t scatter_rows_workspace_bytes(clusten_attn_shape s, int dtype) { return scatter_plan(s, dtype).bytes; }

int launch_scatter_rows(const void* p, const void* x, clusten_strides xs, const int64_t* idx, void* out,
                        void* workspace, clusten_attn_shape s, int dtype, hipStream_t stream, const void* pair_lists) {
    const size_t count = (size_t)s.B * s.H * s.N * s.C;
    const ScatterPlan plan = scatter_plan(s, dtype);
    if (plan.bytes != 0 && !aligned16(workspace)) return CLUSTEN_ERR_UNALIGNED;
    char* ws = static_cast<char*>(workspace);
    int st;
    // lists made of whole clusters: a gather over sorted pair lists, chosen on the device through `flag`
    const int32_t* flag = nullptr;
    if (plan.by_cluster && scatter_by_cluster_supported(p, x, xs, out, s, dtype)) {
        // the caller's pair lists of these lists (built once for every layer and head that uses them), or the
        // workspace's, built now
        char* block = pair_lists != nullptr ? const_cast<char*>(static_cast<const char*>(pair_lists)) : ws;
        int32_t* not_whole = reinterpret_cast<int32_t*>(block + plan.pairs.flag);
        int32_t* pairs = reinterpret_cast<int32_t*>(block + plan.pairs.pairs);
        int32_t* starts = reinterpret_cast<int32_t*>(block + plan.pairs.starts);
        int32_t* ends = reinterpret_cast<int32_t*>(block + plan.pairs.ends);
        if (pair_lists == nullptr) {
            int32_t* keys = reinterpret_cast<int32_t*>(block + plan.pairs.keys);
            int32_t* wg_bad = reinterpret_cast<int32_t*>(block + plan.pairs.wg_bad);
            st = launch_cluster_pairs(idx, keys, wg_bad, not_whole, pairs, starts, ends, s.B, s.N, s.M, s.N, stream);
            if (st != CLUSTEN_OK) return st;
        }
        st = launch_scatter_by_cluster(p, x, xs, starts, ends, pairs, not_whole, out, s, dtype, stream);
        if (st != CLUSTEN_OK) return st;
        flag = not_whole;
    }
    // any other list: atomics (these kernels return at once when the flag says the lists were whole clusters); tiles
    // whose tokens share one list go through the LDS window, the tile kernel takes the others
    uint8_t* handled = nullptr;
    if (plan.window && reinterpret_cast<uintptr_t>(p) % (4 * dtype_size(dtype)) == 0) {
        handled = reinterpret_cast<uint8_t*>(ws + plan.handled);
    }
    switch (dtype) {
        case CLUSTEN_F32:
            st = launch_zero_f32(static_cast<float*>(out), count, stream, flag);
            if (st != CLUSTEN_OK) return st;
            if (handled != nullptr) {
                st = launch_scatter_rows_window(p, x, xs, idx, static_cast<float*>(out), handled, s, dtype, stream, flag);
                if (st != CLUSTEN_OK) return st;
            }
            return scatter_rows_f32(p, x, xs, idx, static_cast<float*>(out), s, stream, flag, handled);
        case CLUSTEN_F16:
        case CLUSTEN_BF16: {
            float* acc32 = reinterpret_cast<float*>(ws + plan.acc32);
            st = launch_zero_f32(acc32, count, stream, flag);
            if (st != CLUSTEN_OK) return st;
            if (handled != nullptr) {
                st = launch_scatter_rows_window(p, x, xs, idx, acc32, handled, s, dtype, stream, flag);
                if (st != CLUSTEN_OK) return st;
            }
            st = dtype == CLUSTEN_F16 ? scatter_rows_f16(p, x, xs, idx, acc32, s, stream, flag, handled)
                                      : scatter_rows_bf16(p, x, xs, idx, acc32, s, stream, flag, handled);
            if (st != CLUSTEN_OK) return st;
            return launch_round_from_f32(acc32, out, count, dtype, stream, flag);
        }
        case CLUSTEN_F64:
            st = launch_zero_f64(static_cast<double*>(out), count, stream);
            if (st != CLUSTEN_OK) return st;
            return scatter_elem<double, double>(p, x, xs, idx, static_cast<double*>(out), s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
