// Storage-type dispatch for the WF kernels (see wf_impl.hpp) and their fp64 instantiations.
#include "wf_impl.hpp"

namespace clusten {

int wf_forward_f32(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);
int wf_forward_f16(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);
int wf_forward_bf16(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);

int launch_wf_forward(const void* w, const void* feat, const int64_t* idx, void* out, clusten_wf_shape s, int dtype,
                      hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return wf_forward_f32(w, feat, idx, out, s, stream);
        case CLUSTEN_F16: return wf_forward_f16(w, feat, idx, out, s, stream);
        case CLUSTEN_BF16: return wf_forward_bf16(w, feat, idx, out, s, stream);
        case CLUSTEN_F64: return wf_forward_elem<double>(w, feat, idx, out, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int wf_forward_mixed_f16(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);
int wf_forward_mixed_bf16(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);

int launch_wf_forward_mixed(const void* w, const void* feat, const int64_t* idx, void* out, clusten_wf_shape s,
                            int feat_dtype, hipStream_t stream) {
    switch (feat_dtype) {
        case CLUSTEN_F16: return wf_forward_mixed_f16(w, feat, idx, out, s, stream);
        case CLUSTEN_BF16: return wf_forward_mixed_bf16(w, feat, idx, out, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int launch_wf_dweights(const void* d_out, const void* feat, const int64_t* idx, void* d_w, clusten_wf_shape s,
                       int dtype, hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return wf_dweights_typed<float>(d_out, feat, idx, d_w, s, stream);
        case CLUSTEN_F16: return wf_dweights_typed<f16_t>(d_out, feat, idx, d_w, s, stream);
        case CLUSTEN_BF16: return wf_dweights_typed<bf16_t>(d_out, feat, idx, d_w, s, stream);
        case CLUSTEN_F64: return wf_dweights_typed<double>(d_out, feat, idx, d_w, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

namespace {

// See ScatterPlan in scatter_rows.hip: pair lists first (when the shape admits the cluster-by-cluster kernel), then
// the fp32 sums of 16-bit data.
struct DfeatPlan {
    bool by_cluster;            // lists made of whole clusters (found out on the device): gather over sorted pair lists
    bool by_row;                // any other list: gather over the entries sorted by destination row
    ClusterPairsLayout pairs;
    RowEntriesLayout rows;
    size_t rows_at;             // offset of the row entries block
    size_t acc32;               // offset of the fp32 buffer of the atomic kernels (16-bit data, shapes by_row does not take)
    size_t bytes;
};

DfeatPlan dfeat_plan(const clusten_wf_shape& s, int dtype) {
    DfeatPlan plan;
    plan.by_cluster = dtype != CLUSTEN_F64 && s.IC == 4 && s.C % 32 == 0 && cluster_pairs_supported(s.B, s.Nout, s.M, s.N);
    plan.by_row = dtype != CLUSTEN_F64 && s.IC <= 4 && s.C % 4 == 0 && row_entries_supported(s.B, s.Nout, s.M, s.N);
    plan.pairs = plan.by_cluster ? cluster_pairs_layout(s.B, s.Nout, s.M, s.N) : ClusterPairsLayout{};
    plan.rows = plan.by_row ? row_entries_layout(s.B, s.Nout, s.M, s.N) : RowEntriesLayout{};
    plan.rows_at = plan.by_cluster ? plan.pairs.bytes : 0;
    plan.acc32 = plan.rows_at + (plan.by_row ? plan.rows.bytes : 0);
    const bool narrow = dtype == CLUSTEN_F16 || dtype == CLUSTEN_BF16;
    plan.bytes = plan.acc32 + (narrow ? (size_t)s.B * s.N * s.C * sizeof(float) : 0);
    return plan;
}

}  // namespace

size_t wf_dfeat_workspace_bytes(clusten_wf_shape s, int dtype) { return dfeat_plan(s, dtype).bytes; }

int launch_wf_dfeat(const void* d_out, const void* w, const int64_t* idx, void* d_feat, void* workspace,
                    clusten_wf_shape s, int dtype, hipStream_t stream) {
    const size_t count = (size_t)s.B * s.N * s.C;
    const DfeatPlan plan = dfeat_plan(s, dtype);
    if (plan.bytes != 0 && !aligned16(workspace)) return CLUSTEN_ERR_UNALIGNED;
    char* ws = static_cast<char*>(workspace);
    int st;
    // lists made of whole clusters: a gather over sorted pair lists, chosen on the device through `flag`
    const int32_t* flag = nullptr;
    if (plan.by_cluster && wf_dfeat_by_cluster_supported(d_out, w, d_feat, s, dtype)) {
        int32_t* not_whole = reinterpret_cast<int32_t*>(ws + plan.pairs.flag);
        int32_t* keys = reinterpret_cast<int32_t*>(ws + plan.pairs.keys);
        int32_t* wg_bad = reinterpret_cast<int32_t*>(ws + plan.pairs.wg_bad);
        int32_t* pairs = reinterpret_cast<int32_t*>(ws + plan.pairs.pairs);
        int32_t* starts = reinterpret_cast<int32_t*>(ws + plan.pairs.starts);
        int32_t* ends = reinterpret_cast<int32_t*>(ws + plan.pairs.ends);
        st = launch_cluster_pairs(idx, keys, wg_bad, not_whole, pairs, starts, ends, s.B, s.Nout, s.M, s.N, stream);
        if (st != CLUSTEN_OK) return st;
        st = launch_wf_dfeat_by_cluster(d_out, w, starts, ends, pairs, not_whole, d_feat, s, dtype, stream);
        if (st != CLUSTEN_OK) return st;
        flag = not_whole;
    }
    // any other list: the entries sorted by destination row, one wave per row (these kernels return at once when the
    // flag says the lists were whole clusters)
    if (plan.by_row && wf_dfeat_rows_supported(d_out, d_feat, s, dtype)) {
        int32_t* entries = reinterpret_cast<int32_t*>(ws + plan.rows_at + plan.rows.entries);
        int32_t* rstarts = reinterpret_cast<int32_t*>(ws + plan.rows_at + plan.rows.starts);
        int32_t* rends = reinterpret_cast<int32_t*>(ws + plan.rows_at + plan.rows.ends);
        st = launch_row_entries(idx, flag, entries, rstarts, rends, s.B, s.Nout, s.M, s.N, stream);
        if (st != CLUSTEN_OK) return st;
        return launch_wf_dfeat_rows(d_out, w, rstarts, rends, entries, flag, d_feat, s, dtype, stream);
    }
    // shapes neither takes (and fp64): atomics
    switch (dtype) {
        case CLUSTEN_F32:
            st = launch_zero_f32(static_cast<float*>(d_feat), count, stream, flag);
            if (st != CLUSTEN_OK) return st;
            return wf_dfeat_typed<float, float>(d_out, w, idx, static_cast<float*>(d_feat), s, stream, flag);
        case CLUSTEN_F16:
        case CLUSTEN_BF16: {
            float* acc32 = reinterpret_cast<float*>(ws + plan.acc32);
            st = launch_zero_f32(acc32, count, stream, flag);
            if (st != CLUSTEN_OK) return st;
            st = dtype == CLUSTEN_F16 ? wf_dfeat_typed<f16_t, float>(d_out, w, idx, acc32, s, stream, flag)
                                      : wf_dfeat_typed<bf16_t, float>(d_out, w, idx, acc32, s, stream, flag);
            if (st != CLUSTEN_OK) return st;
            return launch_round_from_f32(acc32, d_feat, count, dtype, stream, flag);
        }
        case CLUSTEN_F64:
            st = launch_zero_f64(static_cast<double*>(d_feat), count, stream);
            if (st != CLUSTEN_OK) return st;
            return wf_dfeat_typed<double, double>(d_out, w, idx, static_cast<double*>(d_feat), s, stream, nullptr);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
