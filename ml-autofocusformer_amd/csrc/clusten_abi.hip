// extern "C" surface of libclusten_hip.so (declared in include/clusten_hip.h): argument checks,
// then the internal launch functions.  Nothing here allocates, frees or synchronises.
#include "launch.hpp"

using namespace clusten;

namespace {

inline hipStream_t as_stream(clusten_stream s) { return static_cast<hipStream_t>(s); }

inline int check_attn_call(const clusten_attn_shape& s, int dtype) {
    if (!dtype_ok(dtype)) return CLUSTEN_ERR_BAD_DTYPE;
    return check_attn_shape(s);
}

inline clusten_strides contiguous_strides(const clusten_attn_shape& s) {
    clusten_strides r;
    r.n = s.C;
    r.h = (int64_t)s.N * s.C;
    r.b = (int64_t)s.H * s.N * s.C;
    return r;
}

}  // namespace

extern "C" {

int clusten_abi_version(void) { return CLUSTEN_ABI_VERSION; }

const char* clusten_status_string(int status) {
    switch (status) {
        case CLUSTEN_OK: return "ok";
        case CLUSTEN_ERR_NULL_POINTER: return "a required pointer is NULL";
        case CLUSTEN_ERR_BAD_DTYPE: return "unknown dtype code";
        case CLUSTEN_ERR_BAD_DIMS: return "a size is not positive or exceeds the 32-bit indexing limits";
        case CLUSTEN_ERR_BAD_STRIDE: return "a stride is negative or rows overlap";
        case CLUSTEN_ERR_WORKSPACE: return "workspace missing or too small";
        case CLUSTEN_ERR_LAUNCH: return "kernel launch failed";
        case CLUSTEN_ERR_UNALIGNED: return "pointer or stride is not aligned";
        case CLUSTEN_ERR_TOO_LARGE: return "problem exceeds the fixed scratch of the allocation-free entry point";
        default: return "unknown status";
    }
}

int clusten_qk_forward(const void* query, clusten_strides query_strides, const void* key, clusten_strides key_strides,
                       const int64_t* nbhd_idx, void* attn, clusten_attn_shape shape, int dtype,
                       clusten_stream stream) {
    if (!query || !key || !nbhd_idx || !attn) return CLUSTEN_ERR_NULL_POINTER;
    if (int st = check_attn_call(shape, dtype)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    return launch_gather_dot(query, query_strides, key, key_strides, nbhd_idx, attn, shape, dtype, as_stream(stream));
}

size_t clusten_qk_backward_workspace_bytes(clusten_attn_shape shape, int dtype) {
    if (!dtype_ok(dtype) || check_attn_shape(shape) != CLUSTEN_OK) return 0;
    return scatter_rows_workspace_bytes(shape, dtype);
}

int clusten_qk_backward(const void* d_attn, const void* query, clusten_strides query_strides, const void* key,
                        clusten_strides key_strides, const int64_t* nbhd_idx, void* d_query, void* d_key,
                        void* workspace, size_t workspace_bytes, clusten_attn_shape shape, int dtype,
                        clusten_stream stream) {
    if (!d_attn || !query || !key || !nbhd_idx || !d_query || !d_key) return CLUSTEN_ERR_NULL_POINTER;
    if (int st = check_attn_call(shape, dtype)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    const size_t need = scatter_rows_workspace_bytes(shape, dtype);
    if (need && (!workspace || workspace_bytes < need)) return CLUSTEN_ERR_WORKSPACE;
    // d_query = gather_sum(d_attn, key)
    int st = launch_gather_sum(d_attn, key, key_strides, nbhd_idx, d_query, contiguous_strides(shape), shape, dtype,
                               as_stream(stream));
    if (st != CLUSTEN_OK) return st;
    // d_key = scatter_rows(d_attn, query)
    return launch_scatter_rows(d_attn, query, query_strides, nbhd_idx, d_key, workspace, shape, dtype,
                               as_stream(stream));
}

int clusten_av_forward(const void* attn, const void* value, clusten_strides value_strides, const int64_t* nbhd_idx,
                       void* feat, clusten_strides feat_strides, clusten_attn_shape shape, int dtype,
                       clusten_stream stream) {
    if (!attn || !value || !nbhd_idx || !feat) return CLUSTEN_ERR_NULL_POINTER;
    if (int st = check_attn_call(shape, dtype)) return st;
    if (!strides_ok(value_strides, shape.C) || !strides_ok(feat_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    return launch_gather_sum(attn, value, value_strides, nbhd_idx, feat, feat_strides, shape, dtype,
                             as_stream(stream));
}

int clusten_av_forward_mixed(const void* attn, const void* value, clusten_strides value_strides, int value_dtype,
                             const int64_t* nbhd_idx, void* feat, clusten_strides feat_strides, clusten_attn_shape shape,
                             clusten_stream stream) {
    if (!attn || !value || !nbhd_idx || !feat) return CLUSTEN_ERR_NULL_POINTER;
    if (value_dtype != CLUSTEN_F16 && value_dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(value_strides, shape.C) || !strides_ok(feat_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    return launch_gather_sum_mixed(attn, value, value_strides, nbhd_idx, feat, feat_strides, shape, value_dtype,
                                   as_stream(stream));
}

size_t clusten_av_backward_workspace_bytes(clusten_attn_shape shape, int dtype) {
    if (!dtype_ok(dtype) || check_attn_shape(shape) != CLUSTEN_OK) return 0;
    return scatter_rows_workspace_bytes(shape, dtype);
}

int clusten_av_backward(const void* d_feat, clusten_strides d_feat_strides, const void* attn, const void* value,
                        clusten_strides value_strides, const int64_t* nbhd_idx, void* d_attn, void* d_value,
                        void* workspace, size_t workspace_bytes, clusten_attn_shape shape, int dtype,
                        clusten_stream stream) {
    if (!d_feat || !attn || !value || !nbhd_idx || !d_attn || !d_value) return CLUSTEN_ERR_NULL_POINTER;
    if (int st = check_attn_call(shape, dtype)) return st;
    if (!strides_ok(d_feat_strides, shape.C) || !strides_ok(value_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    const size_t need = scatter_rows_workspace_bytes(shape, dtype);
    if (need && (!workspace || workspace_bytes < need)) return CLUSTEN_ERR_WORKSPACE;
    // d_attn = gather_dot(d_feat, value)
    int st = launch_gather_dot(d_feat, d_feat_strides, value, value_strides, nbhd_idx, d_attn, shape, dtype,
                               as_stream(stream));
    if (st != CLUSTEN_OK) return st;
    // d_value = scatter_rows(attn, d_feat)
    return launch_scatter_rows(attn, d_feat, d_feat_strides, nbhd_idx, d_value, workspace, shape, dtype,
                               as_stream(stream));
}

int clusten_wf_forward(const void* weights, const void* feat, const int64_t* nbhd_idx, void* feat_new,
                       clusten_wf_shape shape, int dtype, clusten_stream stream) {
    if (!weights || !feat || !nbhd_idx || !feat_new) return CLUSTEN_ERR_NULL_POINTER;
    if (!dtype_ok(dtype)) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_wf_shape(shape)) return st;
    return launch_wf_forward(weights, feat, nbhd_idx, feat_new, shape, dtype, as_stream(stream));
}

int clusten_wf_forward_mixed(const void* weights, const void* feat, int feat_dtype, const int64_t* nbhd_idx, void* feat_new,
                             clusten_wf_shape shape, clusten_stream stream) {
    if (!weights || !feat || !nbhd_idx || !feat_new) return CLUSTEN_ERR_NULL_POINTER;
    if (feat_dtype != CLUSTEN_F16 && feat_dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_wf_shape(shape)) return st;
    return launch_wf_forward_mixed(weights, feat, nbhd_idx, feat_new, shape, feat_dtype, as_stream(stream));
}

size_t clusten_wf_backward_workspace_bytes(clusten_wf_shape shape, int dtype) {
    if (!dtype_ok(dtype) || check_wf_shape(shape) != CLUSTEN_OK) return 0;
    return wf_dfeat_workspace_bytes(shape, dtype);
}

int clusten_wf_backward(const void* d_feat_new, const void* weights, const void* feat, const int64_t* nbhd_idx,
                        void* d_weights, void* d_feat, void* workspace, size_t workspace_bytes, clusten_wf_shape shape,
                        int dtype, clusten_stream stream) {
    if (!d_feat_new || !weights || !feat || !nbhd_idx || !d_weights || !d_feat) return CLUSTEN_ERR_NULL_POINTER;
    if (!dtype_ok(dtype)) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_wf_shape(shape)) return st;
    const size_t need = wf_dfeat_workspace_bytes(shape, dtype);
    if (need && (!workspace || workspace_bytes < need)) return CLUSTEN_ERR_WORKSPACE;
    int st = launch_wf_dweights(d_feat_new, feat, nbhd_idx, d_weights, shape, dtype, as_stream(stream));
    if (st != CLUSTEN_OK) return st;
    return launch_wf_dfeat(d_feat_new, weights, nbhd_idx, d_feat, workspace, shape, dtype, as_stream(stream));
}

int clusten_cluster_size_for(int M) { return cluster_size_for(M); }

int clusten_qk_forward_clusters(const void* query, clusten_strides query_strides, const void* key,
                                clusten_strides key_strides, const int32_t* cluster_idx, void* attn,
                                clusten_attn_shape shape, int dtype, clusten_stream stream) {
    if (!query || !key || !cluster_idx || !attn) return CLUSTEN_ERR_NULL_POINTER;
    if (int st = check_attn_call(shape, dtype)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    return launch_gather_dot_clusters(query, query_strides, key, key_strides, cluster_idx, attn, shape, dtype,
                                      as_stream(stream));
}

int clusten_av_forward_clusters(const void* attn, const void* value, clusten_strides value_strides,
                                const int32_t* cluster_idx, void* feat, clusten_strides feat_strides,
                                clusten_attn_shape shape, int dtype, clusten_stream stream) {
    if (!attn || !value || !cluster_idx || !feat) return CLUSTEN_ERR_NULL_POINTER;
    if (int st = check_attn_call(shape, dtype)) return st;
    if (!strides_ok(value_strides, shape.C) || !strides_ok(feat_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    return launch_gather_sum_clusters(attn, value, value_strides, cluster_idx, feat, feat_strides, shape, dtype,
                                      as_stream(stream));
}

int clusten_attn_softmax_forward(const void* attn, const void* bias_table, const int64_t* pe_idx, const int64_t* mask,
                                 const float* blank_logit, const void* query, clusten_strides query_strides,
                                 const float* blank_key, float* probs, float* blank_prob, clusten_attn_shape shape,
                                 int dtype, clusten_stream stream) {
    if (!attn || !bias_table || !pe_idx || !probs || !blank_prob) return CLUSTEN_ERR_NULL_POINTER;
    if (!blank_logit && !(query && blank_key)) return CLUSTEN_ERR_NULL_POINTER;
    if (query && !strides_ok(query_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (shape.M > 256 || shape.M % 4 != 0) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(attn) || !aligned16(probs)) return CLUSTEN_ERR_UNALIGNED;
    return launch_attn_softmax(attn, bias_table, pe_idx, mask, blank_logit, blank_logit ? nullptr : query, query_strides,
                               blank_key, probs, blank_prob, shape, dtype, as_stream(stream));
}

int clusten_cluster_attention_forward(const void* query, clusten_strides query_strides, const void* key,
                                      clusten_strides key_strides, const void* value, clusten_strides value_strides,
                                      const int32_t* cluster_idx, const void* bias_table, const int64_t* pe_idx,
                                      const int64_t* mask, int lists_shared, const float* blank_key,
                                      const float* blank_value, void* out, clusten_strides out_strides, float scale,
                                      clusten_attn_shape shape, int dtype, clusten_stream stream) {
    if (!query || !key || !value || !cluster_idx || !bias_table || !pe_idx || !blank_key || !blank_value || !out) {
        return CLUSTEN_ERR_NULL_POINTER;
    }
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16 && dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C) || !strides_ok(value_strides, shape.C) ||
        !strides_ok(out_strides, shape.C)) {
        return CLUSTEN_ERR_BAD_STRIDE;
    }
    return launch_cluster_attention(query, query_strides, key, key_strides, value, value_strides, cluster_idx, bias_table,
                                    pe_idx, mask, blank_key, blank_value, out, out_strides, scale, lists_shared != 0, nullptr,
                                    nullptr, shape, dtype, as_stream(stream));
}

size_t clusten_cluster_attention_plan_bytes(int B, int N, int M) {
    if (B <= 0 || N <= 0) return 0;
    return cluster_attention_plan_bytes(B, N, M);
}

int clusten_cluster_attention_plan(const int32_t* cluster_idx, const int64_t* pe_idx, const int64_t* mask, void* plan,
                                   size_t plan_bytes, int B, int N, int M, clusten_stream stream) {
    if (!cluster_idx || !pe_idx || !plan) return CLUSTEN_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || cluster_attention_plan_bytes(1, 8, M) == 0) return CLUSTEN_ERR_BAD_DIMS;
    if (plan_bytes < cluster_attention_plan_bytes(B, N, M)) return CLUSTEN_ERR_WORKSPACE;
    if (!aligned16(plan)) return CLUSTEN_ERR_UNALIGNED;
    return launch_cluster_attention_plan(cluster_idx, pe_idx, mask, plan, B, N, M, as_stream(stream));
}

int clusten_cluster_attention_forward_planned(const void* query, clusten_strides query_strides, const void* key,
                                              clusten_strides key_strides, const void* value,
                                              clusten_strides value_strides, const void* plan, const void* bias_table,
                                              int lists_shared, const float* blank_key, const float* blank_value, void* out,
                                              clusten_strides out_strides, float scale, clusten_attn_shape shape, int dtype,
                                              clusten_stream stream) {
    if (!query || !key || !value || !plan || !bias_table || !blank_key || !blank_value || !out) {
        return CLUSTEN_ERR_NULL_POINTER;
    }
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16 && dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C) || !strides_ok(value_strides, shape.C) ||
        !strides_ok(out_strides, shape.C)) {
        return CLUSTEN_ERR_BAD_STRIDE;
    }
    if (!aligned16(plan)) return CLUSTEN_ERR_UNALIGNED;
    return launch_cluster_attention(query, query_strides, key, key_strides, value, value_strides, nullptr, bias_table,
                                    nullptr, nullptr, blank_key, blank_value, out, out_strides, scale, lists_shared != 0, plan,
                                    nullptr, shape, dtype, as_stream(stream));
}

int clusten_cluster_attention_forward_train(const void* query, clusten_strides query_strides, const void* key,
                                            clusten_strides key_strides, const void* value, clusten_strides value_strides,
                                            const void* plan, const void* bias_table, int lists_shared,
                                            const float* blank_key, const float* blank_value, void* out,
                                            clusten_strides out_strides, float* lse, float scale, clusten_attn_shape shape,
                                            int dtype, clusten_stream stream) {
    if (!query || !key || !value || !plan || !bias_table || !blank_key || !blank_value || !out || !lse) {
        return CLUSTEN_ERR_NULL_POINTER;
    }
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16 && dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C) || !strides_ok(value_strides, shape.C) ||
        !strides_ok(out_strides, shape.C)) {
        return CLUSTEN_ERR_BAD_STRIDE;
    }
    if (!aligned16(plan)) return CLUSTEN_ERR_UNALIGNED;
    return launch_cluster_attention(query, query_strides, key, key_strides, value, value_strides, nullptr, bias_table,
                                    nullptr, nullptr, blank_key, blank_value, out, out_strides, scale, lists_shared != 0, plan,
                                    lse, shape, dtype, as_stream(stream));
}

int clusten_cluster_attention_backward(const void* query, clusten_strides query_strides, const void* key,
                                       clusten_strides key_strides, const void* value, clusten_strides value_strides,
                                       const void* d_out, clusten_strides d_out_strides, const void* out,
                                       clusten_strides out_strides, const float* lse, const void* plan,
                                       const void* bias_table, int lists_shared, const float* blank_key,
                                       const float* blank_value, void* d_query, clusten_strides d_query_strides,
                                       void* probs, void* d_logit, float* blank_prob, float* d_blank_logit, float scale,
                                       clusten_attn_shape shape, int dtype, clusten_stream stream) {
    if (!query || !key || !value || !d_out || !out || !lse || !plan || !bias_table || !blank_key || !blank_value ||
        !d_query || !probs || !d_logit || !blank_prob || !d_blank_logit) {
        return CLUSTEN_ERR_NULL_POINTER;
    }
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16 && dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C) || !strides_ok(value_strides, shape.C) ||
        !strides_ok(d_out_strides, shape.C) || !strides_ok(out_strides, shape.C) || !strides_ok(d_query_strides, shape.C)) {
        return CLUSTEN_ERR_BAD_STRIDE;
    }
    if (!aligned16(plan)) return CLUSTEN_ERR_UNALIGNED;
    return launch_cluster_attention_backward(query, query_strides, key, key_strides, value, value_strides, d_out,
                                             d_out_strides, out, out_strides, lse, nullptr, bias_table, nullptr, nullptr,
                                             blank_key, blank_value, d_query, d_query_strides, probs, d_logit, blank_prob,
                                             d_blank_logit, scale, lists_shared != 0, plan, shape, dtype, as_stream(stream));
}

size_t clusten_cluster_pairs_bytes(int B, int rows, int M, int n_rows) {
    if (!cluster_pairs_supported(B, rows, M, n_rows)) return 0;
    return cluster_pairs_layout(B, rows, M, n_rows).bytes;
}

int clusten_cluster_pairs(const int64_t* nbhd_idx, void* pair_lists, size_t pair_lists_bytes, int B, int rows, int M,
                          int n_rows, clusten_stream stream) {
    if (!nbhd_idx || !pair_lists) return CLUSTEN_ERR_NULL_POINTER;
    if (!cluster_pairs_supported(B, rows, M, n_rows)) return CLUSTEN_ERR_BAD_DIMS;
    const ClusterPairsLayout l = cluster_pairs_layout(B, rows, M, n_rows);
    if (pair_lists_bytes < l.bytes) return CLUSTEN_ERR_WORKSPACE;
    if (!aligned16(pair_lists)) return CLUSTEN_ERR_UNALIGNED;
    char* ws = static_cast<char*>(pair_lists);
    return launch_cluster_pairs(nbhd_idx, reinterpret_cast<int32_t*>(ws + l.keys), reinterpret_cast<int32_t*>(ws + l.wg_bad),
                                reinterpret_cast<int32_t*>(ws + l.flag),
                                reinterpret_cast<int32_t*>(ws + l.pairs), reinterpret_cast<int32_t*>(ws + l.starts),
                                reinterpret_cast<int32_t*>(ws + l.ends), B, rows, M, n_rows, as_stream(stream));
}

int clusten_cluster_pairs_from_numbers(const int32_t* cluster_idx, void* pair_lists, size_t pair_lists_bytes, int B, int rows,
                                       int nnc, int n_rows, clusten_stream stream) {
    if (!cluster_idx || !pair_lists) return CLUSTEN_ERR_NULL_POINTER;
    if (nnc <= 0 || nnc > kPairMaxSlots / 8) return CLUSTEN_ERR_BAD_DIMS;
    const int M = 8 * nnc;
    if (!cluster_pairs_supported(B, rows, M, n_rows)) return CLUSTEN_ERR_BAD_DIMS;
    const ClusterPairsLayout l = cluster_pairs_layout(B, rows, M, n_rows);
    if (pair_lists_bytes < l.bytes) return CLUSTEN_ERR_WORKSPACE;
    if (!aligned16(pair_lists)) return CLUSTEN_ERR_UNALIGNED;
    char* ws = static_cast<char*>(pair_lists);
    return launch_cluster_pairs(nullptr, reinterpret_cast<int32_t*>(ws + l.keys), reinterpret_cast<int32_t*>(ws + l.wg_bad),
                                reinterpret_cast<int32_t*>(ws + l.flag), reinterpret_cast<int32_t*>(ws + l.pairs),
                                reinterpret_cast<int32_t*>(ws + l.starts), reinterpret_cast<int32_t*>(ws + l.ends), B, rows, M,
                                n_rows, as_stream(stream), cluster_idx);
}

int clusten_wf_backward_by_cluster(const void* d_feat_new, const void* weights, const void* feat, const int64_t* nbhd_idx,
                                   const void* pair_lists, void* d_weights, void* d_feat, clusten_wf_shape shape, int dtype,
                                   clusten_stream stream) {
    if (!d_feat_new || !weights || !feat || !nbhd_idx || !pair_lists || !d_weights || !d_feat) {
        return CLUSTEN_ERR_NULL_POINTER;
    }
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_wf_shape(shape)) return st;
    if (!cluster_pairs_supported(shape.B, shape.Nout, shape.M, shape.N)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(pair_lists)) return CLUSTEN_ERR_UNALIGNED;
    int st = launch_wf_dweights(d_feat_new, feat, nbhd_idx, d_weights, shape, dtype, as_stream(stream));
    if (st != CLUSTEN_OK) return st;
    const ClusterPairsLayout l = cluster_pairs_layout(shape.B, shape.Nout, shape.M, shape.N);
    const char* ws = static_cast<const char*>(pair_lists);
    return launch_wf_dfeat_by_cluster(d_feat_new, weights, reinterpret_cast<const int32_t*>(ws + l.starts),
                                      reinterpret_cast<const int32_t*>(ws + l.ends),
                                      reinterpret_cast<const int32_t*>(ws + l.pairs),
                                      reinterpret_cast<const int32_t*>(ws + l.flag), d_feat, shape, dtype, as_stream(stream));
}

int clusten_scatter_rows_by_cluster(const void* p, const void* x, clusten_strides x_strides, const void* pair_lists, void* y,
                                    clusten_attn_shape shape, int dtype, clusten_stream stream) {
    if (!p || !x || !pair_lists || !y) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(x_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    if (!cluster_pairs_supported(shape.B, shape.N, shape.M, shape.N)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(pair_lists)) return CLUSTEN_ERR_UNALIGNED;
    const ClusterPairsLayout l = cluster_pairs_layout(shape.B, shape.N, shape.M, shape.N);
    const char* ws = static_cast<const char*>(pair_lists);
    return launch_scatter_by_cluster(p, x, x_strides, reinterpret_cast<const int32_t*>(ws + l.starts),
                                     reinterpret_cast<const int32_t*>(ws + l.ends),
                                     reinterpret_cast<const int32_t*>(ws + l.pairs),
                                     reinterpret_cast<const int32_t*>(ws + l.flag), y, shape, dtype, as_stream(stream));
}

size_t clusten_scatter_rows_workspace_bytes(clusten_attn_shape shape, int dtype) {
    if (!dtype_ok(dtype) || check_attn_shape(shape) != CLUSTEN_OK) return 0;
    return scatter_rows_workspace_bytes(shape, dtype);
}

int clusten_scatter_rows(const void* p, const void* x, clusten_strides x_strides, const int64_t* nbhd_idx,
                         const void* pair_lists, void* y, void* workspace, size_t workspace_bytes,
                         clusten_attn_shape shape, int dtype, clusten_stream stream) {
    if (!p || !x || !nbhd_idx || !y) return CLUSTEN_ERR_NULL_POINTER;
    if (int st = check_attn_call(shape, dtype)) return st;
    if (!strides_ok(x_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    const size_t need = scatter_rows_workspace_bytes(shape, dtype);
    if (need && (!workspace || workspace_bytes < need)) return CLUSTEN_ERR_WORKSPACE;
    if (pair_lists) {
        if (!cluster_pairs_supported(shape.B, shape.N, shape.M, shape.N)) return CLUSTEN_ERR_BAD_DIMS;
        if (!aligned16(pair_lists)) return CLUSTEN_ERR_UNALIGNED;
    }
    return launch_scatter_rows(p, x, x_strides, nbhd_idx, y, workspace, shape, dtype, as_stream(stream), pair_lists);
}

int clusten_dense_attention_forward(const void* query, clusten_strides query_strides, const void* key,
                                    clusten_strides key_strides, const void* value, clusten_strides value_strides,
                                    const void* bias_table, const int64_t* pe_idx, const float* blank_key,
                                    const float* blank_value, void* out, clusten_strides out_strides, float scale,
                                    clusten_attn_shape shape, int dtype, clusten_stream stream) {
    if (!query || !key || !value || !bias_table || !pe_idx || !blank_key || !blank_value || !out) {
        return CLUSTEN_ERR_NULL_POINTER;
    }
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C) || !strides_ok(value_strides, shape.C) ||
        !strides_ok(out_strides, shape.C)) {
        return CLUSTEN_ERR_BAD_STRIDE;
    }
    return launch_dense_attention(query, query_strides, key, key_strides, value, value_strides, bias_table, pe_idx,
                                  blank_key, blank_value, out, out_strides, scale, shape, dtype, as_stream(stream));
}

int clusten_linear_supported(int K, int Nout, int act) { return skinny_linear_supported(K, Nout, act) ? 1 : 0; }

int clusten_linear_forward(const void* x, int64_t x_row_stride, const void* weight, const void* bias, void* out,
                           int64_t rows, int K, int Nout, int act, int dtype, clusten_stream stream) {
    if (!x || !weight || !out) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (rows <= 0 || !skinny_linear_supported(K, Nout, act)) return CLUSTEN_ERR_BAD_DIMS;
    if (x_row_stride < K || 16 * x_row_stride * 2 >= ((int64_t)1 << 32)) return CLUSTEN_ERR_BAD_STRIDE;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(out) || (x_row_stride & 7) != 0) return CLUSTEN_ERR_UNALIGNED;
    if (bias && !aligned16(bias)) return CLUSTEN_ERR_UNALIGNED;
    return launch_skinny_linear(x, x_row_stride, weight, bias, out, rows, K, Nout, act, dtype, as_stream(stream));
}

int clusten_layer_norm_forward(const void* x, int in_dtype, const float* weight, const float* bias, void* out,
                               int64_t rows, int C, float eps, int out_dtype, clusten_stream stream) {
    if (!x || !weight || !bias || !out) return CLUSTEN_ERR_NULL_POINTER;
    if (out_dtype != CLUSTEN_F32 && out_dtype != CLUSTEN_F16 && out_dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (in_dtype != CLUSTEN_F32 && in_dtype != CLUSTEN_F16 && in_dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (rows <= 0 || C <= 0 || (rows + 3) / 4 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(bias) || !aligned16(out)) return CLUSTEN_ERR_UNALIGNED;
    return launch_layer_norm(x, in_dtype, weight, bias, out, rows, C, eps, out_dtype, as_stream(stream));
}

int clusten_layer_norm_rows_forward(const void* x, int in_dtype, const int64_t* order, int group, const void* pre_bias,
                                    const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
                                    int out_dtype, clusten_stream stream) {
    if (!x || !weight || !bias || !out) return CLUSTEN_ERR_NULL_POINTER;
    if (out_dtype != CLUSTEN_F32 && out_dtype != CLUSTEN_F16 && out_dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (in_dtype != CLUSTEN_F32 && in_dtype != CLUSTEN_F16 && in_dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (rows <= 0 || C <= 0 || (rows + 3) / 4 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if (order && (group <= 0 || rows % group != 0)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(bias) || !aligned16(out) || (pre_bias && !aligned16(pre_bias))) {
        return CLUSTEN_ERR_UNALIGNED;
    }
    return launch_layer_norm_rows(x, in_dtype, order, order ? group : 1, pre_bias, weight, bias, out, rows, C, eps,
                                  out_dtype, as_stream(stream));
}

int clusten_channel_affine_gelu_forward(const void* x, const float* scale, const float* shift, void* y, int64_t B, int C,
                                        int HW, int dtype, clusten_stream stream) {
    if (!x || !scale || !shift || !y) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (B <= 0 || C <= 0 || HW <= 0 || HW % 8 != 0) return CLUSTEN_ERR_BAD_DIMS;
    if (B * C >= 65536) return CLUSTEN_ERR_BAD_DIMS;  // one grid row per (image, channel) plane
    if (!aligned16(x) || !aligned16(y)) return CLUSTEN_ERR_UNALIGNED;
    return launch_channel_affine_gelu(x, scale, shift, y, B, C, HW, dtype, as_stream(stream));
}

int clusten_add_layer_norm_forward(const void* x, int x_dtype, const void* branch, int branch_dtype, void* sum_out,
                                   const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
                                   clusten_stream stream) {
    if (!x || !branch || !sum_out || !weight || !bias || !out) return CLUSTEN_ERR_NULL_POINTER;
    if (branch_dtype != CLUSTEN_F16 && branch_dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (x_dtype != CLUSTEN_F32 && x_dtype != branch_dtype) return CLUSTEN_ERR_BAD_DTYPE;
    if (rows <= 0 || C <= 0 || (rows + 3) / 4 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(x) || !aligned16(branch) || !aligned16(sum_out) || !aligned16(weight) || !aligned16(bias) ||
        !aligned16(out)) {
        return CLUSTEN_ERR_UNALIGNED;
    }
    return launch_add_layer_norm(x, x_dtype, branch, branch_dtype, sum_out, weight, bias, out, rows, C, eps,
                                 as_stream(stream));
}

int clusten_neighbour_lists(const float* pos, const int64_t* nearest, int64_t* member_idx, int64_t* mask,
                            int64_t* pe_idx, int32_t* cluster_idx, int B, int N, int nnc, int m, int radius,
                            int table_width, clusten_stream stream) {
    if (!pos || !nearest || !member_idx || !pe_idx) return CLUSTEN_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || nnc <= 0 || m <= 0 || table_width <= 0) return CLUSTEN_ERR_BAD_DIMS;
    if (((int64_t)B * N * nnc * m + 255) / 256 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if ((reinterpret_cast<uintptr_t>(pos) & 7) != 0) return CLUSTEN_ERR_UNALIGNED;
    return launch_neighbour_lists(pos, nearest, member_idx, mask, pe_idx, cluster_idx, B, N, nnc, m, radius, table_width,
                                  as_stream(stream));
}

int clusten_add_row_score_forward(const void* x, int x_dtype, const void* branch, void* sum_out, const void* weight,
                                  const void* bias, void* score, int64_t rows, int C, int dtype,
                                  clusten_stream stream) {
    if (!x || !weight || !score || (branch && !sum_out)) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (x_dtype != CLUSTEN_F32 && x_dtype != dtype) return CLUSTEN_ERR_BAD_DTYPE;
    if (rows <= 0 || (rows + 3) / 4 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(x) || !aligned16(weight) || (branch && (!aligned16(branch) || !aligned16(sum_out)))) {
        return CLUSTEN_ERR_UNALIGNED;
    }
    return launch_add_row_score(x, x_dtype, branch, sum_out, weight, bias, score, rows, C, dtype, as_stream(stream));
}

int clusten_attn_softmax_backward(const float* probs, const float* blank_prob, const float* d_probs,
                                  const float* d_blank_prob, void* d_logit, float* d_blank_logit, int64_t rows, int M,
                                  int dtype, clusten_stream stream) {
    if (!probs || !blank_prob || !d_probs || !d_blank_prob || !d_logit || !d_blank_logit) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (rows <= 0 || M <= 0 || M > 256 || M % 4 != 0 || (rows + 3) / 4 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(probs) || !aligned16(d_probs) || !aligned16(d_logit)) return CLUSTEN_ERR_UNALIGNED;
    return launch_attn_softmax_backward(probs, blank_prob, d_probs, d_blank_prob, d_logit, d_blank_logit, rows, M, dtype,
                                        as_stream(stream));
}

int clusten_bias_table_grad(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int N, int M,
                            int rows, int dtype, clusten_stream stream) {
    if (!d_logit || !pe_idx || !d_table) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F32 && dtype != CLUSTEN_F16 && dtype != CLUSTEN_BF16) return CLUSTEN_ERR_BAD_DTYPE;
    if (B <= 0 || H <= 0 || H > 65535 || N <= 0 || M <= 0 || rows <= 0) return CLUSTEN_ERR_BAD_DIMS;
    return launch_bias_table_grad(d_logit, pe_idx, d_table, B, H, N, M, rows, dtype, as_stream(stream));
}

int clusten_merge_weights_forward(const float* table_weights, const int64_t* pe_idx, const int64_t* nbhd_idx,
                                  const float* prob, const int64_t* mask, float* weights, int B, int N, int Nout, int M,
                                  int IC, clusten_stream stream) {
    if (!table_weights || !pe_idx || !weights) return CLUSTEN_ERR_NULL_POINTER;
    if (prob && !nbhd_idx) return CLUSTEN_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || Nout <= 0 || M <= 0 || IC != 4) return CLUSTEN_ERR_BAD_DIMS;
    if (((int64_t)B * Nout * M + 255) / 256 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(table_weights) || !aligned16(weights)) return CLUSTEN_ERR_UNALIGNED;
    return launch_merge_weights(table_weights, pe_idx, nbhd_idx, prob, mask, weights, B, N, Nout, M, as_stream(stream));
}

size_t clusten_scanline_rank_workspace_bytes(int B, int N) {
    if (B <= 0 || N <= 0) return 0;
    return scanline_rank_workspace_bytes(B, N);
}

int clusten_scanline_rank(const float* pos, int64_t* ranking, void* workspace, size_t workspace_bytes, int B, int N,
                          int rows, int cols, float cell_w, float cell_h, clusten_stream stream) {
    if (!pos || !ranking || !workspace) return CLUSTEN_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || N > scanline_rank_max_tokens() || rows <= 0 || cols <= 0 || (int64_t)rows * cols < 2 ||
        (int64_t)rows * cols >= ((int64_t)1 << 24) || !(cell_w > 0.f) || !(cell_h > 0.f)) {
        return CLUSTEN_ERR_BAD_DIMS;
    }
    if (workspace_bytes < scanline_rank_workspace_bytes(B, N)) return CLUSTEN_ERR_WORKSPACE;
    if (!aligned16(workspace) || (reinterpret_cast<uintptr_t>(pos) & 7u) != 0) return CLUSTEN_ERR_UNALIGNED;
    return launch_scanline_rank(pos, ranking, workspace, B, N, rows, cols, cell_w, cell_h, as_stream(stream));
}

int clusten_scanline_rank_max_tokens(void) { return scanline_rank_max_tokens(); }

int clusten_cluster_centres(const float* pos, const int64_t* ranking, float* pos_sorted, float* centres, int B, int N, int m,
                            clusten_stream stream) {
    if (!pos || !ranking || !centres) return CLUSTEN_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || m <= 0 || (int64_t)B * ((N + m - 1) / m) >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if ((reinterpret_cast<uintptr_t>(pos) & 7u) != 0 || (reinterpret_cast<uintptr_t>(centres) & 7u) != 0 ||
        (reinterpret_cast<uintptr_t>(pos_sorted) & 7u) != 0) {
        return CLUSTEN_ERR_UNALIGNED;
    }
    return launch_cluster_centres(pos, ranking, pos_sorted, centres, B, N, m, as_stream(stream));
}

int clusten_gather_rows(const void* x, const int64_t* order, void* out, int64_t B, int N, int row_bytes, int order_shared,
                        clusten_stream stream) {
    if (!x || !order || !out) return CLUSTEN_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || row_bytes <= 0 || row_bytes % 16 != 0) return CLUSTEN_ERR_BAD_DIMS;
    if ((B * N * (row_bytes / 16) + 255) / 256 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    if (!aligned16(x) || !aligned16(out)) return CLUSTEN_ERR_UNALIGNED;
    return launch_gather_rows(x, order, out, B, N, row_bytes, order_shared, as_stream(stream));
}

int clusten_merge_centres_max_tokens(void) { return merge_centres_max_tokens(); }

int clusten_merge_centres(const float* pos, const float* min_dist, const void* learned_prob, int prob_dtype,
                          int64_t* centre, int B, int N, int sample_num, int reserve_num, int reserve_on, float alpha,
                          int stride, clusten_stream stream) {
    if (!pos || !centre) return CLUSTEN_ERR_NULL_POINTER;
    if (learned_prob && prob_dtype != CLUSTEN_F32 && prob_dtype != CLUSTEN_F16 && prob_dtype != CLUSTEN_BF16)
        return CLUSTEN_ERR_BAD_DTYPE;
    if (!(reinterpret_cast<uintptr_t>(pos) % 8 == 0)) return CLUSTEN_ERR_UNALIGNED;
    return launch_merge_centres(pos, min_dist, learned_prob, learned_prob ? prob_dtype : CLUSTEN_F32, centre, B, N,
                                sample_num, reserve_num, reserve_on, alpha, stride, as_stream(stream));
}

int clusten_merge_rows(const void* const* src, void* const* dst, const int* row_bytes, int count, const int64_t* centre,
                       int64_t B, int N, int n_out, clusten_stream stream) {
    if (!src || !dst || !row_bytes || !centre) return CLUSTEN_ERR_NULL_POINTER;
    if (count < 1 || count > 4 || B <= 0 || N <= 0 || n_out <= 0) return CLUSTEN_ERR_BAD_DIMS;
    int64_t words = 0;
    for (int t = 0; t < count; ++t) words += row_bytes[t] / 8;
    if ((B * n_out * words + 255) / 256 >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    return launch_merge_rows(src, dst, row_bytes, count, centre, B, N, n_out, as_stream(stream));
}

int clusten_knn2d(const float* query, const float* database, int64_t* idx, float* dist, int B, int Nq, int N, int K,
                  clusten_stream stream) {
    if (!query || !database || !idx) return CLUSTEN_ERR_NULL_POINTER;
    if (B <= 0 || Nq <= 0 || N <= 0 || K < 1 || K > 8 || K > N) return CLUSTEN_ERR_BAD_DIMS;
    if ((int64_t)B * ((Nq + 255) / 256) >= ((int64_t)1 << 31)) return CLUSTEN_ERR_BAD_DIMS;
    return launch_knn2d(query, database, idx, dist, B, Nq, N, K, as_stream(stream));
}

}  // extern "C"
