// Storage-type dispatch for gather_sum (see gather_sum_impl.hpp) and its fp64 instantiation.
#include "gather_sum_impl.hpp"

namespace clusten {

int gather_sum_f32(const void*, const void*, clusten_strides, const int64_t*, void*, clusten_strides,
                    const clusten_attn_shape&, hipStream_t);
int gather_sum_f16(const void*, const void*, clusten_strides, const int64_t*, void*, clusten_strides,
                    const clusten_attn_shape&, hipStream_t);
int gather_sum_bf16(const void*, const void*, clusten_strides, const int64_t*, void*, clusten_strides,
                    const clusten_attn_shape&, hipStream_t);

int gather_sum_clusters_f32(const void*, const void*, clusten_strides, const int32_t*, void*, clusten_strides,
                            const clusten_attn_shape&, hipStream_t);
int gather_sum_clusters_f16(const void*, const void*, clusten_strides, const int32_t*, void*, clusten_strides,
                            const clusten_attn_shape&, hipStream_t);
int gather_sum_clusters_bf16(const void*, const void*, clusten_strides, const int32_t*, void*, clusten_strides,
                             const clusten_attn_shape&, hipStream_t);

int launch_gather_sum_clusters(const void* p, const void* rows, clusten_strides rs, const int32_t* cluster_idx, void* out,
                               clusten_strides os, clusten_attn_shape s, int dtype, hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return gather_sum_clusters_f32(p, rows, rs, cluster_idx, out, os, s, stream);
        case CLUSTEN_F16: return gather_sum_clusters_f16(p, rows, rs, cluster_idx, out, os, s, stream);
        case CLUSTEN_BF16: return gather_sum_clusters_bf16(p, rows, rs, cluster_idx, out, os, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int gather_sum_mixed_f16(const void*, const void*, clusten_strides, const int64_t*, void*, clusten_strides,
                         const clusten_attn_shape&, hipStream_t);
int gather_sum_mixed_bf16(const void*, const void*, clusten_strides, const int64_t*, void*, clusten_strides,
                          const clusten_attn_shape&, hipStream_t);

int launch_gather_sum_mixed(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                            clusten_strides os, clusten_attn_shape s, int rows_dtype, hipStream_t stream) {
    switch (rows_dtype) {
        case CLUSTEN_F16: return gather_sum_mixed_f16(p, rows, rs, idx, out, os, s, stream);
        case CLUSTEN_BF16: return gather_sum_mixed_bf16(p, rows, rs, idx, out, os, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int launch_gather_sum(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                      clusten_strides os, clusten_attn_shape s, int dtype, hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return gather_sum_f32(p, rows, rs, idx, out, os, s, stream);
        case CLUSTEN_F16: return gather_sum_f16(p, rows, rs, idx, out, os, s, stream);
        case CLUSTEN_BF16: return gather_sum_bf16(p, rows, rs, idx, out, os, s, stream);
        case CLUSTEN_F64: return launch_elem<double>(p, rows, rs, idx, out, os, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
