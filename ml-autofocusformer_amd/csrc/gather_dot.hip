// Storage-type dispatch for gather_dot (see gather_dot_impl.hpp) and its fp64 instantiation.
#include "gather_dot_impl.hpp"

namespace clusten {

int gather_dot_f32(const void*, clusten_strides, const void*, clusten_strides, const int64_t*, void*,
                   const clusten_attn_shape&, hipStream_t);
int gather_dot_f16(const void*, clusten_strides, const void*, clusten_strides, const int64_t*, void*,
                   const clusten_attn_shape&, hipStream_t);
int gather_dot_bf16(const void*, clusten_strides, const void*, clusten_strides, const int64_t*, void*,
                    const clusten_attn_shape&, hipStream_t);

int gather_dot_clusters_f32(const void*, clusten_strides, const void*, clusten_strides, const int32_t*, void*,
                            const clusten_attn_shape&, hipStream_t);
int gather_dot_clusters_f16(const void*, clusten_strides, const void*, clusten_strides, const int32_t*, void*,
                            const clusten_attn_shape&, hipStream_t);
int gather_dot_clusters_bf16(const void*, clusten_strides, const void*, clusten_strides, const int32_t*, void*,
                             const clusten_attn_shape&, hipStream_t);

int cluster_size_for(int M) {
    if (M > 0 && M <= 64 && M % 8 == 0) return 8;
    return runs_length_for(M);
}

int launch_gather_dot_clusters(const void* a, clusten_strides as, const void* rows, clusten_strides rs,
                               const int32_t* cluster_idx, void* out, clusten_attn_shape s, int dtype,
                               hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return gather_dot_clusters_f32(a, as, rows, rs, cluster_idx, out, s, stream);
        case CLUSTEN_F16: return gather_dot_clusters_f16(a, as, rows, rs, cluster_idx, out, s, stream);
        case CLUSTEN_BF16: return gather_dot_clusters_bf16(a, as, rows, rs, cluster_idx, out, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int launch_gather_dot(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx,
                      void* out, clusten_attn_shape s, int dtype, hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return gather_dot_f32(a, as, rows, rs, idx, out, s, stream);
        case CLUSTEN_F16: return gather_dot_f16(a, as, rows, rs, idx, out, s, stream);
        case CLUSTEN_BF16: return gather_dot_bf16(a, as, rows, rs, idx, out, s, stream);
        case CLUSTEN_F64: return launch_elem<double>(a, as, rows, rs, idx, out, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
