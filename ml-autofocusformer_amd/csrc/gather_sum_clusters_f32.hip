// gather_sum kernels for lists given as cluster numbers, float storage (see gather_sum_impl.hpp).
#include "gather_sum_impl.hpp"

namespace clusten {

int gather_sum_clusters_f32(const void* p, const void* rows, clusten_strides rs, const int32_t* cluster_idx, void* out,
                           clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    return gather_sum_clusters_typed<float>(p, rows, rs, cluster_idx, out, os, s, stream);
}

}  // namespace clusten
