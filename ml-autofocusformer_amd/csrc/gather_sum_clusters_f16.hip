// gather_sum kernels for lists given as cluster numbers, f16_t storage (see gather_sum_impl.hpp).
#include "gather_sum_impl.hpp"

namespace clusten {

int gather_sum_clusters_f16(const void* p, const void* rows, clusten_strides rs, const int32_t* cluster_idx, void* out,
                           clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    return gather_sum_clusters_typed<f16_t>(p, rows, rs, cluster_idx, out, os, s, stream);
}

}  // namespace clusten
