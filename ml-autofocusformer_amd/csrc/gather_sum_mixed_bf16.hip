// gather_sum kernels for fp32 weights over bf16 rows (see gather_sum_impl.hpp).
#include "gather_sum_impl.hpp"

namespace clusten {

int gather_sum_mixed_bf16(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                          clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    return gather_sum_mixed_typed<bf16_t>(p, rows, rs, idx, out, os, s, stream);
}

}  // namespace clusten
