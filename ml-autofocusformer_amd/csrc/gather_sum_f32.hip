// gather_sum kernels for float storage (see gather_sum_impl.hpp).
#include "gather_sum_impl.hpp"

namespace clusten {

int gather_sum_f32(const void* p, const void* rows, clusten_strides rs, const int64_t* idx, void* out,
                   clusten_strides os, const clusten_attn_shape& s, hipStream_t stream) {
    return gather_sum_typed<float>(p, rows, rs, idx, out, os, s, stream);
}

}  // namespace clusten
