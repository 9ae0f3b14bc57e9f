// gather_dot kernels for f16_t storage (see gather_dot_impl.hpp).
#include "gather_dot_impl.hpp"

namespace clusten {

int gather_dot_f16(const void* a, clusten_strides as, const void* rows, clusten_strides rs, const int64_t* idx,
                   void* out, const clusten_attn_shape& s, hipStream_t stream) {
    return gather_dot_typed<f16_t>(a, as, rows, rs, idx, out, s, stream);
}

}  // namespace clusten
