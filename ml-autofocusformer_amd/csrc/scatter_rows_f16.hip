// scatter_rows kernels for f16_t storage (see scatter_rows_impl.hpp).
#include "scatter_rows_impl.hpp"

namespace clusten {

int scatter_rows_f16(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32,
                     const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if, const uint8_t* handled) {
    return scatter_rows_typed<f16_t>(p, x, xs, idx, acc32, s, stream, only_if, handled);
}

}  // namespace clusten
