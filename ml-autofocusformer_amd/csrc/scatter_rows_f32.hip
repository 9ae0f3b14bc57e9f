// scatter_rows kernels for float storage (see scatter_rows_impl.hpp).
#include "scatter_rows_impl.hpp"

namespace clusten {

int scatter_rows_f32(const void* p, const void* x, clusten_strides xs, const int64_t* idx, float* acc32,
                     const clusten_attn_shape& s, hipStream_t stream, const int32_t* only_if, const uint8_t* handled) {
    return scatter_rows_typed<float>(p, x, xs, idx, acc32, s, stream, only_if, handled);
}

}  // namespace clusten
