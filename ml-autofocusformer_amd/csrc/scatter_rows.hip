// Storage-type dispatch for scatter_rows (see scatter_rows_impl.hpp): zeroes the fp32 accumulation
// buffer, runs the scatter, and rounds to fp16/bf16 when the storage type is narrower than fp32.
#include "scatter_rows_impl.hpp"

namespace clusten {

int scatter_rows_f32(const void*, const void*, clusten_strides, const int64_t*, float*, const clusten_attn_shape&, hipStream_t);
int scatter_rows_f16(const void*, const void*, clusten_strides, const int64_t*, float*, const clusten_attn_shape&, hipStream_t);
int scatter_rows_bf16(const void*, const void*, clusten_strides, const int64_t*, float*, const clusten_attn_shape&, hipStream_t);

size_t scatter_rows_workspace_bytes(clusten_attn_shape s, int dtype) {
    if (dtype == CLUSTEN_F16 || dtype == CLUSTEN_BF16) return (size_t)s.B * s.H * s.N * s.C * sizeof(float);
    return 0;
}

int launch_scatter_rows(const void* p, const void* x, clusten_strides xs, const int64_t* idx, void* out,
                        void* workspace, clusten_attn_shape s, int dtype, hipStream_t stream) {
    const size_t count = (size_t)s.B * s.H * s.N * s.C;
    int st;
    switch (dtype) {
        case CLUSTEN_F32:
            st = launch_zero_f32(static_cast<float*>(out), count, stream);
            if (st != CLUSTEN_OK) return st;
            return scatter_rows_f32(p, x, xs, idx, static_cast<float*>(out), s, stream);
        case CLUSTEN_F16:
        case CLUSTEN_BF16: {
            float* acc32 = static_cast<float*>(workspace);
            st = launch_zero_f32(acc32, count, stream);
            if (st != CLUSTEN_OK) return st;
            st = dtype == CLUSTEN_F16 ? scatter_rows_f16(p, x, xs, idx, acc32, s, stream)
                                      : scatter_rows_bf16(p, x, xs, idx, acc32, s, stream);
            if (st != CLUSTEN_OK) return st;
            return launch_round_from_f32(acc32, out, count, dtype, stream);
        }
        case CLUSTEN_F64:
            st = launch_zero_f64(static_cast<double*>(out), count, stream);
            if (st != CLUSTEN_OK) return st;
            return scatter_elem<double, double>(p, x, xs, idx, static_cast<double*>(out), s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
