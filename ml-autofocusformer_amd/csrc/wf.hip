// Storage-type dispatch for the WF kernels (see wf_impl.hpp) and their fp64 instantiations.
#include "wf_impl.hpp"

namespace clusten {

int wf_forward_f32(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);
int wf_forward_f16(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);
int wf_forward_bf16(const void*, const void*, const int64_t*, void*, const clusten_wf_shape&, hipStream_t);

int launch_wf_forward(const void* w, const void* feat, const int64_t* idx, void* out, clusten_wf_shape s, int dtype,
                      hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return wf_forward_f32(w, feat, idx, out, s, stream);
        case CLUSTEN_F16: return wf_forward_f16(w, feat, idx, out, s, stream);
        case CLUSTEN_BF16: return wf_forward_bf16(w, feat, idx, out, s, stream);
        case CLUSTEN_F64: return wf_forward_elem<double>(w, feat, idx, out, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

int launch_wf_dweights(const void* d_out, const void* feat, const int64_t* idx, void* d_w, clusten_wf_shape s,
                       int dtype, hipStream_t stream) {
    switch (dtype) {
        case CLUSTEN_F32: return wf_dweights_typed<float>(d_out, feat, idx, d_w, s, stream);
        case CLUSTEN_F16: return wf_dweights_typed<f16_t>(d_out, feat, idx, d_w, s, stream);
        case CLUSTEN_BF16: return wf_dweights_typed<bf16_t>(d_out, feat, idx, d_w, s, stream);
        case CLUSTEN_F64: return wf_dweights_typed<double>(d_out, feat, idx, d_w, s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

size_t wf_dfeat_workspace_bytes(clusten_wf_shape s, int dtype) {
    if (dtype == CLUSTEN_F16 || dtype == CLUSTEN_BF16) return (size_t)s.B * s.N * s.C * sizeof(float);
    return 0;
}

int launch_wf_dfeat(const void* d_out, const void* w, const int64_t* idx, void* d_feat, void* workspace,
                    clusten_wf_shape s, int dtype, hipStream_t stream) {
    const size_t count = (size_t)s.B * s.N * s.C;
    int st;
    switch (dtype) {
        case CLUSTEN_F32:
            st = launch_zero_f32(static_cast<float*>(d_feat), count, stream);
            if (st != CLUSTEN_OK) return st;
            return wf_dfeat_typed<float, float>(d_out, w, idx, static_cast<float*>(d_feat), s, stream);
        case CLUSTEN_F16:
        case CLUSTEN_BF16: {
            float* acc32 = static_cast<float*>(workspace);
            st = launch_zero_f32(acc32, count, stream);
            if (st != CLUSTEN_OK) return st;
            st = dtype == CLUSTEN_F16 ? wf_dfeat_typed<f16_t, float>(d_out, w, idx, acc32, s, stream)
                                      : wf_dfeat_typed<bf16_t, float>(d_out, w, idx, acc32, s, stream);
            if (st != CLUSTEN_OK) return st;
            return launch_round_from_f32(acc32, d_feat, count, dtype, stream);
        }
        case CLUSTEN_F64:
            st = launch_zero_f64(static_cast<double*>(d_feat), count, stream);
            if (st != CLUSTEN_OK) return st;
            return wf_dfeat_typed<double, double>(d_out, w, idx, static_cast<double*>(d_feat), s, stream);
        default: return CLUSTEN_ERR_BAD_DTYPE;
    }
}

}  // namespace clusten
