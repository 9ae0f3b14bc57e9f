// WF forward kernels for fp32 weights over bf16 features (see wf_impl.hpp).
#include "wf_impl.hpp"

namespace clusten {

int wf_forward_mixed_bf16(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                         hipStream_t stream) {
    return wf_forward_mixed_typed<bf16_t>(w, feat, idx, out, s, stream);
}

}  // namespace clusten
