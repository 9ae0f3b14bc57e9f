// WF forward kernels for bf16_t storage (see wf_impl.hpp).
#include "wf_impl.hpp"

namespace clusten {

int wf_forward_bf16(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    return wf_forward_typed<bf16_t>(w, feat, idx, out, s, stream);
}

}  // namespace clusten
