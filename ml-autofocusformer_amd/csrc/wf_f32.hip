// WF forward kernels for float storage (see wf_impl.hpp).
#include "wf_impl.hpp"

namespace clusten {

int wf_forward_f32(const void* w, const void* feat, const int64_t* idx, void* out, const clusten_wf_shape& s,
                   hipStream_t stream) {
    return wf_forward_typed<float>(w, feat, idx, out, s, stream);
}

}  // namespace clusten
