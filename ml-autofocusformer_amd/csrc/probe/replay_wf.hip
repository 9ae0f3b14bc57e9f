// clusten_wf_forward_replay: the WF forward kernels without their arithmetic (see replay_qk.hip).
#define CLUSTEN_REPLAY 1
#define clusten clusten_replay   // the kernels of this file are other functions than the library's own
#include "../wf_impl.hpp"

extern "C" int clusten_wf_forward_replay(const void* weights, const void* feat, const int64_t* nbhd_idx, void* feat_new,
                                         clusten_wf_shape shape, int dtype, clusten_stream stream) {
    using namespace clusten_replay;
    if (!weights || !feat || !nbhd_idx || !feat_new) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_wf_shape(shape)) return st;
    return wf_forward_typed<float>(weights, feat, nbhd_idx, feat_new, shape, static_cast<hipStream_t>(stream));
}
