// clusten_av_forward_replay: the AV forward kernels without their arithmetic (see replay_qk.hip).
#define CLUSTEN_REPLAY 1
#define clusten clusten_replay   // the kernels of this file are other functions than the library's own
#include "../gather_sum_impl.hpp"

extern "C" int clusten_av_forward_replay(const void* attn, const void* value, clusten_strides value_strides,
                                         const int64_t* nbhd_idx, void* feat, clusten_strides feat_strides,
                                         clusten_attn_shape shape, int dtype, clusten_stream stream) {
    using namespace clusten_replay;
    if (!attn || !value || !nbhd_idx || !feat) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(value_strides, shape.C) || !strides_ok(feat_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    return gather_sum_typed<float>(attn, value, value_strides, nbhd_idx, feat, feat_strides, shape,
                                   static_cast<hipStream_t>(stream));
}
