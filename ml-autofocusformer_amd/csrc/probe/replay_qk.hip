// clusten_qk_forward_replay: the QK forward kernels compiled a second time with their matrix instructions replaced
// by one integer operation each (CLUSTEN_REPLAY, see mfma.hpp) — the same loads, LDS traffic and stores in the same
// order, no arithmetic.  A measurement aid: the time of this kernel is what the memory instruction stream of
// clusten_qk_forward costs by itself.  The output holds no meaningful values.
#define CLUSTEN_REPLAY 1
#define clusten clusten_replay   // the kernels of this file are other functions than the library's own
#include "../gather_dot_impl.hpp"

extern "C" int clusten_qk_forward_replay(const void* query, clusten_strides query_strides, const void* key,
                                         clusten_strides key_strides, const int64_t* nbhd_idx, void* attn,
                                         clusten_attn_shape shape, int dtype, clusten_stream stream) {
    using namespace clusten_replay;
    if (!query || !key || !nbhd_idx || !attn) return CLUSTEN_ERR_NULL_POINTER;
    if (dtype != CLUSTEN_F32) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    return gather_dot_typed<float>(query, query_strides, key, key_strides, nbhd_idx, attn, shape,
                                   static_cast<hipStream_t>(stream));
}
