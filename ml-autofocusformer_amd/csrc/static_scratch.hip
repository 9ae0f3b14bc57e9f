// clusten_qk_backward_static: clusten_qk_backward for callers that cannot allocate device memory (code under HIP
// graph capture, serving loops, harnesses that forbid hipMalloc) and therefore have no workspace to hand over.
// The fp32 accumulation buffer the scatter of 16-bit gradients needs lives in a file-scope device array of
// CLUSTEN_STATIC_SCRATCH_BYTES instead; the kernels are the ones clusten_qk_backward launches and take the array's
// device address as their workspace argument.
//
// The array's name is only a host-side handle.  Its address on a device comes from hipGetSymbolAddress, asked once
// per device with that device current (every GPU holds its own copy at its own address) and kept in a table; host
// code below uses that pointer wherever it needs the array's memory.
//
// Every call on a GPU shares that GPU's array: the part a call uses is zeroed by a kernel on the call's stream before
// the scatter adds to it, and two calls that overlap in time on one GPU (different streams, different threads) race.
#include <mutex>

#include "launch.hpp"

namespace {

static __device__ __align__(256) unsigned char scratch[CLUSTEN_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` per device ordinal, nullptr until asked
std::mutex g_scratch_mutex;

// Device address of the scratch array on the current device (first call on a device: one symbol look-up).
int scratch_of_current_device(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return CLUSTEN_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            return CLUSTEN_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return CLUSTEN_OK;
}

}  // namespace

extern "C" int clusten_qk_backward_static(const void* d_attn, const void* query, clusten_strides query_strides,
                                          const void* key, clusten_strides key_strides, const int64_t* nbhd_idx,
                                          void* d_query, void* d_key, clusten_attn_shape shape, int dtype,
                                          clusten_stream stream) {
    using namespace clusten;
    if (!d_attn || !query || !key || !nbhd_idx || !d_query || !d_key) return CLUSTEN_ERR_NULL_POINTER;
    if (!dtype_ok(dtype)) return CLUSTEN_ERR_BAD_DTYPE;
    if (int st = check_attn_shape(shape)) return st;
    if (!strides_ok(query_strides, shape.C) || !strides_ok(key_strides, shape.C)) return CLUSTEN_ERR_BAD_STRIDE;
    const size_t need = scatter_rows_workspace_bytes(shape, dtype);
    if (need > (size_t)CLUSTEN_STATIC_SCRATCH_BYTES) return CLUSTEN_ERR_TOO_LARGE;
    void* ws = nullptr;
    if (need != 0) {
        if (int st = scratch_of_current_device(&ws)) return st;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    clusten_strides out_strides;
    out_strides.n = shape.C;
    out_strides.h = (int64_t)shape.N * shape.C;
    out_strides.b = (int64_t)shape.H * shape.N * shape.C;
    // d_query = gather_sum(d_attn, key); d_key = scatter_rows(d_attn, query), 16-bit sums built in `ws`
    int st = launch_gather_sum(d_attn, key, key_strides, nbhd_idx, d_query, out_strides, shape, dtype, s);
    if (st != CLUSTEN_OK) return st;
    return launch_scatter_rows(d_attn, query, query_strides, nbhd_idx, d_key, ws, shape, dtype, s);
}
