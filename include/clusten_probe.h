/*
 * clusten_probe.h — C ABI of libclusten_probe.so: measurement kernels that sit beside libclusten_hip.so.
 *
 * Nothing here has a counterpart in the reference and nothing here is needed to run the operators: a benchmark
 * loads this library to calibrate a profiler's byte counters against a kernel of known traffic, to print the
 * copy bandwidth the device sustains next to a roofline figure, and to price an operator's memory instruction
 * stream without its arithmetic.  Conventions (device pointers, stream argument, status codes, no allocation,
 * no synchronisation) are those of clusten_hip.h, whose types are used.
 */
#ifndef CLUSTEN_PROBE_H
#define CLUSTEN_PROBE_H

#include "clusten_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define CLUSTEN_PROBE_ABI_VERSION 1

/* CLUSTEN_PROBE_ABI_VERSION the library was built with. */
int clusten_probe_abi_version(void);

/* Plain streaming copy of `bytes` bytes (multiple of 16, both pointers 16-byte aligned) with the
 * same launch shape the gather kernels use: a kernel of known traffic. */
int clusten_copy_probe(const void* src, void* dst, size_t bytes, clusten_stream stream);

/* The two components of a gather operator's memory traffic, alone and together, with no arithmetic at all: one wave
 * per tile (`tiles` of them, dealt to the accelerator dies like the operators' tiles) that, with mode bit 0 set, reads
 * 5 KiB of `in` (tile * 5120 ...) and writes 3 KiB of `out` (tile * 3072 ...) — streams that come from and go to
 * memory — and, with mode bit 1 set, gathers `gathers` (a multiple of 12) times four 256-byte rows picked at random
 * inside its window of `rows` (window number tile / tiles_per_window, window_rows rows each) — reads that hit the L2
 * once the window has been touched.  mode 1, 2 and 3 timed on the same buffers show how far the device overlaps the
 * two (on an MI355X: not at all — the times add up).  in >= tiles * 5120 bytes, out >= tiles * 3072 bytes, rows >=
 * ceil(tiles / tiles_per_window) * window_rows * 256 bytes, all 16-byte aligned. */
int clusten_stream_gather_probe(const void* in, void* out, const void* rows, int tiles, int gathers, int window_rows,
                                int tiles_per_window, int mode, clusten_stream stream);

/* clusten_qk_forward, clusten_av_forward and clusten_wf_forward without their arithmetic: the same kernels compiled a
 * second time with every matrix instruction replaced by one integer operation on its operands, so that they issue the
 * same global loads, LDS accesses and stores in the same order and nothing else.  Arguments as for the functions they
 * shadow; dtype F32 only (else CLUSTEN_ERR_BAD_DTYPE); the outputs hold no meaningful values.  A benchmark prints,
 * next to the time of a kernel, what its memory instruction stream costs by itself on the same inputs. */
int clusten_qk_forward_replay(const void* query, clusten_strides query_strides,
                              const void* key, clusten_strides key_strides,
                              const int64_t* nbhd_idx, void* attn,
                              clusten_attn_shape shape, int dtype, clusten_stream stream);
int clusten_av_forward_replay(const void* attn,
                              const void* value, clusten_strides value_strides,
                              const int64_t* nbhd_idx,
                              void* feat, clusten_strides feat_strides,
                              clusten_attn_shape shape, int dtype, clusten_stream stream);
int clusten_wf_forward_replay(const void* weights, const void* feat, const int64_t* nbhd_idx,
                              void* feat_new, clusten_wf_shape shape, int dtype, clusten_stream stream);

#ifdef __cplusplus
}
#endif

#endif /* CLUSTEN_PROBE_H */
