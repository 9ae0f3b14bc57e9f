/*
 * clusten_hip.h — C ABI of libclusten_hip.so: the CLUSTEN neighbourhood-gather ops
 * (QK, AV, WF; forward and backward) as hand-written gfx950 HIP kernels.
 *
 * Every entry point
 *   - takes plain device pointers, sizes, element strides, a dtype code and a HIP stream;
 *   - enqueues its kernels on that stream and returns without synchronising;
 *   - never allocates or frees memory (scratch comes in through a workspace argument; the one entry point
 *     without such an argument, clusten_qk_backward_static, uses a fixed device array of the library);
 *   - returns a clusten_status (0 = ok) instead of throwing;
 *   - is re-entrant: the library keeps no mutable global state (clusten_qk_backward_static excepted: calls
 *     that overlap in time on one GPU share its scratch array and race).
 *
 * The entry points stand in for the six functions the reference binds through pybind11
 * (three extension modules, each exporting `forward` and `backward`):
 *   clusten/src/clustenqk_cuda.cpp:25-51, clusten/src/clustenav_cuda.cpp:25-51,
 *   clusten/src/clustenwf_cuda.cpp:25-51.
 * Differences a caller must know:
 *   - outputs are caller-allocated (the reference allocates them with torch::zeros);
 *   - `key` is passed un-transposed, (B,H,N,C) — the reference's wrapper hands its kernel a
 *     (B,H,C,N) copy (clusten/clusten.py:30), which is an implementation detail of that kernel;
 *   - query / key / value may be strided views: element strides for the batch, head and token
 *     axes are explicit arguments, the channel axis must have stride 1.  Passing the strides of a
 *     (B,N,H,C)-stored tensor avoids the `.contiguous()` copies of clusten/clusten.py:23-24,49-50.
 *
 * Index convention: `nbhd_idx` is int64, contiguous, values in [0, N) — unchecked, as in the
 * reference.  All tensors of one call live on the device that is current for `stream`.
 */
#ifndef CLUSTEN_HIP_H
#define CLUSTEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CLUSTEN_ABI_VERSION 4

/* Element type of every floating-point tensor of a call.  The reference dispatches
 * double / float / half (AT_DISPATCH_FLOATING_TYPES_AND_HALF, clustenqk_cuda_kernel.cu:78);
 * bfloat16 has no reference kernel and is checked against the gather oracle only. */
typedef enum clusten_dtype {
    CLUSTEN_F32 = 0,
    CLUSTEN_F16 = 1,
    CLUSTEN_BF16 = 2,
    CLUSTEN_F64 = 3
} clusten_dtype;

typedef enum clusten_status {
    CLUSTEN_OK = 0,
    CLUSTEN_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
    CLUSTEN_ERR_BAD_DTYPE = 2,      /* dtype code not in clusten_dtype */
    CLUSTEN_ERR_BAD_DIMS = 3,       /* a size is <= 0, or N >= 2^31, or a per-batch slice >= 2^31 elements */
    CLUSTEN_ERR_BAD_STRIDE = 4,     /* a stride is negative or makes rows overlap */
    CLUSTEN_ERR_WORKSPACE = 5,      /* workspace missing or smaller than *_workspace_bytes() */
    CLUSTEN_ERR_LAUNCH = 6,         /* hipGetLastError() reported a failure after a launch */
    CLUSTEN_ERR_UNALIGNED = 7,      /* an optional entry point (e.g. clusten_attn_softmax_forward) was handed a pointer
                                       that is not 16-byte aligned (the gather ops route unaligned operands to
                                       element-wise kernels) */
    CLUSTEN_ERR_TOO_LARGE = 8       /* clusten_qk_backward_static: the problem needs more scratch than
                                       CLUSTEN_STATIC_SCRATCH_BYTES */
} clusten_status;

/* Opaque stream handle: a hipStream_t.  NULL is the legacy default stream. */
typedef void* clusten_stream;

/* Shape of one QK / AV problem.
 *   query/key/value : (B,H,N,C), element (b,h,n,c) at b*stride_b + h*stride_h + n*stride_n + c
 *   nbhd_idx        : (B,N,M) int64 contiguous, shared by all heads
 *   attn            : (B,H,N,M) contiguous */
typedef struct clusten_attn_shape {
    int32_t B, H, N, C, M;
} clusten_attn_shape;

/* Element strides of a (B,H,N,C) operand whose channel stride is 1. */
typedef struct clusten_strides {
    int64_t b, h, n;
} clusten_strides;

/* Shape of one WF problem.
 *   weights  : (B,Nout,M,IC) contiguous
 *   feat     : (B,N,C) contiguous
 *   nbhd_idx : (B,Nout,M) int64 contiguous, values in [0,N)
 *   feat_new : (B,Nout,IC,C) contiguous */
typedef struct clusten_wf_shape {
    int32_t B, N, Nout, C, M, IC;
} clusten_wf_shape;

/* ---- library ------------------------------------------------------------------------------ */

/* CLUSTEN_ABI_VERSION the library was built with. */
int clusten_abi_version(void);

/* Static, NUL-terminated description of a status code. */
const char* clusten_status_string(int status);

/* ---- QK:  attn[b,h,i,j] = sum_c query[b,h,i,c] * key[b,h,nbhd_idx[b,i,j],c] ------------------- */

/* Replaces clustenqk_cuda.forward (clusten/src/clustenqk_cuda.cpp:25-33, kernel
 * clustenqk_cuda_kernel.cu:18-89).  `attn` need not be zeroed. */
int clusten_qk_forward(const void* query, clusten_strides query_strides,
                       const void* key, clusten_strides key_strides,
                       const int64_t* nbhd_idx, void* attn,
                       clusten_attn_shape shape, int dtype, clusten_stream stream);

/* Replaces clustenqk_cuda.backward (clustenqk_cuda.cpp:35-45, clustenqk_cuda_kernel.cu:91-178):
 *   d_query[b,h,i,c] = sum_j key[b,h,idx[b,i,j],c] * d_attn[b,h,i,j]
 *   d_key[b,h,n,c]   = sum_{(i,j): idx[b,i,j]=n} query[b,h,i,c] * d_attn[b,h,i,j]
 * d_query, d_key are (B,H,N,C) contiguous, need not be zeroed.  `workspace` (clusten_qk_backward_workspace_bytes,
 * 16-byte aligned) holds what the scatter needs: the pair lists of lists made of whole clusters (see
 * clusten_cluster_pairs below: built on every call; such lists take a gather without atomics whose sums repeat bit
 * for bit, chosen on the device — the host reads nothing back), one byte per tile of 8 tokens (which tiles the
 * kernel that sums shared lists in LDS has added) and, for F16/BF16, the fp32 sums of the atomic kernels that any
 * other list takes (rounded once). */
size_t clusten_qk_backward_workspace_bytes(clusten_attn_shape shape, int dtype);
int clusten_qk_backward(const void* d_attn,
                        const void* query, clusten_strides query_strides,
                        const void* key, clusten_strides key_strides,
                        const int64_t* nbhd_idx, void* d_query, void* d_key,
                        void* workspace, size_t workspace_bytes,
                        clusten_attn_shape shape, int dtype, clusten_stream stream);

/* clusten_qk_backward without a workspace argument and without any allocation, for callers that cannot call
 * hipMalloc (code under HIP graph capture, tight serving loops, harnesses that forbid it).  It has no counterpart
 * in the reference.  Same arguments, results and kernels as clusten_qk_backward; the fp32 buffer in which the d_key of F16/BF16 data is
 * summed is a device array of CLUSTEN_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on until
 * the process ends.  clusten_qk_backward_workspace_bytes(shape, dtype) bytes of it are used: a problem that needs more
 * is refused with CLUSTEN_ERR_TOO_LARGE.  The array's address on a device is looked up on the first call made with that device
 * current: make that call outside any stream capture (every later call, recorded or not, launches kernels and nothing else).
 * Calls on one GPU share the array (each clears the part it uses on its own stream first), so calls that
 * overlap in time on one GPU race: keep them on one stream or order them with events. */
#define CLUSTEN_STATIC_SCRATCH_BYTES (32u << 20)
int clusten_qk_backward_static(const void* d_attn,
                               const void* query, clusten_strides query_strides,
                               const void* key, clusten_strides key_strides,
                               const int64_t* nbhd_idx, void* d_query, void* d_key,
                               clusten_attn_shape shape, int dtype, clusten_stream stream);

/* ---- AV:  feat[b,h,i,c] = sum_j attn[b,h,i,j] * value[b,h,nbhd_idx[b,i,j],c] ------------------ */

/* Replaces clustenav_cuda.forward (clusten/src/clustenav_cuda.cpp:25-33, kernel
 * clustenav_cuda_kernel.cu:18-90).  `feat` is written with the strides given (channel stride 1),
 * so a caller can have it land directly in (B,N,H,C) storage. */
int clusten_av_forward(const void* attn,
                       const void* value, clusten_strides value_strides,
                       const int64_t* nbhd_idx,
                       void* feat, clusten_strides feat_strides,
                       clusten_attn_shape shape, int dtype, clusten_stream stream);

/* clusten_av_forward for fp32 attention weights over 16-bit values — what mixed precision hands the operator: the
 * softmax that precedes it returns fp32, the value projection fp16 or bf16, and the reference's wrapper casts the
 * values up first (clusten/clusten.py:52-53).  Here the 16-bit rows are read in place and widened on the way to the
 * staging buffer: the same values and arithmetic as clusten_av_forward on a cast copy (bit-identical results),
 * without that pass over the value tensor.  attn (B,H,N,M) and feat (strided (B,H,N,C)) fp32; value strided (B,H,N,C)
 * of value_dtype, F16 or BF16 (else CLUSTEN_ERR_BAD_DTYPE).  Lists of more than 64 slots that clusten_av_forward hands
 * to its kernels for long runs (M a multiple of 24, 32 or 16 with at most 8 runs) are turned down with
 * CLUSTEN_ERR_BAD_DIMS: cast the values and call clusten_av_forward. */
int clusten_av_forward_mixed(const void* attn,
                             const void* value, clusten_strides value_strides, int value_dtype,
                             const int64_t* nbhd_idx,
                             void* feat, clusten_strides feat_strides,
                             clusten_attn_shape shape, clusten_stream stream);

/* Replaces clustenav_cuda.backward (clustenav_cuda.cpp:35-45, clustenav_cuda_kernel.cu:93-218):
 *   d_attn[b,h,i,j]  = sum_c value[b,h,idx[b,i,j],c] * d_feat[b,h,i,c]
 *   d_value[b,h,n,c] = sum_{(i,j): idx[b,i,j]=n} attn[b,h,i,j] * d_feat[b,h,i,c]
 * d_attn (B,H,N,M) and d_value (B,H,N,C) are contiguous, need not be zeroed. */
size_t clusten_av_backward_workspace_bytes(clusten_attn_shape shape, int dtype);
int clusten_av_backward(const void* d_feat, clusten_strides d_feat_strides,
                        const void* attn,
                        const void* value, clusten_strides value_strides,
                        const int64_t* nbhd_idx, void* d_attn, void* d_value,
                        void* workspace, size_t workspace_bytes,
                        clusten_attn_shape shape, int dtype, clusten_stream stream);

/* ---- WF:  feat_new[b,i,ic,c] = sum_j weights[b,i,j,ic] * feat[b,nbhd_idx[b,i,j],c] ------------ */

/* Replaces clustenwf_cuda.forward (clusten/src/clustenwf_cuda.cpp:25-33, kernel
 * clustenwf_cuda_kernel.cu:18-93). */
int clusten_wf_forward(const void* weights, const void* feat, const int64_t* nbhd_idx,
                       void* feat_new, clusten_wf_shape shape, int dtype, clusten_stream stream);

/* clusten_wf_forward for fp32 weights over 16-bit features, read in place (the reference's wrapper casts the features
 * up first, clusten/clusten.py:78-79); bit-identical to clusten_wf_forward on a cast copy.  weights (B,Nout,M,IC) and
 * feat_new (B,Nout,IC,C) fp32; feat (B,N,C) of feat_dtype, F16 or BF16 (else CLUSTEN_ERR_BAD_DTYPE). */
int clusten_wf_forward_mixed(const void* weights, const void* feat, int feat_dtype, const int64_t* nbhd_idx,
                             void* feat_new, clusten_wf_shape shape, clusten_stream stream);

/* Replaces clustenwf_cuda.backward (clustenwf_cuda.cpp:35-45, clustenwf_cuda_kernel.cu:96-229):
 *   d_weights[b,i,j,ic] = sum_c feat[b,idx[b,i,j],c] * d_feat_new[b,i,ic,c]
 *   d_feat[b,n,c]       = sum_{(i,j): idx[b,i,j]=n} sum_ic d_feat_new[b,i,ic,c] * weights[b,i,j,ic] */
size_t clusten_wf_backward_workspace_bytes(clusten_wf_shape shape, int dtype);
int clusten_wf_backward(const void* d_feat_new, const void* weights, const void* feat,
                        const int64_t* nbhd_idx, void* d_weights, void* d_feat,
                        void* workspace, size_t workspace_bytes,
                        clusten_wf_shape shape, int dtype, clusten_stream stream);

/* ---- compact neighbourhood lists (optional) --------------------------------------------------- */

/* QK and AV forward with the neighbourhoods given as cluster numbers instead of row lists.  The reference's
 * BasicLayer builds nbhd_idx by expanding the nnc nearest clusters of every token into their 8 members
 * (models/aff_transformer.py:476-480; members of cluster g are rows 8g..8g+7 of the cluster-ordered
 * sequence, pad slots of the last cluster hold row 0, models/point_utils.py:203-206): an int64 (B,N,8*nnc)
 * tensor that is 30-55 % of the operators' traffic.  These entry points take the (B,N,nnc) cluster numbers
 * themselves, as int32 — 1/16 of the bytes — and compute exactly what clusten_qk_forward /
 * clusten_av_forward compute on the expanded lists:
 *     nbhd_idx[b,i,8*r+t] = 8*cluster_idx[b,i,r]+t   if that is < N,   else 0.
 * shape.M = 8 * nnc (a multiple of 8, at most 64).  Longer lists are lists of larger clusters: for 64 < M <= 256 the
 * cluster size is L = clusten_cluster_size_for(M) (24 if M is a multiple of 24 of at most 8 clusters, else 32, else
 * 16 by the same rule: M = 144 is the 6 clusters of 24 tokens of the 384 x 384 configurations,
 * configs/aff_base_22kto1k_384.yaml:10-11), cluster_idx is (B,N,M/L) and
 *     nbhd_idx[b,i,L*r+t] = L*cluster_idx[b,i,r]+t   if that is < N,   else 0
 * (a cluster number whose first row is outside [0,N) stands for L slots of row 0).
 * Tile kernels only: dtype F32/F16/BF16, head dim 16/32/64 (for M > 64: rows of at least 64 bytes), else
 * CLUSTEN_ERR_BAD_DIMS; rows 16-byte aligned (else CLUSTEN_ERR_UNALIGNED).  Forward only:
 * for training expand the lists and use the functions above.  No counterpart in the reference's extension
 * modules. */
int clusten_cluster_size_for(int M);   /* 8 for M <= 64 (M % 8 == 0), L as above for 64 < M <= 256, 0 otherwise */
int clusten_qk_forward_clusters(const void* query, clusten_strides query_strides,
                                const void* key, clusten_strides key_strides,
                                const int32_t* cluster_idx, void* attn,
                                clusten_attn_shape shape, int dtype, clusten_stream stream);
int clusten_av_forward_clusters(const void* attn, const void* value, clusten_strides value_strides,
                                const int32_t* cluster_idx, void* feat, clusten_strides feat_strides,
                                clusten_attn_shape shape, int dtype, clusten_stream stream);

/* ---- glue between QK and AV (optional) -------------------------------------------------------- */

/* The arithmetic the model does between CLUSTENQKFunction and CLUSTENAVFunction, in one pass:
 *   probs[b,h,i,:M], blank_prob[b,h,i] = softmax over the M neighbours and one blank token of
 *     attn[b,h,i,j] + bias_table[pe_idx[b,i,j], h] - 100 * (1 - mask[b,i,j])   and   blank_logit[b,h,i].
 * It has no entry point in the reference, which writes these steps as tensor expressions
 * (models/aff_transformer.py:122-147: position-bias gather, two additions, cat with the blank token,
 * softmax, two slices); it replaces those for inference and leaves the three operators as they are.
 *   attn (B,H,N,M) and bias_table (rows,H): `dtype` (F32, F16 or BF16), contiguous;
 *   pe_idx (B,N,M) int64 with values in [0, rows) — unchecked; mask (B,N,M) int64 of 0/1, or NULL;
 *   blank_logit (B,H,N), probs (B,H,N,M), blank_prob (B,H,N): fp32, contiguous.
 * blank_logit may be NULL when query (strided (B,H,N,C) like clusten_qk_forward's, `dtype`) and blank_key
 * ((H,C), fp32, contiguous) are given: the logit is then their dot product per token and head
 * (`(q * blank_k).sum(-1)`, models/aff_transformer.py:144), computed in fp32 inside the same pass.
 * M <= 256 and M % 4 == 0, else CLUSTEN_ERR_BAD_DIMS; attn and probs 16-byte aligned, else
 * CLUSTEN_ERR_UNALIGNED. */
int clusten_attn_softmax_forward(const void* attn, const void* bias_table, const int64_t* pe_idx,
                                 const int64_t* mask, const float* blank_logit, const void* query,
                                 clusten_strides query_strides, const float* blank_key, float* probs,
                                 float* blank_prob, clusten_attn_shape shape, int dtype,
                                 clusten_stream stream);

/* Local attention of a cluster-ordered token sequence in one kernel (inference): CLUSTENQKFunction, the
 * arithmetic clusten_attn_softmax_forward describes, CLUSTENAVFunction and the blank token's value
 * (models/aff_transformer.py:120-155), on lists given as cluster numbers, without the (B,H,N,M) logits and
 * probabilities ever reaching memory:
 *   logit[b,h,i,j] = scale * <query[b,h,i], key[b,h,row(i,j)]> + bias_table[pe_idx[b,i,j], h] - 100 * (1 - mask[b,i,j])
 *   blank[b,h,i]   = scale * <query[b,h,i], blank_key[h]>
 *   p, p_blank     = softmax over the M neighbours and the blank token
 *   out[b,h,i]     = sum_j p[b,h,i,j] * value[b,h,row(i,j)] + p_blank[b,h,i] * blank_value[h]
 *   row(i,j)       = S * cluster_idx[b,i,j/S] + j%S, row 0 where that is not in [0,N);  S = M / 6, the cluster size
 * query, key, value, out: strided (B,H,N,C) of `dtype`; bias_table (rows,H) of `dtype`, contiguous;
 * cluster_idx (B,N,6) int32; pe_idx (B,N,M) int64 in [0,rows) — unchecked; mask (B,N,M) int64 of 0/1 or NULL;
 * with lists_shared != 0 these three are (1,N,.) tensors that serve every batch element (the tokens of a
 * regular grid have the same neighbourhoods in every image);
 * blank_key, blank_value (H,C) fp32, contiguous.  Pass the unscaled query and the model's scale, or a scaled
 * query and 1.  The probabilities are rounded to `dtype` before they weigh the value rows; sums are fp32.
 * dtype F16, BF16 or F32 (else CLUSTEN_ERR_BAD_DTYPE); C = 32; M = 48 (six clusters of 8: the 224 x 224 models) or,
 * for F16 / BF16, M = 144 (six clusters of 24: the 384 x 384 models, configs/aff_base_22kto1k_384.yaml:10-11), else
 * CLUSTEN_ERR_BAD_DIMS; rows 16-byte aligned (else CLUSTEN_ERR_UNALIGNED).  No counterpart in the reference's
 * extension modules. */
int clusten_cluster_attention_forward(const void* query, clusten_strides query_strides,
                                      const void* key, clusten_strides key_strides,
                                      const void* value, clusten_strides value_strides,
                                      const int32_t* cluster_idx, const void* bias_table,
                                      const int64_t* pe_idx, const int64_t* mask, int lists_shared,
                                      const float* blank_key, const float* blank_value,
                                      void* out, clusten_strides out_strides, float scale,
                                      clusten_attn_shape shape, int dtype, clusten_stream stream);

/* The same kernel with what it works out from cluster_idx, pe_idx and mask before its first head — the distinct
 * clusters of every tile of 8 tokens, the bias-table row and mask bit of every slot, the runs a token repeats —
 * handed over as a plan: the lists of a stage serve all its layers (models/aff_transformer.py:454-487 builds them once
 * per stage, :505-507 runs the blocks on them), so the plan is built once per stage and read by every layer.
 *   clusten_cluster_attention_plan_bytes(B, N, M): size of the plan for index tensors of B batch elements (B = 1 when
 *   the lists are shared by every image) and M = 48 or 144 neighbours per token (0 for any other M);
 *   clusten_cluster_attention_plan: fills it from cluster_idx (B,N,6) int32, pe_idx (B,N,M) int64 and mask (B,N,M)
 *   int64 or NULL; plan 16-byte aligned (else CLUSTEN_ERR_UNALIGNED), plan_bytes at least the size above (else
 *   CLUSTEN_ERR_WORKSPACE);
 *   clusten_cluster_attention_forward_planned: clusten_cluster_attention_forward with `plan` in the place of the three
 *   index tensors; same results bit for bit.
 * No counterpart in the reference's extension modules. */
size_t clusten_cluster_attention_plan_bytes(int B, int N, int M);
int clusten_cluster_attention_plan(const int32_t* cluster_idx, const int64_t* pe_idx, const int64_t* mask, void* plan,
                                   size_t plan_bytes, int B, int N, int M, clusten_stream stream);
int clusten_cluster_attention_forward_planned(const void* query, clusten_strides query_strides,
                                              const void* key, clusten_strides key_strides,
                                              const void* value, clusten_strides value_strides,
                                              const void* plan, const void* bias_table, int lists_shared,
                                              const float* blank_key, const float* blank_value,
                                              void* out, clusten_strides out_strides, float scale,
                                              clusten_attn_shape shape, int dtype, clusten_stream stream);

/* clusten_cluster_attention_forward_planned for a forward pass whose backward will follow: it also writes
 * lse[b,h,i] = log of the denominator of token i's softmax (fp32, (B,H,N) contiguous), from which
 * clusten_cluster_attention_backward recomputes the probabilities.  dtype F16, BF16 or F32. */
int clusten_cluster_attention_forward_train(const void* query, clusten_strides query_strides,
                                            const void* key, clusten_strides key_strides,
                                            const void* value, clusten_strides value_strides,
                                            const void* plan, const void* bias_table, int lists_shared,
                                            const float* blank_key, const float* blank_value,
                                            void* out, clusten_strides out_strides, float* lse, float scale,
                                            clusten_attn_shape shape, int dtype, clusten_stream stream);

/* The query-side half of the backward of the kernel above, in one kernel (the backward of
 * models/aff_transformer.py:120-155: clustenqk_cuda_kernel.cu:51-132, the tensor expressions between the operators,
 * clustenav_cuda_kernel.cu:51-127).  With p = exp(logit - lse), delta[i] = <d_out[i], out[i]>:
 *   d_logit[b,h,i,j] = p * (<d_out[b,h,i], value[b,h,row(i,j)]> - delta),   d_blank_logit likewise with blank_value
 *   d_query[b,h,i]   = scale * (sum_j d_logit[b,h,i,j] * key[b,h,row(i,j)] + d_blank_logit[b,h,i] * blank_key[h])
 * It writes d_query (strided (B,H,N,C)), probs and d_logit ((B,H,N,M) of `dtype`, contiguous), blank_prob and
 * d_blank_logit (fp32 (B,H,N)).  The rest of the backward are sums other entry points form:
 *   d_value = clusten_scatter_rows_by_cluster(probs, d_out),  d_key = scale * clusten_scatter_rows_by_cluster(d_logit, query),
 *   d_bias_table = clusten_bias_table_grad(d_logit),  d_blank_key = scale * sum d_blank_logit * query,
 *   d_blank_value = sum blank_prob * d_out.
 * d_out, out: strided (B,H,N,C) like query (the forward's result and its gradient); dtype F16, BF16 or F32 (for F32
 * the bias table is fp32 too, as in the forward), C = 32, M = 48.  No counterpart in the reference's extension
 * modules. */
int clusten_cluster_attention_backward(const void* query, clusten_strides query_strides,
                                       const void* key, clusten_strides key_strides,
                                       const void* value, clusten_strides value_strides,
                                       const void* d_out, clusten_strides d_out_strides,
                                       const void* out, clusten_strides out_strides,
                                       const float* lse, const void* plan, const void* bias_table, int lists_shared,
                                       const float* blank_key, const float* blank_value,
                                       void* d_query, clusten_strides d_query_strides,
                                       void* probs, void* d_logit, float* blank_prob, float* d_blank_logit,
                                       float scale, clusten_attn_shape shape, int dtype, clusten_stream stream);

/* ---- lists made of whole clusters: the backward scatters as gathers (optional) ------------------------------ */

/* The pair lists of neighbour lists made of whole clusters, built on the device without any read-back by the host.
 * A list tensor nbhd_idx (B,rows,M) int64 that points into sequences of n_rows rows is "made of whole clusters" when
 * every run of 8 slots holds the 8 rows of one cluster: nbhd_idx[b,i,8r+t] = 8 c(b,i,r) + t (the lists of
 * models/aff_transformer.py:476-480); when n_rows % 8 != 0 the last cluster has n_rows % 8 rows and the slots past
 * them hold row 0 (models/point_utils.py:203-206).  For such lists the block `pair_lists` receives, for every cluster
 * (b,g), the pairs (i,r) with c(b,i,r) = g in ascending order — what clusten_scatter_rows_by_cluster and
 * clusten_wf_backward_by_cluster read; it can serve every head and every layer that uses the same lists.  The block is
 * opaque but for its first int32, the flag `not_whole`: 0 when the lists are made of whole clusters, 1 when some run is
 * not (the rest of the block then means nothing, and the two consumers leave their outputs untouched).
 * clusten_qk_backward, clusten_av_backward and clusten_wf_backward build the same lists in their workspace on every
 * call and select their kernels through the same flag on the device.
 *   clusten_cluster_pairs_bytes: size of the block; 0 when the shape is not supported (M % 8 != 0, M > 256, n_rows < 8,
 *   or more than about 7000 clusters per image); pair_lists must be 16-byte aligned (else CLUSTEN_ERR_UNALIGNED).
 * rows = N for attention lists (n_rows = N too), Nout for a merge's lists (n_rows = N).  No counterpart in the
 * reference's extension modules. */
size_t clusten_cluster_pairs_bytes(int B, int rows, int M, int n_rows);
int clusten_cluster_pairs(const int64_t* nbhd_idx, void* pair_lists, size_t pair_lists_bytes, int B, int rows, int M,
                          int n_rows, clusten_stream stream);
/* The same block from the lists given as cluster numbers (the format of clusten_qk_forward_clusters, clusters of 8
 * rows): cluster_idx (B,rows,nnc) int32, block of clusten_cluster_pairs_bytes(B, rows, 8 * nnc, n_rows) bytes.  With it the
 * backward of the cluster-number forms needs no row lists at all:
 *   d_query = clusten_av_forward_clusters(d_attn, key, cluster_idx),  d_key   = clusten_scatter_rows_by_cluster(d_attn, query, block)
 *   d_attn  = clusten_qk_forward_clusters(d_feat, value, cluster_idx), d_value = clusten_scatter_rows_by_cluster(attn, d_feat, block)
 * A number outside [0, ceil(n_rows / 8)) sets the block's flag (the forward forms read row 0 for such a number; the
 * by-cluster scatter then leaves its output untouched: check the flag, or keep the numbers in range, as the lists of
 * models/aff_transformer.py:476 are).  No counterpart in the reference's extension modules. */
int clusten_cluster_pairs_from_numbers(const int32_t* cluster_idx, void* pair_lists, size_t pair_lists_bytes, int B,
                                       int rows, int nnc, int n_rows, clusten_stream stream);

/* The scatter of the two attention backward passes as a gather, for lists made of whole clusters:
 *   y[b,h, 8g+t, :] = sum over the pairs (i,r) with c(b,i,r) = g of  p[b,h,i,8r+t] * x[b,h,i,:]
 * which equals the d_key of clusten_qk_backward (p = d_attn, x = query) and the d_value of clusten_av_backward
 * (p = attn, x = d_feat) on such lists, without atomics, zero-fill or workspace, every sum in fp32 in a fixed order
 * (results repeat bit for bit).  pair_lists: the block clusten_cluster_pairs filled for (B, N, M, N).
 * p (B,H,N,M) and y (B,H,N,C) contiguous, x strided (B,H,N,C), all of `dtype` (F32, F16 or BF16); every row of y is
 * written — unless the block's flag says the lists are not made of whole clusters: then y is left untouched.
 * C in {16,32,64}, N >= 8, M % 8 == 0, M <= 256 (else CLUSTEN_ERR_BAD_DIMS); rows 16-byte aligned (else
 * CLUSTEN_ERR_UNALIGNED).  No counterpart in the reference's extension modules. */
int clusten_scatter_rows_by_cluster(const void* p, const void* x, clusten_strides x_strides, const void* pair_lists,
                                    void* y, clusten_attn_shape shape, int dtype, clusten_stream stream);

/* The scatter of the two attention backward passes alone, for any lists:
 *   y[b,h,nbhd_idx[b,i,j],:] += p[b,h,i,j] * x[b,h,i,:]          (y need not be zeroed)
 * the d_key of clusten_qk_backward (p = d_attn, x = query; clustenqk_cuda_kernel.cu:91-132) and the d_value of
 * clusten_av_backward (p = attn, x = d_feat; clustenav_cuda_kernel.cu:93-127), with the kernels of those two entry
 * points: the gather over pair lists when the lists are made of whole clusters, atomics otherwise, chosen on the device.
 * pair_lists: the block clusten_cluster_pairs filled for (B, N, M, N), or NULL.  A caller that keeps the block of a
 * list tensor (one per stage of a model: it serves every layer and head) saves the rebuild on every call; when the
 * block's flag says the lists are not made of whole clusters the atomic kernels run, so y is always the full sum.
 * p (B,H,N,M) and y (B,H,N,C) contiguous, x strided (B,H,N,C); workspace of clusten_scatter_rows_workspace_bytes
 * (= clusten_qk_backward_workspace_bytes) bytes, 16-byte aligned, whether or not pair_lists is given. */
size_t clusten_scatter_rows_workspace_bytes(clusten_attn_shape shape, int dtype);
int clusten_scatter_rows(const void* p, const void* x, clusten_strides x_strides, const int64_t* nbhd_idx,
                         const void* pair_lists, void* y, void* workspace, size_t workspace_bytes,
                         clusten_attn_shape shape, int dtype, clusten_stream stream);

/* clusten_wf_backward for lists made of whole clusters, the feature gradient as a gather (no atomics, no workspace,
 * every row of d_feat written once from an fp32 sum in a fixed order):
 *   d_feat[b, 8g+t, :] = sum over the pairs (i,r) of cluster (b,g) of  sum_ic weights[b,i,8r+t,ic] * d_feat_new[b,i,ic,:]
 * pair_lists: the block clusten_cluster_pairs filled for (B, Nout, M, N) (i counts the output tokens, g the clusters
 * of the N feature rows); d_weights as clusten_wf_backward computes it.  When the block's flag says the lists are not
 * made of whole clusters d_feat is left untouched.  IC = 4, C % 32 == 0, N >= 8, M % 8 == 0, M <= 256 (else
 * CLUSTEN_ERR_BAD_DIMS); dtype F32, F16 or BF16.  No counterpart in the reference's extension modules. */
int clusten_wf_backward_by_cluster(const void* d_feat_new, const void* weights, const void* feat,
                                   const int64_t* nbhd_idx, const void* pair_lists,
                                   void* d_weights, void* d_feat, clusten_wf_shape shape, int dtype,
                                   clusten_stream stream);

/* Attention of every token over every token of a short sequence, fused: the branch the reference model takes in
 * a stage whose neighbourhood size reaches its number of tokens (models/aff_transformer.py:108-113 and :125-155:
 * `q @ key^T`, position bias, blank token, softmax, `attn @ v`, blank value), without the (B,H,N,N) logits and
 * probabilities ever reaching memory:
 *   logit[b,h,i,j] = scale * <query[b,h,i], key[b,h,j]> + bias_table[pe_idx[b,i,j], h]
 *   blank[b,h,i]   = scale * <query[b,h,i], blank_key[h]>
 *   p, p_blank     = softmax over the N tokens and the blank token
 *   out[b,h,i]     = sum_j p[b,h,i,j] * value[b,h,j] + p_blank[b,h,i] * blank_value[h]
 * query, key, value, out: strided (B,H,N,C) of `dtype`; bias_table (rows,H) of `dtype`, contiguous; pe_idx (B,N,N)
 * int64 in [0,rows) — unchecked; blank_key, blank_value (H,C) fp32, contiguous.  shape.M must equal shape.N.
 * The probabilities are rounded to `dtype` before they weigh the value rows; sums are fp32.
 * dtype F16 or BF16 (else CLUSTEN_ERR_BAD_DTYPE), C = 32 and N = M <= 64 (else CLUSTEN_ERR_BAD_DIMS), rows 16-byte
 * aligned (else CLUSTEN_ERR_UNALIGNED).  Inference only.  No counterpart in the reference's extension modules. */
int clusten_dense_attention_forward(const void* query, clusten_strides query_strides,
                                    const void* key, clusten_strides key_strides,
                                    const void* value, clusten_strides value_strides,
                                    const void* bias_table, const int64_t* pe_idx,
                                    const float* blank_key, const float* blank_value,
                                    void* out, clusten_strides out_strides, float scale,
                                    clusten_attn_shape shape, int dtype, clusten_stream stream);

/* A Linear layer on a tall 16-bit activation matrix and a small weight matrix, optionally followed by GELU:
 *   out[m,n] = act( sum_k x[m,k] * weight[n,k] + bias[n] ),  act = identity (0) or the exact (erf) GELU (1)
 * what `nn.Linear` (and `nn.GELU` after the first MLP layer) compute around the first-stage attention of the
 * reference model (models/aff_transformer.py:60-68 q / kv / proj, :181-196 the MLP), where K and Nout are 64 to
 * 192 and the layer is bound by reading x and writing out once.  x (rows,K) of `dtype` with row stride
 * x_row_stride elements (a multiple of 8), weight (Nout,K) and bias (Nout, or NULL) of `dtype`, contiguous;
 * out (rows,Nout) of `dtype`, contiguous; all 16-byte aligned (else CLUSTEN_ERR_UNALIGNED).  Sums are fp32; with
 * GELU the sum is rounded to `dtype` before the activation, as a separate activation kernel would see it.
 * dtype F16 or BF16 (else CLUSTEN_ERR_BAD_DTYPE); (K,Nout,act) must be one of the combinations
 * clusten_linear_supported accepts — (64,64|128|192,0|1), (128,64,0), (192,64,0) — else CLUSTEN_ERR_BAD_DIMS.
 * Inference only.  No counterpart in the reference's extension modules. */
int clusten_linear_supported(int K, int Nout, int act);
int clusten_linear_forward(const void* x, int64_t x_row_stride, const void* weight, const void* bias, void* out,
                           int64_t rows, int K, int Nout, int act, int dtype, clusten_stream stream);

/* Layer normalisation over the last axis, computed in fp32 from fp32, fp16 or bf16 input and written as fp32,
 * fp16 or bf16:
 *   out[r,c] = (x[r,c] - mean_r) * rsqrt(var_r + eps) * weight[c] + bias[c]      (biased variance)
 * what `nn.LayerNorm` computes in the reference model before every attention and MLP block
 * (models/aff_transformer.py:220, :231, and the norms at :362, :546, :663), with the rounding to 16 bits that
 * mixed precision applies to the following Linear layer's input (and the widening it applies to a 16-bit
 * input of the normalisation) done in the same pass.  x (rows,C) of in_dtype, out (rows,C) of out_dtype (F32,
 * F16 or BF16 each); weight, bias (C) fp32; all contiguous and 16-byte aligned (else CLUSTEN_ERR_UNALIGNED);
 * C in {64,128,256,384,512,768,1024} (else CLUSTEN_ERR_BAD_DIMS).
 * Inference only (no statistics are kept for a backward pass).  No counterpart in the reference's extension
 * modules. */
int clusten_layer_norm_forward(const void* x, int in_dtype, const float* weight, const float* bias, void* out,
                               int64_t rows, int C, float eps, int out_dtype, clusten_stream stream);

/* Layer normalisation (as clusten_layer_norm_forward) of rows read in a given order, with a per-channel bias added
 * first:
 *   out[g*group + i, :] = layer norm of ( x[g*group + order[i], :] + pre_bias[:] )     i < group, g < rows / group
 * the norm that ends the patch embedding of the reference model (models/aff_transformer.py:542-546) with the second
 * convolution's bias and the reordering of the tokens into cluster order (:465-466) taken along.  order (group)
 * int64, a permutation of 0..group-1, or NULL (then group is ignored); pre_bias (C) of in_dtype or NULL, added with a
 * rounding to in_dtype as a separate addition would leave it; rows % group == 0 (else CLUSTEN_ERR_BAD_DIMS); the
 * rest as clusten_layer_norm_forward.  No counterpart in the reference's extension modules. */
int clusten_layer_norm_rows_forward(const void* x, int in_dtype, const int64_t* order, int group, const void* pre_bias,
                                    const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
                                    int out_dtype, clusten_stream stream);

/* y = GELU(x * scale[c] + shift[c]) over a contiguous (B,C,H,W) tensor of F16 or BF16 data (exact GELU, fp32
 * arithmetic, one rounding): convolution bias, inference BatchNorm and activation of the patch embedding
 * (`self.act1(self.bn(self.proj1(x)))`, models/aff_transformer.py:542) in one pass over the convolution's output,
 * with scale = gamma / sqrt(running_var + eps) and shift = (conv_bias - running_mean) * scale + beta prepared by
 * the caller.  scale, shift (C) fp32; HW = H*W a multiple of 8 and B*C < 65536 (else CLUSTEN_ERR_BAD_DIMS); x, y
 * 16-byte aligned;
 * y may be x.  No counterpart in the reference's extension modules. */
int clusten_channel_affine_gelu_forward(const void* x, const float* scale, const float* shift, void* y, int64_t B, int C,
                                        int HW, int dtype, clusten_stream stream);

/* The residual addition ahead of a layer normalisation, and the normalisation, in one pass:
 *   sum_out[r,c] = x[r,c] + branch[r,c]   (rounded to x's type, as the framework's addition leaves it)
 *   out[r,c]     = layer norm of sum_out[r,:] as clusten_layer_norm_forward computes it, written in branch's type
 * i.e. `feat = shortcut + attn_out; self.norm2(feat)` (models/aff_transformer.py:230-231) and
 * `feat = feat + mlp_out` followed by the next block's `self.norm1(feat)` (:232, :219) in inference under mixed
 * precision.  branch and out (rows,C) of branch_dtype, F16 or BF16; x and sum_out (rows,C) of x_dtype, F32 or
 * branch_dtype (else CLUSTEN_ERR_BAD_DTYPE); sum_out may be x itself; weight, bias (C) fp32; everything contiguous
 * and 16-byte aligned; C as for clusten_layer_norm_forward.  No counterpart in the reference's extension modules. */
int clusten_add_layer_norm_forward(const void* x, int x_dtype, const void* branch, int branch_dtype, void* sum_out,
                                   const float* weight, const float* bias, void* out, int64_t rows, int C,
                                   float eps, clusten_stream stream);

/* The index tensors of a stage's local attention from the nearest clusters of every token of a cluster-ordered
 * sequence (models/aff_transformer.py:476-487), in one pass instead of a gather and some ten tensor operations:
 *   row(i,j)         = m * nearest[b,i,j/m] + j%m                        (j < nnc*m)
 *   member_idx[b,i,j] = row(i,j) if row(i,j) < N else 0;   mask[b,i,j] = row(i,j) < N
 *   pe_idx[b,i,j]    = trunc((y' - (y - radius)) * table_width + (x' - (x - radius))),  (x,y) = pos[b,i],
 *                      (x',y') = pos[b, member_idx[b,i,j]]    (fp32, each operation rounded on its own)
 *   cluster_idx[b,i,r] = (int32) nearest[b,i,r]
 * pos (B,N,2) fp32 as (x,y); nearest (B,N,nnc) int64 with values >= 0; member_idx, pe_idx (B,N,nnc*m) int64;
 * mask (B,N,nnc*m) int64 or NULL; cluster_idx (B,N,nnc) int32 or NULL; all contiguous.  No counterpart in the
 * reference's extension modules. */
int clusten_neighbour_lists(const float* pos, const int64_t* nearest, int64_t* member_idx, int64_t* mask,
                            int64_t* pe_idx, int32_t* cluster_idx, int B, int N, int nnc, int m, int radius,
                            int table_width, clusten_stream stream);

/* The importance score of every token before a merge (`self.prob_net(feat).sigmoid()`, a Linear layer with one
 * output: models/aff_transformer.py:498), with the last block's residual addition (:232) taken along when branch is
 * given:
 *   sum_out[r,:] = x[r,:] + branch[r,:]                 (rounded to x's type; skipped when branch is NULL)
 *   score[r]     = sigmoid( round_T( <round_T(sum_out[r,:]), weight> + bias ) ), rounded to T
 * T = dtype, F16 or BF16: the type of weight (C), bias (1 element, or NULL), branch and score (rows); x and sum_out
 * (rows,C) of x_dtype, F32 or dtype (else CLUSTEN_ERR_BAD_DTYPE); sum_out may be x.  C in {64,128,256,512} (else
 * CLUSTEN_ERR_BAD_DIMS); everything contiguous, x / branch / sum_out / weight 16-byte aligned.  Inference only.  No
 * counterpart in the reference's extension modules. */
int clusten_add_row_score_forward(const void* x, int x_dtype, const void* branch, void* sum_out, const void* weight,
                                  const void* bias, void* score, int64_t rows, int C, int dtype,
                                  clusten_stream stream);

/* Backward of clusten_attn_softmax_forward with respect to its logits:
 *   s = sum_j probs[r,j] * d_probs[r,j] + blank_prob[r] * d_blank_prob[r]
 *   d_logit[r,j] = probs[r,j] * (d_probs[r,j] - s);   d_blank_logit[r] = blank_prob[r] * (d_blank_prob[r] - s)
 * for the `rows` = B*H*N rows of M neighbours.  d_logit is the gradient of the attention logits, and, through
 * clusten_bias_table_grad, of the bias table (both enter the softmax as a sum; the mask is a constant).  probs,
 * d_probs (rows,M), blank_prob, d_blank_prob, d_blank_logit (rows) fp32; d_logit (rows,M) of `dtype` (F32, F16 or
 * BF16); M <= 256, M % 4 == 0 (else CLUSTEN_ERR_BAD_DIMS); 16-byte aligned.  No counterpart in the reference's
 * extension modules. */
int clusten_attn_softmax_backward(const float* probs, const float* blank_prob, const float* d_probs,
                                  const float* d_blank_prob, void* d_logit, float* d_blank_logit, int64_t rows, int M,
                                  int dtype, clusten_stream stream);

/* Gradient of the relative-position bias table of an attention layer, the backward of
 * `pe_table.gather(index=pe_idx...)` added to the logits (models/aff_transformer.py:131-133):
 *   d_table[pe_idx[b,i,j], h] += d_logit[b,h,i,j]
 * summed per workgroup in LDS before it reaches memory.  d_logit (B,H,N,M) of `dtype` (F32, F16 or BF16), pe_idx
 * (B,N,M) int64 (entries outside [0,rows) are skipped), d_table (rows,H) fp32, zeroed by the caller; all
 * contiguous.  A workgroup sums its share of the values for the table's 20000 middle rows (all rows of a smaller
 * table) exactly, in 64-bit integer cells scaled to the share's largest magnitude, and only the workgroups' partial
 * sums meet in fp32 atomics, whose order varies from run to run; values for other rows, infinities and NaNs are added
 * to the table one atomic each, as a scatter-add does.  No counterpart in the reference's extension modules. */
int clusten_bias_table_grad(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int N, int M,
                            int rows, int dtype, clusten_stream stream);

/* The `weights` operand of clusten_wf_forward as the reference model builds it before a merge
 * (models/aff_transformer.py:340-358), in one pass instead of a row lookup, a gather and two multiplications:
 *   weights[b,i,j,:] = table_weights[pe_idx[b,i,j], :] * prob[b, nbhd_idx[b,i,j]] * mask[b,i,j]
 * table_weights (rows,IC), prob (B,N) or NULL, weights (B,Nout,M,IC): fp32, contiguous; pe_idx (values in
 * [0,rows) — unchecked), nbhd_idx (values in [0,N) — unchecked; may be NULL when prob is), mask (0/1, or NULL):
 * int64 (B,Nout,M).  IC = 4 (else CLUSTEN_ERR_BAD_DIMS); table_weights and weights 16-byte aligned (else
 * CLUSTEN_ERR_UNALIGNED).  Inference only.  No counterpart in the reference's extension modules. */
int clusten_merge_weights_forward(const float* table_weights, const int64_t* pe_idx, const int64_t* nbhd_idx,
                                  const float* prob, const int64_t* mask, float* weights,
                                  int B, int N, int Nout, int M, int IC, clusten_stream stream);

/* The order in which the reference's balanced clustering lines up the tokens of each image
 * (`space_filling_cluster`, models/point_utils.py:61-208, default scan-line path with anchors; the ranking of
 * point_utils.py:139-159):
 *   ranking[b,:] = stable argsort of  rank * (max ratio of the batch + 1) + ratio,
 * rank = position of the token's anchor cell on the row-by-row walk (alternating direction) over a rows x cols
 * grid of cells of cell_w x cell_h, ratio = squared distance to the previous anchor of the walk over (squared
 * distance to the next + 1e-5); every float operation rounded as the reference's tensor expressions round it.
 *   pos (B,N,2) fp32 as (x, y), inside the canvas; ranking (B,N) int64; N <= clusten_scanline_rank_max_tokens()
 *   (the sort of an image runs in the LDS of one compute unit: 16384 tokens on an MI355X, which covers the 9216
 *   tokens of the first stage of a 384 x 384 model), rows * cols >= 2 (else CLUSTEN_ERR_BAD_DIMS); workspace:
 *   clusten_scanline_rank_workspace_bytes(B, N) bytes, 16-byte aligned.
 * No counterpart in the reference's extension modules. */
int clusten_scanline_rank_max_tokens(void);
size_t clusten_scanline_rank_workspace_bytes(int B, int N);
int clusten_scanline_rank(const float* pos, int64_t* ranking, void* workspace, size_t workspace_bytes,
                          int B, int N, int rows, int cols, float cell_w, float cell_h, clusten_stream stream);

/* What `space_filling_cluster` does with the ranking (models/point_utils.py:161-208): the positions in cluster order
 * and the mean position of every cluster of m consecutive tokens of that order,
 *   pos_sorted[b,i] = pos[b, ranking[b,i]]          centres[b,g] = mean of pos_sorted[b, g*m .. min(g*m+m, N))
 * (a short last cluster is averaged over the tokens it has, as the reference's masked mean does).  pos, pos_sorted
 * (B,N,2), centres (B,ceil(N/m),2): fp32, 8-byte aligned; ranking (B,N) int64, a permutation per image — unchecked;
 * pos_sorted may be NULL.  No counterpart in the reference's extension modules. */
int clusten_cluster_centres(const float* pos, const int64_t* ranking, float* pos_sorted, float* centres,
                            int B, int N, int m, clusten_stream stream);

/* Rows of a (B,N,.) tensor in a given order, out[b,i,:] = x[b, order[b,i], :]: the reordering of the tokens into
 * cluster order at the start of a stage (`feat.gather(index=ranking.expand(...), dim=1)`,
 * models/aff_transformer.py:465-466) without an index per element.  Rows of row_bytes bytes (a multiple of 16, else
 * CLUSTEN_ERR_BAD_DIMS), x and out 16-byte aligned; order (B,N) int64 with values in [0,N) — unchecked —, or (N) for
 * every image when order_shared != 0.  No counterpart in the reference's extension modules. */
int clusten_gather_rows(const void* x, const int64_t* order, void* out, int64_t B, int N, int row_bytes,
                        int order_shared, clusten_stream stream);

/* The merge centres of the adaptive down-sampling (`ClusterMerging.forward`, models/aff_transformer.py:296-334):
 *   prior   = 1 where both coordinates of the token are multiples of its grid spacing, else 0; the spacing is
 *             `stride` when min_dist is NULL (:297), else 2^(ceil(log2(min_dist)) + 1) per token (:299-303)
 *   score   = prior + learned_prob * alpha (product rounded in prob_dtype, :306-309; skipped when learned_prob is NULL)
 *             + (-100 where both coordinates are multiples of 2*stride, when reserve_on, :312-315)
 *   centre[b, 0 .. sample_num)                = the sample_num tokens of image b with the highest score (:320)
 *   centre[b, sample_num .. +reserve_num)     = with reserve_on, the tokens on that coarse grid, ascending index (:323)
 * `topk(sorted=False)` leaves the order of the sampled tokens open; here it is fixed: the tokens whose score is above
 * the sample_num-th highest by ascending index, then as many of those equal to it as are needed, by ascending index.
 * pos (B,N,2) fp32, 8-byte aligned; min_dist (B,N) fp32 or NULL; learned_prob (B,N) of prob_dtype or NULL; centre
 * (B, sample_num + (reserve_on ? reserve_num : 0)) int64.  An image should hold reserve_num tokens on the coarse
 * grid (the reference's reshape demands exactly that many and raises otherwise): further ones are left out, and the
 * slots of missing ones hold -1, which clusten_merge_rows reads as row 0.  0 < sample_num, sample_num
 * [+ reserve_num] <= N <= clusten_merge_centres_max_tokens(), else CLUSTEN_ERR_BAD_DIMS.  No counterpart in the
 * reference's extension modules. */
int clusten_merge_centres_max_tokens(void);
int clusten_merge_centres(const float* pos, const float* min_dist, const void* learned_prob, int prob_dtype,
                          int64_t* centre, int B, int N, int sample_num, int reserve_num, int reserve_on, float alpha,
                          int stride, clusten_stream stream);

/* The rows of up to four per-token tensors at the merge centres in one launch (the `gather` calls of
 * models/aff_transformer.py:337-344 on pos, member_idx, pe_idx and cluster_mask):
 *   dst[t][b,i,:] = src[t][b, centre[b,i], :]      t < count, 1 <= count <= 4
 * src[t] (B,N,.) and dst[t] (B,n_out,.) contiguous with rows of row_bytes[t] bytes, a multiple of 8 (else
 * CLUSTEN_ERR_BAD_DIMS), 8-byte aligned (else CLUSTEN_ERR_UNALIGNED); src, dst and row_bytes are host arrays of
 * `count` entries; centre (B,n_out) int64 with values in [0,N); a value outside that range reads row 0.  No
 * counterpart in the reference's extension modules. */
int clusten_merge_rows(const void* const* src, void* const* dst, const int* row_bytes, int count,
                       const int64_t* centre, int64_t B, int N, int n_out, clusten_stream stream);

/* ---- producer of the neighbourhood lists (optional) ------------------------------------------- */

/* K nearest neighbours of 2-D points inside each batch element: for query point q of batch element b,
 * idx[b,q,0..K) are the indices of the K database points of b nearest to it, ascending Euclidean
 * distance, equal distances by ascending index; dist (may be NULL) holds the distances.
 * Replaces knn_keops (models/point_utils.py:27-58; call sites models/aff_transformer.py:298,476), which
 * delegates to an external library and leaves the order of equal distances to it.
 *   query (B,Nq,2), database (B,N,2): fp32 contiguous; idx (B,Nq,K): int64; dist (B,Nq,K): fp32.
 * 1 <= K <= 8 and K <= N, else CLUSTEN_ERR_BAD_DIMS. */
int clusten_knn2d(const float* query, const float* database, int64_t* idx, float* dist,
                  int B, int Nq, int N, int K, clusten_stream stream);

#ifdef __cplusplus
}
#endif

#endif /* CLUSTEN_HIP_H */
