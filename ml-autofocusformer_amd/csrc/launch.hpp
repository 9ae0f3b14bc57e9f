// Internal launch functions behind the C ABI.  Each one validates nothing: the extern "C" layer
// has already checked pointers, sizes and strides.  All return a clusten_status.
#pragma once

#include "common.hpp"

namespace clusten {

// An entry of a pair list (cluster_pairs.hip) names run r of token i of its image as i << kPairRunBits | r: lists of
// up to 256 slots, i.e. 32 runs of 8.  Bit 30 flags the second listing of a pair that names a short last cluster.
constexpr int kPairRunBits = 5;
constexpr int kPairRunMask = (1 << kPairRunBits) - 1;
constexpr int kPairMaxSlots = 8 << kPairRunBits;


// out[b,h,i,j] = sum_c a[b,h,i,c] * rows[b,h,idx[b,i,j],c]      (QK forward; AV's d_attn)
//   a, rows : strided (B,H,N,C);  out : contiguous (B,H,N,M)
int launch_gather_dot(const void* a, clusten_strides a_strides, const void* rows, clusten_strides rows_strides,
                      const int64_t* idx, void* out, clusten_attn_shape s, int dtype, hipStream_t stream);

// The same with the lists given as cluster numbers: cluster_idx (B,N,M/8) int32, slot j of a token = row
// 8*g + j%8 of its cluster number j/8 (row 0 where that is >= N).  F32/F16/BF16, C in {16,32,64}, M % 8 == 0, M <= 64.
int launch_gather_dot_clusters(const void* a, clusten_strides a_strides, const void* rows, clusten_strides rows_strides,
                               const int32_t* cluster_idx, void* out, clusten_attn_shape s, int dtype,
                               hipStream_t stream);

// out[b,h,i,c] = sum_j p[b,h,i,j] * rows[b,h,idx[b,i,j],c]      (AV forward; QK's d_query)
//   p : contiguous (B,H,N,M);  rows, out : strided (B,H,N,C)
int launch_gather_sum(const void* p, const void* rows, clusten_strides rows_strides, const int64_t* idx, void* out,
                      clusten_strides out_strides, clusten_attn_shape s, int dtype, hipStream_t stream);

// The same for fp32 p and out over rows of rows_dtype = F16 / BF16, read in place (equal to a cast of the rows first).
int launch_gather_sum_mixed(const void* p, const void* rows, clusten_strides rows_strides, const int64_t* idx, void* out,
                            clusten_strides out_strides, clusten_attn_shape s, int rows_dtype, hipStream_t stream);

// Cluster size the cluster-number forms read a list of M slots in: 8 up to 64 slots, then the run length of the kernels
// for long runs (24, 32 or 16; gather_runs_impl.hpp), 0 when M is neither.
int cluster_size_for(int M);
// The same with the lists given as cluster numbers (see launch_gather_dot_clusters).
int launch_gather_sum_clusters(const void* p, const void* rows, clusten_strides rows_strides, const int32_t* cluster_idx,
                               void* out, clusten_strides out_strides, clusten_attn_shape s, int dtype,
                               hipStream_t stream);

// out[b,h,idx[b,i,j],c] += p[b,h,i,j] * x[b,h,i,c]               (QK's d_key; AV's d_value)
//   p : contiguous (B,H,N,M);  x : strided (B,H,N,C);  out : contiguous (B,H,N,C), zeroed here.
//   Lists made of whole clusters (found out on the device) go through pair lists in `workspace` and a gather without
//   atomics; for any other list the sum is built with fp32 atomics (for F16/BF16 in `workspace`, rounded once).
//   `pair_lists` (may be null): the block launch_cluster_pairs filled for these lists (layout cluster_pairs_layout(B,
//   N, M, N)); the pair lists are then not rebuilt in the workspace.
size_t scatter_rows_workspace_bytes(clusten_attn_shape s, int dtype);
int launch_scatter_rows(const void* p, const void* x, clusten_strides x_strides, const int64_t* idx, void* out,
                        void* workspace, clusten_attn_shape s, int dtype, hipStream_t stream,
                        const void* pair_lists = nullptr);

// out[b,i,ic,c] = sum_j w[b,i,j,ic] * feat[b,idx[b,i,j],c]      (WF forward)
int launch_wf_forward(const void* w, const void* feat, const int64_t* idx, void* out, clusten_wf_shape s, int dtype,
                      hipStream_t stream);

// The same for fp32 w and out over feat of feat_dtype = F16 / BF16, read in place (equal to a cast of feat first).
int launch_wf_forward_mixed(const void* w, const void* feat, const int64_t* idx, void* out, clusten_wf_shape s,
                            int feat_dtype, hipStream_t stream);

// d_w[b,i,j,ic] = sum_c feat[b,idx[b,i,j],c] * d_out[b,i,ic,c]  (WF backward, weights)
int launch_wf_dweights(const void* d_out, const void* feat, const int64_t* idx, void* d_w, clusten_wf_shape s,
                       int dtype, hipStream_t stream);

// d_feat[b,idx[b,i,j],c] += sum_ic d_out[b,i,ic,c] * w[b,i,j,ic]  (WF backward, features; zeroed here)
size_t wf_dfeat_workspace_bytes(clusten_wf_shape s, int dtype);
int launch_wf_dfeat(const void* d_out, const void* w, const int64_t* idx, void* d_feat, void* workspace,
                    clusten_wf_shape s, int dtype, hipStream_t stream);

// probs[b,h,i,:M], blank_prob[b,h,i] = softmax over j <= M of
//   attn[b,h,i,j] + table[pe_idx[b,i,j], h] - 100 * (1 - mask[b,i,j])  (j < M)  and  blank[b,h,i]  (j = M)
//   attn, table : T;  pe_idx, mask (may be null) : int64 (B,N,M);  blank, probs, blank_prob : fp32.  M <= 64, M % 4 == 0.
//   With q (strided (B,H,N,C), T) and blank_k ((H,C), fp32) given, blank[b,h,i] is computed here as their dot product.
int launch_attn_softmax(const void* attn, const void* table, const int64_t* pe_idx, const int64_t* mask,
                        const float* blank, const void* q, clusten_strides qs, const float* blank_k, float* probs,
                        float* blank_prob, clusten_attn_shape s, int dtype, hipStream_t stream);

// Local attention of a cluster-ordered sequence in one kernel (QK, position bias, mask, blank token, softmax, AV,
// blank value): see cluster_attention.hip.  q, k, v, out : strided (B,H,N,C) of T in {F16, BF16, F32}, C = 32;
//   cluster_idx (B,N,6) int32; table (rows,H) of T; pe_idx, mask (may be null) : int64 (B,N,M) — or (1,N,.) each
//   when lists_shared; M = 48 (clusters of 8) or, for 16-bit data, 144 (clusters of 24);
//   blank_k, blank_v : fp32 (H,C);  lse (may be null): fp32 (B,H,N), the logarithm of each softmax's denominator.
int launch_cluster_attention(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                             clusten_strides vs, const int32_t* cluster_idx, const void* table, const int64_t* pe_idx,
                             const int64_t* mask, const float* blank_k, const float* blank_v, void* out,
                             clusten_strides os, float scale, int lists_shared, const void* plan, float* lse,
                             clusten_attn_shape s, int dtype, hipStream_t stream);
// The query-side half of that kernel's backward (16-bit data): d_q, the recomputed probabilities and the logit
// gradients as (B,H,N,48) tensors of T, the blank token's probability and logit gradient as fp32 (B,H,N): see
// cluster_attention_bwd.hip.  d_out, out: strided (B,H,N,C) like q; lse: what the forward wrote.
int launch_cluster_attention_backward(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                                      clusten_strides vs, const void* d_out, clusten_strides gs, const void* out,
                                      clusten_strides os, const float* lse, const int32_t* cluster_idx, const void* table,
                                      const int64_t* pe_idx, const int64_t* mask, const float* blank_k,
                                      const float* blank_v, void* d_q, clusten_strides dqs, void* probs, void* d_logit,
                                      float* p_blank, float* ds_blank, float scale, int lists_shared, const void* plan,
                                      clusten_attn_shape s, int dtype, hipStream_t stream);
// The per-tile plan the kernel above reads instead of cluster_idx, pe_idx and mask when it is given one (what it
// would work out from them before its first head): B = batch elements of the index tensors, M = 48 or 144.
size_t cluster_attention_plan_bytes(int B, int N, int M);
int launch_cluster_attention_plan(const int32_t* cluster_idx, const int64_t* pe_idx, const int64_t* mask, void* plan,
                                  int B, int N, int M, hipStream_t stream);

// The pair lists of lists made of whole clusters (cluster_pairs.hip), built on the device: for `rows` list rows per
//   image of M slots that point into a sequence of D rows (K = ceil(D/8) clusters), pairs[starts[b*K+g] .. ends[b*K+g])
//   holds the entries i*8 + r whose run r of list row i is cluster g of image b, ascending; *not_whole becomes 1 when
//   some run is not a whole cluster (then the other outputs mean nothing), else 0.  `keys` and `wg_bad` are scratch.
//   Sizes as cluster_pairs_layout() gives them (byte offsets into one 16-byte aligned block, `bytes` in all).
struct ClusterPairsLayout {
    size_t flag, wg_bad, keys, pairs, starts, ends, bytes;
};
bool cluster_pairs_supported(int B, int rows, int M, int D);
ClusterPairsLayout cluster_pairs_layout(int B, int rows, int M, int D);
// `numbers` != nullptr: the lists as (B,rows,M/8) int32 cluster numbers instead of `idx` (not read then); a number
//   outside [0, ceil(D/8)) raises *not_whole.
int launch_cluster_pairs(const int64_t* idx, int32_t* keys, int32_t* wg_bad, int32_t* not_whole, int32_t* pairs,
                         int32_t* starts, int32_t* ends, int B, int rows, int M, int D, hipStream_t stream,
                         const int32_t* numbers = nullptr);
// The entries (i, j) of a list tensor (B, rows, M) by the row of the D-row sequence they name, built on the device
//   (cluster_pairs.hip): entries[starts[b*D+n] .. ends[b*D+n]) holds e = i*M + j for every idx[b,i,j] = n, ascending.
//   `only_if` (may be null): device flag; nothing is done when it points to zero.  Sizes as row_entries_layout() gives
//   them (byte offsets into one 16-byte aligned block).
struct RowEntriesLayout {
    size_t entries, starts, ends, bytes;
};
bool row_entries_supported(int B, int rows, int M, int D);
RowEntriesLayout row_entries_layout(int B, int rows, int M, int D);
int launch_row_entries(const int64_t* idx, const int32_t* only_if, int32_t* entries, int32_t* starts, int32_t* ends, int B,
                       int rows, int M, int D, hipStream_t stream);
// d_feat[b,n,:] = sum over the entries (i,j) of row (b,n) of sum_ic w[b,i,j,ic] * d_out[b,i,ic,:]: see wf_dfeat_rows.hip.
bool wf_dfeat_rows_supported(const void* d_out, const void* d_feat, const clusten_wf_shape& s, int dtype);
int launch_wf_dfeat_rows(const void* d_out, const void* w, const int32_t* starts, const int32_t* ends,
                         const int32_t* entries, const int32_t* only_if, void* d_feat, clusten_wf_shape s, int dtype,
                         hipStream_t stream);

// y[b,h,8g+t,:] = sum over the listed pairs (i,r) of cluster (b,g) of p[b,h,i,8r+t] * x[b,h,i,:]: see scatter_by_cluster.hip.
//   C in {16,32,64}.  `not_whole` (may be null): device flag; the kernel does nothing when it points to non-zero.
bool scatter_by_cluster_supported(const void* p, const void* x, clusten_strides xs, const void* y,
                                  const clusten_attn_shape& s, int dtype);
int launch_scatter_by_cluster(const void* p, const void* x, clusten_strides xs, const int32_t* starts, const int32_t* ends,
                              const int32_t* pairs, const int32_t* not_whole, void* y, clusten_attn_shape s, int dtype,
                              hipStream_t stream);
// d_feat[b,8g+t,:] = sum over the listed pairs (i,r) of cluster (b,g) of sum_ic w[b,i,8r+t,ic] * d_out[b,i,ic,:]: see
//   wf_dfeat_by_cluster.hip.  IC = 4, C % 32 == 0.  `not_whole` as above.
bool wf_dfeat_by_cluster_supported(const void* d_out, const void* w, const void* d_feat, const clusten_wf_shape& s,
                                   int dtype);
int launch_wf_dfeat_by_cluster(const void* d_out, const void* w, const int32_t* starts, const int32_t* ends,
                               const int32_t* pairs, const int32_t* not_whole, void* d_feat, clusten_wf_shape s, int dtype,
                               hipStream_t stream);

// Attention of every token over every token (N <= 64) in one kernel: see dense_attention.hip.  q, k, v, out : strided
//   (B,H,N,C) of T in {F16, BF16}, C = 32; table (rows,H) of T; pe_idx int64 (B,N,N); blank_k, blank_v : fp32 (H,C).
int launch_dense_attention(const void* q, clusten_strides qs, const void* k, clusten_strides ks, const void* v,
                           clusten_strides vs, const void* table, const int64_t* pe_idx, const float* blank_k,
                           const float* blank_v, void* out, clusten_strides os, float scale, clusten_attn_shape s,
                           int dtype, hipStream_t stream);

// y = act(x W^T + b) for tall x and small W (see skinny_linear.hip): x (M,K) of T with row stride ldx elements,
//   w (NOUT,K), bias (NOUT) or null, y (M,NOUT), all of T in {F16, BF16}; act 0 = identity, 1 = exact GELU.
bool skinny_linear_supported(int K, int NOUT, int act);
int launch_skinny_linear(const void* x, int64_t ldx, const void* w, const void* bias, void* y, int64_t M, int K, int NOUT,
                         int act, int dtype, hipStream_t stream);

// out[r,:] = (x[r,:] - mean) * rsqrt(var + eps) * weight + bias for `rows` rows of C channels
//   (C in {64,128,256,384,512,768,1024}); x and out of dtype F32, F16 or BF16 each, arithmetic in fp32.
int launch_layer_norm(const void* x, int in_dtype, const float* weight, const float* bias, void* out, int64_t rows, int C,
                      float eps, int out_dtype, hipStream_t stream);

// layer norm of rows read in a given order (order may be null) with a per-channel bias (may be null) added first.
int launch_layer_norm_rows(const void* x, int in_dtype, const int64_t* order, int group, const void* pre_bias,
                           const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
                           int out_dtype, hipStream_t stream);

// y = GELU(x * scale[c] + shift[c]) over (B,C,HW) of T in {F16, BF16}; HW % 8 == 0.
int launch_channel_affine_gelu(const void* x, const float* scale, const float* shift, void* y, int64_t B, int C, int HW,
                               int dtype, hipStream_t stream);

// sum_out = x + branch (x's type), out = layer norm of sum_out (branch's 16-bit type); x of F32 or branch's type.
int launch_add_layer_norm(const void* x, int x_dtype, const void* branch, int branch_dtype, void* sum_out,
                          const float* weight, const float* bias, void* out, int64_t rows, int C, float eps,
                          hipStream_t stream);

// member_idx, mask (may be null), pe_idx (B,N,nnc*m) int64 and cluster_idx (B,N,nnc) int32 (may be null) from
//   nearest (B,N,nnc) int64 and pos (B,N,2) fp32: see neighbour_lists.hip.
int launch_neighbour_lists(const float* pos, const int64_t* nearest, int64_t* member_idx, int64_t* mask, int64_t* pe_idx,
                           int32_t* cluster_idx, int B, int N, int nnc, int m, int radius, int table_width,
                           hipStream_t stream);

// score[r] = sigmoid(<x[r] (+ branch[r]), w> + b) with the sum written to sum_out: see row_score.hip.
int launch_add_row_score(const void* x, int x_dtype, const void* branch, void* sum_out, const void* w, const void* b,
                         void* score, int64_t rows, int C, int dtype, hipStream_t stream);

// d_logit = probs * (d_probs - s), d_blank_logit = blank_prob * (d_blank_prob - s), s the row's sum of p * dp.
int launch_attn_softmax_backward(const float* probs, const float* blank_prob, const float* d_probs,
                                 const float* d_blank_prob, void* d_logit, float* d_blank_logit, int64_t rows, int M,
                                 int dtype, hipStream_t stream);

// d_table[pe_idx[b,i,j], h] += d_logit[b,h,i,j]; d_table (rows,H) fp32 zeroed by the caller.
int launch_bias_table_grad(const void* d_logit, const int64_t* pe_idx, float* d_table, int B, int H, int N, int M, int rows,
                           int dtype, hipStream_t stream);

// w[b,i,j,:4] = table_w[pe_idx[b,i,j], :4] * prob[b, nbhd_idx[b,i,j]] * mask[b,i,j]   (prob, mask may be null)
//   table_w (rows,4), prob (B,N), w (B,Nout,M,4): fp32;  pe_idx, nbhd_idx, mask: int64 (B,Nout,M).
int launch_merge_weights(const float* table_w, const int64_t* pe_idx, const int64_t* nbhd_idx, const float* prob,
                         const int64_t* mask, float* out, int B, int N, int Nout, int M, hipStream_t stream);

// ranking[b,:] = the order of the tokens of image b along the scan-line walk over a rows x cols anchor grid with
//   cells of cell_w x cell_h (see scanline_rank.hip).  pos (B,N,2) fp32 as (x, y); ranking (B,N) int64; N <= scanline_rank_max_tokens()
//   (the sort of an image runs in the LDS of one compute unit: 16384 tokens on an MI355X),
//   rows * cols >= 2; workspace of scanline_rank_workspace_bytes(B, N) bytes.
size_t scanline_rank_workspace_bytes(int B, int N);
int scanline_rank_max_tokens();   // the longest sequence the LDS of the current device sorts (a power of two)

// pos_sorted[b,i] = pos[b, ranking[b,i]] (may be null) and centres[b,g] = mean of the positions of tokens
//   ranking[b, g*m .. g*m+m-1] (the last cluster may be short): pos, pos_sorted (B,N,2), centres (B,ceil(N/m),2) fp32.
int launch_cluster_centres(const float* pos, const int64_t* ranking, float* pos_sorted, float* centres, int B, int N, int m,
                           hipStream_t stream);

// out[b,i,:] = x[b, order[b,i], :] for rows of row_bytes bytes (a multiple of 16); order (B,N) int64, or (N) for
//   every b when order_shared.
int launch_gather_rows(const void* x, const int64_t* order, void* out, int64_t B, int N, int row_bytes, int order_shared,
                       hipStream_t stream);
// centre[b, :] = the tokens the adaptive down-sampling keeps (models/aff_transformer.py:296-334): the sample_num tokens
//   of highest score = grid prior + prob * alpha [- 100 on the reserved grid], ascending index among those above the
//   sample_num-th score, then those equal to it; then, with reserve_on, the reserve_num reserved tokens by ascending
//   index.  pos (B,N,2) fp32; min_dist (B,N) fp32 distance to the nearest other token, or null for the regular grid of
//   `stride`; prob (B,N) of prob_dtype or null; centre (B, sample_num [+ reserve_num]) int64.
int merge_centres_max_tokens();
int launch_merge_centres(const float* pos, const float* min_dist, const void* prob, int prob_dtype, int64_t* centre, int B,
                         int N, int sample_num, int reserve_num, int reserve_on, float alpha, int stride,
                         hipStream_t stream);
// dst[t][b,i,:] = src[t][b, centre[b,i], :] for t < count <= 4 tensors (B,N,.) with rows of row_bytes[t] bytes
//   (multiples of 8); centre (B,n_out) int64.
int launch_merge_rows(const void* const* src, void* const* dst, const int* row_bytes, int count, const int64_t* centre,
                      int64_t B, int N, int n_out, hipStream_t stream);
int launch_scanline_rank(const float* pos, int64_t* ranking, void* workspace, int B, int N, int rows, int cols,
                         float cell_w, float cell_h, hipStream_t stream);

// idx[b,q,:K], dist[b,q,:K] = the K (1..8, K <= N) database points of batch element b nearest to query q,
//   ascending Euclidean distance, equal distances by index.  query (B,Nq,2), database (B,N,2): fp32;
//   idx int64; dist fp32 or null.
int launch_knn2d(const float* query, const float* database, int64_t* idx, float* dist, int B, int Nq, int N, int K,
                 hipStream_t stream);

// Fill `count` fp32 / fp64 words with zero (a kernel, so that callers may capture it in a HIP graph).
//   `only_if` (may be null): a device flag; the kernel does nothing when it points to zero.
int launch_zero_f32(float* dst, size_t count, hipStream_t stream, const int32_t* only_if = nullptr);
int launch_zero_f64(double* dst, size_t count, hipStream_t stream);

// dst[i] = round(src[i]) for i < count, T in {F16, BF16}.  `only_if` as above.
int launch_round_from_f32(const float* src, void* dst, size_t count, int dtype, hipStream_t stream,
                          const int32_t* only_if = nullptr);

}  // namespace clusten
