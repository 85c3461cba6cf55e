/*
 * mindspeed_amd.h — C ABI of the MI355X (gfx950) MoE expert hot path.
 *
 * One shared library, libmindspeed_amd.so, exports these entry points.  They
 * take plain pointers, sizes and strides; every pointer is a device pointer
 * unless stated otherwise.  Conventions shared by all entry points:
 *
 *   - return 0 (MS_OK) on success, a non-zero ms_status otherwise; the text of
 *     the last failure on the calling thread is returned by ms_last_error();
 *   - all work is enqueued on the given stream (a hipStream_t passed as
 *     void*; NULL is the default stream); no entry point synchronises, reads
 *     device data on the host, allocates or frees device memory;
 *   - the caller owns inputs, outputs and workspace and keeps them alive until
 *     the stream has passed the call; workspace sizes come from the matching
 *     *_workspace_size function and may be over-provisioned;
 *   - strides are in elements; row data of 16-bit types is processed with
 *     16-byte vectors when pointers and strides allow it and with an
 *     element-wise path otherwise (same results).
 *
 * Each declaration cites the reference interface (paths relative to the
 * reference root) that it stands in for.  The reference reaches its vendor
 * kernels through a two-phase "GetWorkspaceSize / run on stream" C ABI
 * (mindspeed/ops/csrc/cann/inc/aclnn_common.h:587-644); this header keeps that
 * two-phase shape.
 */
#ifndef MINDSPEED_AMD_H_
#define MINDSPEED_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *ms_stream_t; /* hipStream_t */

typedef enum ms_status {
    MS_OK = 0,
    MS_ERR_INVALID_ARGUMENT = 1,
    MS_ERR_UNSUPPORTED = 2,
    MS_ERR_WORKSPACE_TOO_SMALL = 3,
    MS_ERR_HIP = 4
} ms_status;

typedef enum ms_dtype { MS_BF16 = 0, MS_FP16 = 1, MS_FP32 = 2 } ms_dtype;
typedef enum ms_index_dtype { MS_INT32 = 0, MS_INT64 = 1 } ms_index_dtype;

/* Largest expert id + 1 the permute sort accepts.  The sort's key range is the
 * power of two that holds num_experts_hint (MS_MAX_EXPERTS without a hint); ids
 * outside it are clamped into it (negative ones to 0, large ones to the last key)
 * and sorted as such, so no id can address memory out of range. */
#define MS_MAX_EXPERTS 1024

/* Library identification and error text (thread-local, never NULL). */
int ms_version(void);
const char *ms_last_error(void);

/* ------------------------------------------------------------------------
 * Token permute — stands in for aclnnMoeTokenPermute as called from
 * mindspeed/ops/csrc/cann/npu_moe_token_permute.cpp:65-97 (Python surface
 * mindspeed/ops/npu_moe_token_permute.py:13-20).
 *
 * indices [num_tokens, topk] (int32 or int64 expert ids) are flattened
 * token-major and stably sorted by expert id.  Outputs:
 *   permuted_tokens [num_out_tokens, hidden]   row r = tokens[sorted_indices[r] / topk]
 *   row_id_map      int32 [num_tokens*topk]    output row of flat position i
 *                                              (entries >= num_out_tokens are dropped rows)
 *   sorted_indices  int32 [num_out_tokens]     optional (may be NULL): flat position of row r,
 *                                              the order the torch path returns
 *                                              (mindspeed/core/transformer/moe/moe_utils.py:206-208)
 *   tokens_per_expert int64 [num_experts_hint] optional (may be NULL; needs num_experts_hint > 0)
 * num_experts_hint: number of experts if known (bounds the sort's key range),
 * 0 if unknown (MS_MAX_EXPERTS is assumed).
 * ---------------------------------------------------------------------- */
int ms_moe_token_permute_workspace_size(int64_t num_tokens, int64_t topk,
                                        int64_t num_experts_hint, size_t *bytes);
int ms_moe_token_permute(ms_stream_t stream, const void *tokens, const void *indices,
                         int index_dtype, int64_t num_tokens, int64_t topk, int64_t hidden,
                         int dtype, int64_t num_out_tokens, int64_t num_experts_hint,
                         void *permuted_tokens, int32_t *row_id_map, int32_t *sorted_indices,
                         int64_t *tokens_per_expert, void *workspace, size_t workspace_bytes);

/* Token permute backward — stands in for aclnnMoeTokenPermuteGrad
 * (npu_moe_token_permute.cpp:99-118):
 *   grad_tokens[t] = sum_j grad_permuted[row_id_map[t*topk+j]]  (dropped rows add 0),
 * accumulated in fp32 and rounded once. */
int ms_moe_token_permute_grad(ms_stream_t stream, const void *grad_permuted_tokens,
                              const int32_t *row_id_map, int64_t num_tokens, int64_t topk,
                              int64_t hidden, int dtype, int64_t num_permuted_rows,
                              void *grad_tokens);

/* Token unpermute — stands in for aclnnMoeTokenUnpermute
 * (mindspeed/ops/csrc/cann/npu_moe_token_unpermute.cpp:95-122; Python surface
 * mindspeed/ops/npu_moe_token_unpermute.py:13-22):
 *   out[t] = sum_j probs[t,j] * permuted[row_id_map[t*topk+j]]
 * probs may be NULL (unweighted sum); probs_dtype is their own element type: dtype, or MS_FP32
 * (fp32 router probabilities beside 16-bit tokens are used unrounded).  fp32 accumulation, one
 * rounding to the tokens' dtype. */
int ms_moe_token_unpermute(ms_stream_t stream, const void *permuted_tokens,
                           const int32_t *row_id_map, const void *probs, int probs_dtype,
                           int64_t num_tokens, int64_t topk, int64_t hidden, int dtype,
                           int64_t num_permuted_rows, void *unpermuted_tokens);

/* Token unpermute backward — stands in for aclnnMoeTokenUnpermuteGrad
 * (npu_moe_token_unpermute.cpp:124-148):
 *   grad_permuted[row_id_map[t*topk+j]] = probs[t,j] * grad_out[t]
 *   grad_probs[t,j] = <grad_out[t], permuted[row_id_map[t*topk+j]]>   (fp32 dot)
 * probs / grad_probs / permuted_tokens may be NULL together (then
 * grad_permuted[row] = grad_out[token of row]).  probs and grad_probs share probs_dtype. */
int ms_moe_token_unpermute_grad(ms_stream_t stream, const void *permuted_tokens,
                                const void *grad_unpermuted_tokens, const int32_t *row_id_map,
                                const void *probs, int probs_dtype, int64_t num_tokens, int64_t topk,
                                int64_t hidden, int dtype, int64_t num_permuted_rows,
                                void *grad_permuted_tokens, void *grad_probs);

/* ------------------------------------------------------------------------
 * Routing-map (mask) mode of permute / unpermute — stands in for
 * torch_npu.npu_moe_token_permute_with_routing_map[_grad] and
 * torch_npu._npu_moe_token_unpermute_with_routing_map[_grad] as called from
 * mindspeed/te/pytorch/permutation.py:23-24,52-60,84-86,118-142 (Python surface
 * mindspeed/core/fusions/fused_moe_permute.py:50-85).
 *
 * routing_map [num_tokens, num_experts] bytes (torch.bool).  Flat entry
 * i = t*num_experts + e.  Without drop-and-pad the set entries are laid out
 * expert-major, token-ascending:
 *   permuted_tokens [num_out_tokens, hidden]     row r = tokens[sorted_flat[r] / num_experts]
 *   row_id_map  int32 [num_tokens*num_experts]   output row of flat entry i; unset entries and
 *                                                rows >= num_out_tokens hold 0x7fffffff (dropped)
 *   sorted_flat int32 [num_out_tokens]           flat entry of row r (-1 for a row nothing maps to,
 *                                                which only happens when num_out_tokens exceeds the
 *                                                number of set entries; such rows are not written)
 *   tokens_per_expert int64 [num_experts]        optional: set entries per expert
 * With drop_and_pad != 0, num_out_tokens = num_experts * capacity and expert e owns rows
 * [e*capacity, (e+1)*capacity): its routed tokens in ascending order, then (as padding) its
 * non-routed tokens in ascending order, cut at capacity — the selection
 * routing_map.T.argsort(descending, stable)[:, :capacity] makes; tokens_per_expert = capacity.
 * tokens / permuted_tokens may be NULL to compute the maps only (unpermute needs them again).
 * Permuted rows that no entry maps to (num_out_tokens above the number of set entries) are zeros.
 * The row maps plug into ms_moe_token_permute_grad / ms_moe_token_unpermute[_grad] with
 * topk = num_experts.
 *
 * ms_moe_routing_map_probs:      permuted_probs[r] = probs.flat[sorted_flat[r]] (0 for r unmapped),
 *                                sorted_token_ids[r] = sorted_flat[r] / num_experts (int64, the
 *                                sorted_indices the Python surface returns); either output may be NULL.
 * ms_moe_routing_map_probs_grad: grad_probs.flat[i] = grad_permuted_probs[row_id_map[i]], 0 for
 *                                dropped entries.
 * ---------------------------------------------------------------------- */
int ms_moe_routing_map_workspace_size(int64_t num_tokens, int64_t num_experts, int drop_and_pad,
                                      size_t *bytes);
int ms_moe_routing_map_permute(ms_stream_t stream, const void *tokens, const void *routing_map,
                               int64_t num_tokens, int64_t num_experts, int64_t hidden, int dtype,
                               int64_t num_out_tokens, int drop_and_pad, void *permuted_tokens,
                               int32_t *row_id_map, int32_t *sorted_flat, int64_t *tokens_per_expert,
                               void *workspace, size_t workspace_bytes);
int ms_moe_routing_map_probs(ms_stream_t stream, const int32_t *sorted_flat, int64_t num_out_tokens,
                             int64_t num_experts, const void *probs, int dtype, void *permuted_probs,
                             int64_t *sorted_token_ids);
int ms_moe_routing_map_probs_grad(ms_stream_t stream, const int32_t *row_id_map, int64_t num_entries,
                                  const void *grad_permuted_probs, int dtype, int64_t num_out_tokens,
                                  void *grad_probs);
/* Rows of a [num_out_tokens, hidden] matrix in permuted layout that no map entry leads to (sorted_flat[r] < 0:
 * only when num_out_tokens exceeds the number of set entries) are written as zeros, all others left alone.
 * The gradient of the routing-map unpermute w.r.t. the permuted rows (torch_npu.npu_moe_token_unpermute_with_
 * routing_map_grad behind mindspeed/te/pytorch/permutation.py:107-148) is completed with it, so that no row of it
 * is left unwritten. */
int ms_moe_zero_unmapped_rows(ms_stream_t stream, const int32_t *sorted_flat, int64_t num_out_tokens,
                              int64_t hidden, int dtype, void *rows);

/* ------------------------------------------------------------------------
 * Grouped matmul — stands in for aclnnGroupedMatmulV2 / V4 as called from
 * mindspeed/ops/csrc/cann/gmm.cpp:77-167 (Python surface
 * mindspeed/ops/gmm.py:164-175), including the backward recipes of
 * gmm.cpp:169-246 which are further calls of the same entry point on
 * transposed views, and, with accumulate != 0, for the ATB
 * GroupedMatmulInplaceAdd call of
 * mindspeed/ops/csrc/atb/groupmatmul_add.cpp:39-64.
 *
 * group_type 0 (split on rows of x):
 *     x [m, k], weight [num_groups, k, n], y [m, n];
 *     y[o_g:o_{g+1}] = x[o_g:o_{g+1}] @ weight[g]; rows past the last offset are zero.
 * group_type 2 (split on the reduction dim):
 *     x [k, m] (normally a transposed view), weight [m, n], y [num_groups, k, n];
 *     y[g] = x[:, o_g:o_{g+1}] @ weight[o_g:o_{g+1}]; an empty group gives zeros.
 * group_list: device int64 [num_groups]; group_list_type 0 = cumulative
 * offsets (npu_gmm), 1 = per-group counts (npu_gmm_v2).  It is never read on
 * the host.
 * x / weight are addressed through explicit element strides, so transposed
 * views need no copy; for each of x and weight one of the two matrix strides
 * must be 1.  y is row-major with row stride y_stride_row (group_type 2:
 * group stride k*y_stride_row).
 * dtype: element type of x and weight (bf16 / fp16: MFMA 32x32x16 with fp32
 * accumulation; fp32: MFMA 32x32x2 fp32).  out_dtype: dtype, or MS_FP32.
 * accumulate != 0: y += result (requires out_dtype == MS_FP32).
 * ---------------------------------------------------------------------- */
int ms_gmm_workspace_size(int64_t num_groups, int64_t m, int group_type, size_t *bytes);
/* The second form of the workspace query (the GetWorkspaceSize half of the two-phase aclnnGroupedMatmul
 * call, aclnn_common.h:587-644, sees all operands too): at least ms_gmm_workspace_size, and up to 32 MiB
 * more where ms_gmm may then split the reduction of small tail tiles.  That applies to group_type 0 with a
 * 16-bit output when the launch has few rounds of tiles and k >= 4096: the 64- / 128-row tile that ends a
 * ragged group is computed in up to 4 parts along k (fp32 partial sums in the workspace, added in part
 * order and rounded once by a second small kernel), so that the last round of the launch does not leave
 * most compute units waiting for a few long tiles.  With the smaller workspace ms_gmm runs unsplit; results of
 * the two differ by the rounding of the summation order in the rows of those tail tiles only. */
int ms_gmm_workspace_size_split(int64_t num_groups, int64_t m, int64_t k, int64_t n, int group_type,
                                int dtype, int out_dtype, int accumulate, size_t *bytes);
/* Diagnostic, host only (no counterpart in the reference): which tile of a group of num_row_tiles x
 * num_col_tiles output tiles the grouped-matmul kernels take as their index-th (blocks of 4 row tiles x 8
 * column panels, chosen for L2 reuse).  Evaluates the function the kernels call, so a test can check that
 * the order visits every tile exactly once. */
int ms_gmm_tile_order(int num_row_tiles, int num_col_tiles, int index, int *row_tile, int *col_tile);
/* Diagnostic, host only (no counterpart in the reference): the number of workgroups per XCD (an eighth of the
 * grid) that ms_gmm launches for a 16-bit problem of these sizes.  lists: the launch may deal whole groups out to
 * single XCDs (16 to 256 groups); split: it may split the reduction of its tail tiles.  A test can check with it
 * that no table the schedule kernel writes needs more slots than the launch has: with per-XCD lists and a split on
 * the reduction dim (group_type 2) the fullest XCD holds ceil(num_groups / 8) whole output blocks. */
int ms_gmm_launch_slots(int64_t num_groups, int64_t m, int64_t k, int64_t n, int group_type, int lists,
                        int split, int64_t *slots_per_xcd);
int ms_gmm(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1,
           const void *weight, int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1,
           void *y, int64_t y_stride_row, const int64_t *group_list, int group_list_type,
           int group_type, int64_t num_groups, int64_t m, int64_t k, int64_t n, int dtype,
           int out_dtype, int accumulate, void *workspace, size_t workspace_bytes);

/* ms_gmm for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same arguments without the workspace pair, the same
 * kernels and the results of ms_gmm with the workspace of ms_gmm_workspace_size (tail tiles are never
 * split).  It has no counterpart in the reference, whose shims always draw a workspace
 * from the framework's allocator.  The tile table lives in a fixed device array inside the library
 * (about 340 KB per GPU, held until the process ends), which bounds num_groups to 1024; more groups
 * report MS_ERR_UNSUPPORTED.  The call allocates and frees nothing.  The first call on a device looks
 * the array's address up (hipGetSymbolAddress), so make that call outside a graph capture.  All calls
 * on one GPU share the array: calls that may overlap on one GPU (different streams, different
 * threads) race on it and must be ordered by the caller. */
int ms_gmm_noalloc(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1,
                   const void *weight, int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1,
                   void *y, int64_t y_stride_row, const int64_t *group_list, int group_list_type,
                   int group_type, int64_t num_groups, int64_t m, int64_t k, int64_t n, int dtype,
                   int out_dtype, int accumulate);

/* First grouped matmul of an expert MLP with the SwiGLU (x per-row probability) activation fused into
 * its epilogue: the op sequence fc1 = gmm(x, w1); act = (silu(gate) * up * probs).to(dtype) of
 * mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:113-127 (activation: :41-44) in one launch.
 * weight [num_groups, k, 2*ffn] (gate columns first); y [m, 2*ffn] receives the fc1 output (kept
 * for backward; may be NULL), act [m, ffn] the activation, computed from the rounded fc1 values
 * exactly as ms_swiglu computes it from y.  probs: optional [m] (bf16 / fp16 / fp32).  group_type 0
 * only; bf16 / fp16; needs the vector-access layout (16-byte aligned pointers, x contiguous along k,
 * weight contiguous along its columns, k, ffn and all strides multiples of 8) and reports
 * MS_ERR_UNSUPPORTED otherwise.  Workspace size: ms_gmm_workspace_size. */
int ms_gmm_swiglu(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1,
                  const void *weight, int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1,
                  void *y, int64_t y_stride_row, void *act, int64_t act_stride_row, const void *probs,
                  int probs_dtype, const int64_t *group_list, int group_list_type, int64_t num_groups,
                  int64_t m, int64_t k, int64_t ffn, int dtype, void *workspace, size_t workspace_bytes);

/* Backward counterpart: dact = dy @ W2^T (the dX product of the second grouped matmul) with the
 * SwiGLU backward of mindspeed/ops/csrc/atb/swiglu.cpp:96-126 (and the probability factor of
 * experts.py:41-44) fused into its epilogue, so dact is never written:
 *   d_fc1[r, c]       = dact[r, c] * probs[r] * up   * sig * (1 + gate * (1 - sig))
 *   d_fc1[r, ffn + c] = dact[r, c] * probs[r] * gate * sig            (sig = sigmoid(gate))
 *   grad_probs[r]     = sum_c dact[r, c] * gate * sig * up            (fp32; summed per 64 columns
 *                       in the epilogue, then over the row by a second small kernel)
 * with gate = fc1[r, c], up = fc1[r, ffn + c] and dact rounded to dtype first, i.e. the values
 * ms_gmm followed by ms_swiglu_grad produce.  dy [m, k]; weight is the transposed view of
 * W2 [num_groups, ffn, k] (w_stride0 = 1 along k, w_stride1 = k along ffn); fc1 / d_fc1 [m, 2*ffn];
 * probs / grad_probs optional together.  Same layout conditions as ms_gmm_swiglu. */
int ms_gmm_swiglu_grad_workspace_size(int64_t num_groups, int64_t m, int64_t ffn, size_t *bytes);
int ms_gmm_swiglu_grad(ms_stream_t stream, const void *dy, int64_t dy_stride0, int64_t dy_stride1,
                       const void *weight, int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1,
                       const void *fc1, int64_t fc1_stride_row, const void *probs, int probs_dtype,
                       void *d_fc1, int64_t d_fc1_stride_row, void *grad_probs,
                       const int64_t *group_list, int group_list_type, int64_t num_groups, int64_t m,
                       int64_t k, int64_t ffn, int dtype, void *workspace, size_t workspace_bytes);

/* The same product (group_type 0 only) with one separately allocated weight matrix per group —
 * the form torch_npu.npu_grouped_matmul([x], [w_0 .. w_{E-1}], ...) takes from
 * mindspeed/te/pytorch/module/grouped_linear.py:61-69,85-93 (per-expert parameters
 * weight0 .. weight{E-1}, :196-222).  weights: HOST array of num_groups device pointers; every
 * matrix is [k, n] addressed with the same element strides (w_stride0, w_stride1), so the
 * [n, k] parameters are read in place as transposed views.  At most 256 groups (the pointer
 * differences travel as a kernel argument; stack the weights and use ms_gmm beyond that).
 * Workspace size: ms_gmm_workspace_size. */
int ms_gmm_weight_list(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1,
                       const void *const *weights, int64_t w_stride0, int64_t w_stride1, void *y,
                       int64_t y_stride_row, const int64_t *group_list, int group_list_type,
                       int64_t num_groups, int64_t m, int64_t k, int64_t n, int dtype, int out_dtype,
                       void *workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * SwiGLU (+ optional per-row probability) — stands in for the ATB
 * ACTIVATION_SWIGLU_FORWARD / BACKWARD calls of
 * mindspeed/ops/csrc/atb/swiglu.cpp:64-126 and the probs product of
 * mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:41-44:
 *   y[r, c] = silu(x[r, c]) * x[r, ffn + c] * (probs ? probs[r] : 1)
 * x [rows, 2*ffn], y [rows, ffn], probs fp32-or-dtype [rows] (probs_dtype).
 * Backward writes grad_x [rows, 2*ffn] and, if probs, grad_probs [rows]
 * (same dtype as probs). fp32 math, one rounding.
 * ---------------------------------------------------------------------- */
int ms_swiglu(ms_stream_t stream, const void *x, const void *probs, int probs_dtype,
              int64_t rows, int64_t ffn, int dtype, void *y);
int ms_swiglu_grad(ms_stream_t stream, const void *grad_y, const void *x, const void *probs,
                   int probs_dtype, int64_t rows, int64_t ffn, int dtype, void *grad_x,
                   void *grad_probs);

/* ------------------------------------------------------------------------
 * Chunk sort — stands in for sort_chunks_by_idxs of the alltoall dispatcher
 * (torch statement: mindspeed/core/transformer/moe/moe_feature/overlap/
 * moe_common.py:377-398; fused form: mindspeed/lite/ops/triton/
 * sort_chunks_by_idx.py:300-348):
 *   out = cat([split(input, split_sizes)[i] for i in sorted_idxs])
 * split_sizes int64 [num_chunks] and sorted_idxs int64 [num_chunks] are device
 * arrays.  row_map int32 [rows] receives the source row of every output row
 * (the backward is the same call with the inverse map, see ms_gather_rows).
 * probs (optional, [rows], probs_dtype) are reordered into out_probs.
 * ---------------------------------------------------------------------- */
int ms_sort_chunks(ms_stream_t stream, const void *input, const int64_t *split_sizes,
                   const int64_t *sorted_idxs, int64_t num_chunks, int64_t rows, int64_t hidden,
                   int dtype, const void *probs, int probs_dtype, void *out, void *out_probs,
                   int32_t *row_map);
/* out[r] = input[row_map[r]] (inverse != 0: out[row_map[r]] = input[r]). */
int ms_gather_rows(ms_stream_t stream, const void *input, const int32_t *row_map, int64_t rows,
                   int64_t hidden, int dtype, int inverse, void *out);

/* The chunk sort's row map alone, in the direction make_chunk_sort_map of the fused form returns it
 * (mindspeed/lite/ops/triton/sort_chunks_by_idx.py:67-115): row_id_map int32 [rows], entry r = output row of
 * source row r (-1 for rows past the sum of the sizes).  ms_gather_rows moves rows by it: inverse != 0 is the
 * forward direction of sort_chunks_by_map (:167-221), inverse == 0 its backward. */
int ms_chunk_sort_map(ms_stream_t stream, const int64_t *split_sizes, const int64_t *sorted_idxs,
                      int64_t num_chunks, int64_t rows, int32_t *row_id_map);
#ifdef __cplusplus
}
#endif
#endif /* MINDSPEED_AMD_H_ */
