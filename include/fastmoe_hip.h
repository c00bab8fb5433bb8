/*
 * fastmoe_hip.h — C ABI of the MI355X (gfx950) dropless-MoE kernel library `libfastmoe_hip.so`.
 *
 * Every entry point
 *   - takes plain device pointers, 64-bit sizes/strides (in elements) and small integer enums;
 *   - launches asynchronously on the HIP stream passed last (`void *` holding a `hipStream_t`, NULL = default
 *     stream) and never synchronises, allocates or frees device memory, or keeps a caller's pointer after it
 *     returns: outputs and every workspace are the caller's, and a workspace may be reused as soon as the stream
 *     has passed the call;
 *   - returns `FM_OK` (0), a positive remark (the work was launched), or a negative `fm_status`; the message of a
 *     negative status for the calling thread is read with `fm_last_error()`. Only negative values are errors: test
 *     `status < 0`, not `status != FM_OK` (a remark leaves no message). No C++ exception crosses this boundary.
 *
 * The reference (ServiceNow/Fast-LLM) has no FFI for this path: its "operator API" is a set of Python
 * callables that launch Triton kernels. Each function below replaces the kernel launch inside one of those
 * callables; the citation names the reference launch site it stands in for.
 */
#ifndef FASTMOE_HIP_H
#define FASTMOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FM_VERSION 10

/* Element type of activations, weights and outputs. */
enum fm_dtype { FM_DTYPE_F32 = 0, FM_DTYPE_BF16 = 1, FM_DTYPE_F16 = 2 };

/* Integer type of `sparse_rows`, `expert_ends` and `expert_pad_begins`.
 * The reference picks int16 when the padded row count is below 32768, else int32
 * (fast_llm/functional/triton/sparse_copy.py:270); hand-built maps in its tests are int64
 * (tests/functional/test_sparse_matmul.py:51-62). */
enum fm_index_dtype { FM_INDEX_I16 = 0, FM_INDEX_I32 = 1, FM_INDEX_I64 = 2 };

enum fm_status {
    /* Positive: the call succeeded and was launched, with a remark. The three grouped products return this one when
     * bf16/fp16 operands had to take the bounds-checked multiply-add kernel instead of the matrix cores (a stride
     * that is not 1 on either axis, rows not 16-byte aligned, reduction not a multiple of 64, stride >= 2^21). */
    FM_NOTE_GENERIC_KERNEL = 1,
    FM_OK = 0,
    FM_ERR_INVALID_ARGUMENT = -1, /* bad enum, negative size, null pointer, misaligned/unsupported stride */
    FM_ERR_UNSUPPORTED = -2,      /* valid request that this build has no kernel for */
    FM_ERR_LAUNCH = -3            /* the HIP runtime rejected the launch */
};

/* Activation of the MLP (fast_llm/functional/config.py:50-60; the kernels implement the five the
 * reference's Triton kernels implement, fast_llm/functional/triton/mlp.py:49-67). */
enum fm_activation {
    FM_ACT_GELU = 0, /* tanh approximation */
    FM_ACT_SILU = 1,
    FM_ACT_RELU = 2,
    FM_ACT_SQUARED_RELU = 3,
    FM_ACT_IDENTITY = 4
};

/* Library / ABI version (== FM_VERSION of the header it was built from). */
int fm_version(void);

/* Message of the last failing call on this thread ("" if none). The pointer stays valid until the next
 * failing call on the same thread. */
const char *fm_last_error(void);

/* ---------------------------------------------------------------------------------------------------------
 * Routing: sparse map.
 * Replaces `sparse_histogram_kernel` + `_compute_expert_layout`
 * (fast_llm/functional/triton/sparse_copy.py:200-221, 241-255, launched from `get_sparse_map`, :272-288).
 *
 *   count[e]             = #{i : top_experts.flat[i] == e}
 *   padded[e]            = ceil(count[e] / pad_to_multiple) * pad_to_multiple
 *   expert_ends[e]       = sum_{e' <= e} padded[e']
 *   expert_pad_begins[e] = expert_ends[e] - padded[e] + count[e]
 *   sparse_rows.flat[i]  = expert_ends[e] - padded[e] + #{i' < i : top_experts.flat[i'] == e},  e = top_experts.flat[i]
 *
 * Integer only and deterministic: the result is bit-identical from run to run. Entries of `top_experts`
 * outside [0, num_experts) are not counted and get sparse row -1 (the copy kernels skip negative rows).
 *
 * `workspace` is caller-provided device scratch of at least `fm_sparse_map_workspace_size(...)` bytes,
 * 16-byte aligned; its content on entry is irrelevant and it may be reused as soon as the stream has
 * passed the call.
 * --------------------------------------------------------------------------------------------------------- */
size_t fm_sparse_map_workspace_size(int64_t num_rows_dense, int64_t num_experts_per_token, int64_t num_experts);

int fm_sparse_map(const int64_t *top_experts,   /* [num_rows_dense, num_experts_per_token], contiguous */
                  int64_t num_rows_dense, int64_t num_experts_per_token, int64_t num_experts,
                  int64_t pad_to_multiple,
                  int index_dtype,              /* fm_index_dtype of the three outputs */
                  void *sparse_rows,            /* [num_rows_dense, num_experts_per_token] */
                  void *expert_ends,            /* [num_experts] */
                  void *expert_pad_begins,      /* [num_experts] */
                  void *workspace, size_t workspace_size, void *stream);

/* The same map for callers that cannot allocate device memory or bring a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid allocation). It has no counterpart in the reference. Same arguments,
 * results and kernels as `fm_sparse_map`, but the scratch is a fixed array of FM_SPARSE_MAP_STATIC_SCRATCH_BYTES of
 * device memory inside the library (every GPU the library runs on holds its copy until the process ends), and the
 * call allocates and frees nothing. Inputs whose `fm_sparse_map_workspace_size(...)` exceeds the array are refused
 * with FM_ERR_UNSUPPORTED (1 MiB covers e.g. 131072 x 8 entries over 128 experts, or 16384 x 8 over 1024). All calls
 * on one GPU share that GPU's array: calls that may overlap (different streams, different threads) race; calls on one
 * stream are safe. The array's address is looked up at a device's first call (a host-side query, no allocation); make
 * that first call outside graph capture. The device the stream belongs to must be the current device (the array is
 * looked up for the current device and the kernels run where the stream lives): a stream of another device is
 * FM_ERR_INVALID_ARGUMENT. */
#define FM_SPARSE_MAP_STATIC_SCRATCH_BYTES (1 << 20)
size_t fm_sparse_map_static_scratch_size(void);
int fm_sparse_map_static(const int64_t *top_experts, int64_t num_rows_dense, int64_t num_experts_per_token,
                         int64_t num_experts, int64_t pad_to_multiple, int index_dtype, void *sparse_rows,
                         void *expert_ends, void *expert_pad_begins, void *stream);

/* ---------------------------------------------------------------------------------------------------------
 * Sparse copies. `scores` may be NULL (un-scored copy); otherwise [num_rows_dense, num_experts_per_token]
 * of `scores_dtype`. All row-major contiguous with `num_columns` columns. `num_rows_sparse` is the row
 * count of the sparse buffer: entries of `sparse_rows` outside [0, num_rows_sparse) are skipped (not copied, and
 * they add nothing to a combine or a score gradient, which is 0 for them), never dereferenced.
 * --------------------------------------------------------------------------------------------------------- */

/* Dispatch: output[sparse_rows[t, j], :] = input[t, :] * (scores[t, j] or 1), product in fp32, one rounding.
 * Rows of `output` that no (t, j) maps to are left untouched.
 * Replaces `copy_dense_to_sparse_kernel` (sparse_copy.py:27-49, launched at :57-65). */
int fm_copy_dense_to_sparse(const void *input, const void *scores, const void *sparse_rows, void *output,
                            int64_t num_rows_dense, int64_t num_columns, int64_t num_experts_per_token,
                            int64_t num_rows_sparse, int dtype, int scores_dtype, int index_dtype, void *stream);

/* Combine: output[t, :] = sum_{j = 0..k-1, in that order} input[sparse_rows[t, j], :] * (scores[t, j] or 1),
 * accumulated in fp32, one rounding.
 * Replaces `copy_sparse_to_dense_kernel` (sparse_copy.py:69-90, launched at :97-107). */
int fm_copy_sparse_to_dense(const void *input, const void *scores, const void *sparse_rows, void *output,
                            int64_t num_rows_dense, int64_t num_columns, int64_t num_experts_per_token,
                            int64_t num_rows_sparse, int dtype, int scores_dtype, int index_dtype, void *stream);

/* Score gradient of the combine: grad_scores[t, j] = <input[sparse_rows[t, j], :], grad_output[t, :]> in fp32,
 * stored as `out_dtype`.
 * Replaces `copy_sparse_to_dense_grad_score_kernel` (sparse_copy.py:111-148, launched at :156-164). */
int fm_copy_sparse_to_dense_grad_score(const void *input, const void *grad_output, const void *sparse_rows,
                                       void *grad_scores, int64_t num_rows_dense, int64_t num_columns,
                                       int64_t num_experts_per_token, int64_t num_rows_sparse, int dtype,
                                       int out_dtype, int index_dtype, void *stream);

/* Whole backward of the combine in one pass over `grad_output`:
 *   grad_input[sparse_rows[t, j], :] = grad_output[t, :] * scores[t, j]
 *   grad_scores[t, j]                = <input[sparse_rows[t, j], :], grad_output[t, :]>
 * Same results as the two calls above; replaces the pair launched by `copy_sparse_to_dense_backward`
 * (sparse_copy.py:190-194). `scores` must not be NULL. */
int fm_copy_sparse_to_dense_backward(const void *input, const void *grad_output, const void *scores,
                                     const void *sparse_rows, void *grad_input, void *grad_scores,
                                     int64_t num_rows_dense, int64_t num_columns, int64_t num_experts_per_token,
                                     int64_t num_rows_sparse, int dtype, int scores_dtype, int out_dtype,
                                     int index_dtype, void *stream);

/* ---------------------------------------------------------------------------------------------------------
 * Top-k routing (the step just before the sparse map). `logits` is [num_tokens, num_experts], contiguous, of
 * `dtype`; num_experts <= 1024, experts_per_token <= 64.
 * --------------------------------------------------------------------------------------------------------- */

/* top_experts[t, j] (int64) = expert of the j-th largest logit of token t (ties: lower expert first);
 * scores[t, :] (fp32) = softmax over those experts_per_token logits, computed in fp32.
 * Replaces the torch.topk + torch.softmax pair of `MixtureOfExpertMLP._topk_routing`
 * (fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244). */
int fm_topk_routing(const void *logits, void *top_experts, void *scores, int64_t num_tokens, int64_t num_experts,
                    int64_t experts_per_token, int dtype, void *stream);

/* grad_logits[t, top_experts[t, j]] = scores[t, j] * (grad_scores[t, j] - <scores[t, :], grad_scores[t, :]>), zero
 * elsewhere: what autograd derives for the pair above (same lines of the reference). grad_scores/scores are fp32,
 * grad_logits has `dtype`. */
int fm_topk_routing_backward(const void *grad_scores, const void *scores, const void *top_experts, void *grad_logits,
                             int64_t num_tokens, int64_t num_experts, int64_t experts_per_token, int dtype,
                             void *stream);

/* The whole router front end of `MixtureOfExpertMLP._forward` between the logits and the sparse map, from one read
 * of the logits [num_tokens, num_experts] (`dtype`), where num_experts counts the routed (unshared) experts:
 *   - z-loss = mean_t logsumexp(logits[t, :])^2 on the logits as given
 *     (fast_llm/layers/decoder/mlp/mixture_of_experts.py:147-154, layers/language_model/loss/z_loss.py:88-92);
 *   - jitter: if `noise` (same shape and dtype, drawn by the caller) is not null, routing uses logits * noise rounded
 *     to `dtype` (:157-159, 234-235);
 *   - top-k and fp32 softmax over the selected logits (:243-244), as fm_topk_routing;
 *   - load-balancing loss = sum_e mean_t softmax(routed logits)[t, e] * mean_t selected[t, e] (:245-254);
 *   - shared experts (:264-278): top_experts/scores are [num_tokens, shared_experts + experts_per_token]; the first
 *     shared_experts slots of every token hold experts num_experts, num_experts + 1, ... with score 1.
 * Outputs: top_experts (int64), scores (fp32), lse [num_tokens, 2] fp32 (logsumexp of the routed and of the given
 * logits; kept for the backward), statistics [2 * num_experts + 1] fp32 (per expert: sum_t softmax, number of tokens
 * that selected it; then sum_t logsumexp^2), losses [2] fp32 (load balancing, z). Sums over tokens are added in a
 * fixed order. `workspace`: fm_router_workspace_size(num_tokens, num_experts) bytes of device memory. */
size_t fm_router_workspace_size(int64_t num_tokens, int64_t num_experts);
int fm_router_forward(const void *logits, const void *noise, void *top_experts, void *scores, void *lse,
                      void *statistics, void *losses, void *workspace, size_t workspace_size, int64_t num_tokens,
                      int64_t num_experts, int64_t experts_per_token, int64_t shared_experts, int dtype, void *stream);

/* Gradient of the logits given grad_scores [num_tokens, shared_experts + experts_per_token] (fp32; the shared slots
 * are ignored) and the constant gradients the reference attaches to the two losses through `AuxiliaryLoss`
 * (fast_llm/functional/utils.py:63-71; mixture_of_experts.py:154, 257-261): auxiliary_loss_grad for the load-balancing
 * loss and z_loss_grad for the z-loss, 0 for a loss that is not trained on. logits, noise, scores, top_experts, lse
 * and statistics are the forward's. grad_logits has `dtype`. */
int fm_router_backward(const void *grad_scores, const void *scores, const void *top_experts, const void *logits,
                       const void *noise, const void *lse, const void *statistics, void *grad_logits,
                       double auxiliary_loss_grad, double z_loss_grad, int64_t num_tokens, int64_t num_experts,
                       int64_t experts_per_token, int64_t shared_experts, int dtype, void *stream);

/* The sparse map from the router's own counts: `fm_router_forward` has already counted, per workgroup of its kernel,
 * how many tokens selected each routed expert, and left the counts in its workspace. Given that workspace unmodified
 * (same num_tokens; num_experts here counts routed + shared experts), this builds the map of `top_experts`
 * [num_tokens, shared_experts + experts_per_token] without the counting pass over `top_experts`. Same results as
 * `fm_sparse_map(top_experts, num_tokens, shared_experts + experts_per_token, num_experts, ...)`, bit for bit.
 * Precondition (not checked, the counts are trusted): `top_experts` is exactly what that `fm_router_forward` call
 * wrote. Selections edited since (masking, capacity or dropping) or counts of another call give expert ranges that
 * overlap or run past `expert_ends`; rebuild the map with `fm_sparse_map` then.
 * Replaces the same reference lines as `fm_sparse_map`, for the caller
 * fast_llm/layers/decoder/mlp/mixture_of_experts.py:163-171, 193-196 (routing followed by `get_sparse_map`).
 * `workspace`: fm_sparse_map_from_router_workspace_size(num_tokens, num_experts) bytes, 16-byte aligned. */
size_t fm_sparse_map_from_router_workspace_size(int64_t num_tokens, int64_t num_experts);
int fm_sparse_map_from_router(const int64_t *top_experts, const void *router_workspace, size_t router_workspace_size,
                              int64_t num_tokens, int64_t num_experts, int64_t experts_per_token,
                              int64_t shared_experts, int64_t pad_to_multiple, int index_dtype, void *sparse_rows,
                              void *expert_ends, void *expert_pad_begins, void *workspace, size_t workspace_size,
                              void *stream);

/* ---------------------------------------------------------------------------------------------------------
 * MLP activation. `input` is [num_rows, num_columns * (gated ? 2 : 1)], `output`/`grad_output` are
 * [num_rows, num_columns]; all contiguous. Gated: out = act(in[:, :n]) * in[:, n:]. Math in fp32.
 * `row_limit` (may be NULL) points to one device integer of `index_dtype`, the number of rows in use: rows at and
 * past it are neither read nor written. Passing the address of the last entry of a sparse map's `expert_ends`
 * keeps the kernels off the rows of the static worst-case layout that no expert owns (the reference's kernels
 * stream through them; nothing ever reads what they produce there).
 * --------------------------------------------------------------------------------------------------------- */

/* Replaces `triton_mlp_activation_forward_kernel` (fast_llm/functional/triton/mlp.py:29-71, launched :153-162). */
int fm_mlp_activation_forward(const void *input, void *output, int64_t num_rows, int64_t num_columns, int gated,
                              int activation, int dtype, const void *row_limit, int index_dtype, void *stream);

/* grad_input has the shape of input. `output` (may be NULL) receives the recomputed forward output.
 * Replaces `triton_mlp_activation_backward_kernel` (mlp.py:74-139, launched :177-189). */
int fm_mlp_activation_backward(const void *grad_output, void *grad_input, const void *input, void *output,
                               int64_t num_rows, int64_t num_columns, int gated, int activation, int dtype,
                               const void *row_limit, int index_dtype, void *stream);

/* ---------------------------------------------------------------------------------------------------------
 * Grouped ("sparse") matrix products. Strides are in elements. `lhs`/`rhs` share `dtype`; `out` has
 * `out_dtype`; accumulation is fp32 with a single rounding at the store. With `accumulate` != 0 the previous
 * content of `out` is added (in fp32) before the store. `expert_ends` (and `expert_pad_begins`) have
 * `index_dtype`; the expert of a 128-row block is `#{e : expert_ends[e] <= first row of the block}`, so every
 * expert boundary must be a multiple of 128 rows (the reference's MAX_DROPLESS_BLOCK_SIZE_ROW contract,
 * fast_llm/functional/config.py:106, sparse_linear.py:274; the kernels here take any boundary: a multiple of 128 is
 * only what keeps the matrix-core tiles full). If `expert_ends` is NULL the product is an
 * ordinary dense one (a single expert owning all rows), which is what the reference does for
 * `sparse_map=None` (sparse_linear.py:276-277, 404-405, 537-538).
 * Results are deterministic (no floating-point atomics; every sum has a fixed order that depends only on the
 * arguments and the expert map).
 *
 * `workspace`: device scratch (64-byte aligned, content irrelevant) of `fm_grouped_gemm_workspace_size(...)` bytes
 * (`fm_input_row_sparse_matmul_workspace_size(...)` for the row-sparse product). With it, a small kernel first writes
 * where every tile of the launch lies, so that the workgroups of the product look their tiles up instead of each
 * scanning the expert map (same tiles, same results); and a launch of few, long tiles (at most 16 rounds of 256
 * tiles of 256 x 256, reduction of 2048 or more) of the output-sparse and input-inner-sparse products, which would
 * leave most CUs idle in its last round, cuts the reductions of that round's tiles into 2, 4 or 8 pieces that fill
 * the CUs and adds the pieces in piece order. Whether that split happens depends on the dimensions and on whether a
 * workspace is passed, on nothing else (not on the stream, the device's free memory or earlier calls): NULL with
 * size 0 selects the unsplit sums, which differ from the split ones in the last bits; a non-null workspace smaller
 * than required or misaligned is FM_ERR_INVALID_ARGUMENT. Calls that may overlap (different streams) need different
 * workspaces. Products that do not run on the matrix cores (fp32 operands, odd strides) ignore the pair.
 * --------------------------------------------------------------------------------------------------------- */

/* Bytes of workspace for a product `out [row_dim, col_dim] = lhs [row_dim, inner_dim] x rhs` of `dtype` operands over
 * `num_experts` experts (1 for a dense product): the tile table and, where the last round is split, its pieces.
 * 0 for fp32 operands or an empty product. Depends on these five numbers only. */
size_t fm_grouped_gemm_workspace_size(int64_t row_dim, int64_t col_dim, int64_t inner_dim, int64_t num_experts,
                                      int dtype);

/* The same for the row-sparse product `out [row_sparse_dim * num_experts, col_dim]` (its reductions are never split:
 * the tile table only). */
size_t fm_input_row_sparse_matmul_workspace_size(int64_t row_sparse_dim, int64_t col_dim, int64_t inner_dim,
                                                 int64_t num_experts, int dtype);

/* out[i, j] = sum_k lhs[i, k] * rhs[k, j + col_sparse_dim * e(i)]   for i < expert_ends[-1]; rows past the last
 * expert ("phantom" rows) are neither read nor written. Padding rows inside an expert are computed like
 * real rows. lhs [row_dim, inner_dim], rhs [inner_dim, col_sparse_dim * num_experts], out [row_dim, col_sparse_dim].
 * Replaces `output_sparse_matmul_kernel` (sparse_linear.py:185-258, launched :288-306). */
int fm_output_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                            int64_t row_dim, int64_t col_sparse_dim, int64_t inner_dim, int64_t num_experts,
                            int64_t lhs_stride_row, int64_t lhs_stride_inner, int64_t rhs_stride_inner,
                            int64_t rhs_stride_col, int64_t out_stride_row, int64_t out_stride_col,
                            int accumulate, int dtype, int out_dtype, int index_dtype, void *workspace,
                            size_t workspace_size, void *stream);

/* out[i, j] = sum_k lhs[i, k] * rhs[k + inner_sparse_dim * e(i), j]; same row rules as above.
 * lhs [row_dim, inner_sparse_dim], rhs [inner_sparse_dim * num_experts, col_dim], out [row_dim, col_dim].
 * Replaces `input_inner_sparse_matmul_kernel` (sparse_linear.py:310-385, launched :415-433). */
int fm_input_inner_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                                 int64_t row_dim, int64_t col_dim, int64_t inner_sparse_dim, int64_t num_experts,
                                 int64_t lhs_stride_row, int64_t lhs_stride_inner, int64_t rhs_stride_inner,
                                 int64_t rhs_stride_col, int64_t out_stride_row, int64_t out_stride_col,
                                 int accumulate, int dtype, int out_dtype, int index_dtype, void *workspace,
                                 size_t workspace_size, void *stream);

/* out[i + row_sparse_dim * e, j] = sum_{k in [begin_e, expert_pad_begins[e])} lhs[i, k] * rhs[k, j],
 * begin_e = expert_ends[e - 1] (0 for e = 0). Rows of the inner dimension outside that range (padding and
 * phantom rows) are replaced by zero before the multiply, so NaN/Inf stored there cannot leak. An expert
 * without rows gives zeros (or leaves `out` unchanged when accumulating).
 * lhs [row_sparse_dim, inner_dim], rhs [inner_dim, col_dim], out [row_sparse_dim * num_experts, col_dim].
 * Replaces `input_row_sparse_matmul_kernel` (sparse_linear.py:437-517, launched :551-569). */
int fm_input_row_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                               const void *expert_pad_begins, int64_t row_sparse_dim, int64_t col_dim,
                               int64_t inner_dim, int64_t num_experts, int64_t lhs_stride_row,
                               int64_t lhs_stride_inner, int64_t rhs_stride_inner, int64_t rhs_stride_col,
                               int64_t out_stride_row, int64_t out_stride_col, int accumulate, int dtype,
                               int out_dtype, int index_dtype, void *workspace, size_t workspace_size, void *stream);

/* Layer 1 of a gated MLP with the activation fused into the product's epilogue: what the reference does with
 * `output_sparse_matmul` (fast_llm/functional/triton/sparse_linear.py:261-306) followed by
 * `triton_mlp_activation_forward` (fast_llm/functional/triton/mlp.py:29-67, 131-154), as called from `mlp_forward`
 * (:246-258). lhs [row_dim, inner_dim]; rhs [inner_dim, num_experts * 2 * activation_dim] (per expert the gate
 * columns, then the up columns); layer_1_out [row_dim, 2 * activation_dim] contiguous, or null when it is not kept;
 * activation_out [row_dim, activation_dim] contiguous = act(gate) * up, computed from the rounded product, so both
 * outputs are bit-identical to the two separate calls. Returns FM_ERR_UNSUPPORTED when the shape does not fit the
 * matrix-core kernel (fp32; operands not contiguous along inner_dim; inner_dim not a multiple of 64; activation_dim
 * not a multiple of 128): call the product and the activation separately then. */
int fm_output_sparse_matmul_gated_activation(const void *lhs, const void *rhs, void *layer_1_out, void *activation_out,
                                             const void *expert_ends, int64_t row_dim, int64_t activation_dim,
                                             int64_t inner_dim, int64_t num_experts, int64_t lhs_stride_row,
                                             int64_t lhs_stride_inner, int64_t rhs_stride_inner, int64_t rhs_stride_col,
                                             int activation, int dtype, int index_dtype, void *stream);

/* The gradient of layer 1's output in the backward of a gated MLP: the product of the reference's layer-2 input
 * gradient `output_sparse_matmul(grad_output, weight_2_t, sparse_map)` (fast_llm/functional/triton/mlp.py:352-359)
 * is not stored but handed, tile by tile, to the activation backward `triton_mlp_activation_backward` (:70-128,
 * 157-185, called at :373-375). lhs [row_dim, inner_dim]; rhs [inner_dim, num_experts * activation_dim];
 * layer_1_out and grad_layer_1_out [row_dim, 2 * activation_dim] contiguous; activation_out
 * [row_dim, activation_dim] or null: the recomputed activation output. Bit-identical to the two separate calls.
 * FM_ERR_UNSUPPORTED as above (activation_dim a multiple of 8 is enough here). */
int fm_output_sparse_matmul_gated_activation_backward(const void *lhs, const void *rhs, const void *layer_1_out,
                                                      void *grad_layer_1_out, void *activation_out,
                                                      const void *expert_ends, int64_t row_dim, int64_t activation_dim,
                                                      int64_t inner_dim, int64_t num_experts, int64_t lhs_stride_row,
                                                      int64_t lhs_stride_inner, int64_t rhs_stride_inner,
                                                      int64_t rhs_stride_col, int activation, int dtype,
                                                      int index_dtype, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* FASTMOE_HIP_H */
