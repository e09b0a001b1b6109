/*
 * cute_hip.h — C ABI of the gfx950 (MI355X) kernel library behind the `cute_kernels` Python API.
 *
 * Conventions shared by every entry point
 *   - every pointer is a DEVICE pointer unless the comment says otherwise;
 *   - the caller owns every buffer (inputs, outputs and workspaces); the library never allocates,
 *     frees or keeps a reference after the call returns;
 *   - `stream` is a hipStream_t passed as void*; the work is enqueued there and the call returns
 *     without synchronising;
 *   - the return value is a ck_status (0 = CK_OK).  Nothing is launched when it is non-zero;
 *   - `dtype` is a ck_dtype; fp32 accumulation is used for every floating-point type;
 *   - index tensors are int64 unless an `ids_are_i32`-style flag says otherwise.
 *
 * Each declaration cites the reference interface it replaces (paths under the reference repo).
 */
#ifndef CUTE_HIP_H
#define CUTE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { CK_F32 = 0, CK_F16 = 1, CK_BF16 = 2 } ck_dtype;

typedef enum {
    CK_OK = 0,
    CK_ERR_DTYPE = 1,     /* unsupported ck_dtype */
    CK_ERR_SHAPE = 2,     /* a size / stride the kernels cannot handle */
    CK_ERR_NULL = 3,      /* required pointer is NULL */
    CK_ERR_WORKSPACE = 4, /* workspace smaller than the *_workspace_size query */
    CK_ERR_LAUNCH = 5,    /* hipGetLastError() reported a launch failure */
    CK_ERR_ALIGN = 6,     /* pointer not aligned to the element size */
    CK_ERR_SCRATCH = 7,   /* problem too large for the library's built-in scratch buffer (ck_moe_sort_noalloc) */
    CK_ERR_RUNTIME = 8    /* a HIP runtime query (current device, symbol address) failed */
} ck_status;

/* Human-readable text for a ck_status (host pointer to a static string). */
const char* ck_status_string(int status);
/* Library version, bumped when a signature changes. */
int ck_abi_version(void);

/* ---------------------------------------------------------------------------------------------
 * SwiGLU on two tensors: y = up * gate * sigmoid(gate)
 * replaces cute_kernels/kernels/swiglu/cuda_implementation/ops.cpp:3-18
 *   (swiglu_forward_cuda(gate, up, output, BLOCK_SIZE), swiglu_backward_cuda(...))
 * and the Triton launchers swiglu/triton_implementation/kernels_forward.py:28-39,
 * kernels_backward.py:36-56.  `block_size` is the threads per workgroup (64..1024, multiple of 64).
 * ------------------------------------------------------------------------------------------- */
int ck_swiglu_forward(const void* gate, const void* up, void* output, int64_t num_elements, int dtype,
                      int block_size, void* stream);
int ck_swiglu_backward(const void* gate, const void* up, const void* output_grad, void* gate_grad,
                       void* up_grad, int64_t num_elements, int dtype, int block_size, void* stream);

/* ---------------------------------------------------------------------------------------------
 * SwiGLU on one tensor x[B, 2h]: up = x[:, :h], gate = x[:, h:], y[B, h]
 * replaces swiglu_unchunked/triton_implementation/kernels_forward.py:41-56 and
 * kernels_backward.py:51-71.  x_grad has x's layout (d_up in the first half, d_gate in the second).
 * ------------------------------------------------------------------------------------------- */
int ck_swiglu_unchunked_forward(const void* x, void* output, int64_t B, int64_t H_full, int dtype,
                                int block_size, void* stream);
int ck_swiglu_unchunked_backward(const void* x, const void* output_grad, void* x_grad, int64_t B,
                                 int64_t H_full, int dtype, int block_size, void* stream);

/* ---------------------------------------------------------------------------------------------
 * RMSNorm over the last dimension of x[B, H]
 * replaces rmsnorm/triton_implementation/kernels_forward.py:77-107 (rmsnorm_forward_triton) and
 * kernels_backward.py:99-228 (rmsnorm_backward_triton, weighted and unweighted).
 *   weight   : [H] or NULL
 *   rstd     : fp32 [B] or NULL.  forward: written when non-NULL.  backward: read when non-NULL,
 *              recomputed from x when NULL (the reference's `memory_efficient` mode)
 *   backward : weight_grad ([H], dtype of x) is written when weight != NULL; it is reduced without
 *              atomics through `workspace` (ck_rmsnorm_backward_workspace_size bytes).
 * H must be <= 65536 (the reference's MAX_TRITON_BLOCK_SIZE limit, rmsnorm/forward.py:31-32).
 * block_size_b is the reference's tunable BLOCK_SIZE_B (rows per program, kernels_forward.py:63-107,
 * kernels_backward.py:177-228), here the launch variant for rows that one wavefront holds (up to 512 packets of 16
 * bytes: 4096 16-bit elements): forward 1, 2 = rows a wave requests at once before it ends (3 .. 7 are the launch of
 * 2), 8 or more = waves that walk rows with the next row in flight; backward 1 = two workgroups per compute unit without a row in flight,
 * 2 or more = one workgroup per compute unit with.  0 = the library's default.  Every variant gives the same values.
 * ------------------------------------------------------------------------------------------- */
int ck_rmsnorm_forward(const void* x, const void* weight, void* output, float* rstd, int64_t B, int64_t H,
                       float eps, int dtype, int block_size_b, void* stream);

/* Residual addition and RMSNorm in one pass (no counterpart in the reference, whose transformer blocks would run
 * x + residual through add_tensor (kernels/add/add_tensor/__init__.py) and then rmsnorm (kernels/rmsnorm/__init__.py)):
 *   residual_out = x + residual  (fp32 sum, rounded to the storage type),  output = rmsnorm(residual_out) as above.
 * Same values as ck_add_tensor_forward followed by ck_rmsnorm_forward, with one read of the sum less.  All tensors
 * are dense [B, H]; rstd and block_size_b as in ck_rmsnorm_forward.  The gradient of the pair is ck_rmsnorm_backward on
 * residual_out plus whatever gradient reaches residual_out (ck_add_tensor_forward). */
int ck_residual_rmsnorm_forward(const void* x, const void* residual, const void* weight, void* output,
                                void* residual_out, float* rstd, int64_t B, int64_t H, float eps, int dtype,
                                int block_size_b, void* stream);
int64_t ck_rmsnorm_backward_workspace_size(int64_t B, int64_t H);
int ck_rmsnorm_backward(const void* x, const void* weight, const void* output_grad, const float* rstd,
                        void* x_grad, void* weight_grad, void* workspace, int64_t workspace_bytes,
                        int64_t B, int64_t H, float eps, int dtype, int block_size_b, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Embedding gather / scatter-add
 * replaces embedding/triton_implementation/kernels_forward.py:42-64 (embedding_forward_triton) and
 * kernels_backward.py:48-75 (embedding_backward_triton).
 *   forward : output[i, :] = weight[ids[i], :]  (bit-exact copy; an id outside [0, V) yields a zero row)
 *   backward: weight_grad[V, H] is written completely (rows no id selects become zero); duplicates are
 *             accumulated in fp32 in ascending token position and rounded once.
 *             (CK_EMBEDDING_BWD_PRELUDE=short in the environment, read at every call, sorts the ids in one
 *             workgroup behind two small launches instead of seven grid-wide ones, for up to 131072 ids; the
 *             results are the same bits.)
 * ------------------------------------------------------------------------------------------- */
int ck_embedding_forward(const void* ids, int ids_are_i32, const void* weight, void* output,
                         int64_t num_ids, int64_t V, int64_t H, int dtype, void* stream);
int64_t ck_embedding_backward_workspace_size(int64_t num_ids, int64_t V, int64_t H);
int ck_embedding_backward(const void* ids, int ids_are_i32, const void* output_grad, void* weight_grad,
                          void* workspace, int64_t workspace_bytes, int64_t num_ids, int64_t V, int64_t H,
                          int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Histogram of small non-negative integers: out[c] = #{i : x[i] == c}, c < size, int32
 * replaces contiguous_count/triton_implementation/kernels_forward.py:46-66 (contiguous_count_triton).
 * Values outside [0, size) are ignored.
 * ------------------------------------------------------------------------------------------- */
int ck_contiguous_count(const void* x, int x_is_i32, int32_t* output, int64_t n, int64_t size, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Element-wise additions: output = x + y and output = x + scalar (sum formed in fp32, one rounding)
 * replace add_tensor_forward_cuda (kernels/add/add_tensor/cuda_implementation/ops.cpp:3-7) and
 *         add_scalar_forward_cuda (kernels/add/add_scalar/cuda_implementation/ops.cpp:3-7);
 * the reference's vector_instruction_width has no counterpart: packets are 16 bytes whenever the
 * pointers allow it.  Tensors are dense with identical layout; block_size as for the SwiGLU kernels.
 * ------------------------------------------------------------------------------------------- */
int ck_add_tensor_forward(const void* x, const void* y, void* output, int64_t num_elements, int dtype,
                          int block_size, void* stream);
int ck_add_scalar_forward(const void* x, double y, void* output, int64_t num_elements, int dtype, int block_size,
                          void* stream);

/* ---------------------------------------------------------------------------------------------
 * Expert sort for the MoE layer: STABLE ascending sort of expert ids with their positions, plus the
 * inclusive prefix sum of the per-expert counts.
 * replaces scattermoe/triton_implementation/__init__.py:80-81
 *   (selected_experts.flatten().sort(); contiguous_count_cute(...).cumsum(-1)).
 *   expert_ids            : int64 (or int32) [M], values in [0, E)
 *   sorted_expert_idxs    : int64 [M]
 *   sorted_scattered_idxs : int64 [M]  (position in expert_ids of each sorted element)
 *   expert_offsets        : int64 [E]  (expert_offsets[e] = number of ids <= e)
 * ------------------------------------------------------------------------------------------- */
int64_t ck_moe_sort_workspace_size(int64_t M, int64_t E);
int ck_moe_sort(const void* expert_ids, int ids_are_i32, int64_t* sorted_expert_idxs,
                int64_t* sorted_scattered_idxs, int64_t* expert_offsets, void* workspace,
                int64_t workspace_bytes, int64_t M, int64_t E, void* stream);

/* ck_moe_sort for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference, which takes every buffer from torch's
 * allocator.  Same arguments and results as ck_moe_sort, minus the workspace: that lives in a device array of
 * CK_MOE_SORT_NOALLOC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process ends.  The call
 * makes no hipMalloc / hipFree and no allocating library call; the first call on a device looks the array's
 * address up once (hipGetSymbolAddress, which may load the code object and the 4 MiB array): make that first call
 * per device outside any stream capture, every later one may be captured.  (M, E) whose ck_moe_sort_workspace_size exceeds the array gives CK_ERR_SCRATCH and launches
 * nothing (the limit is far away: 98304 ids of 64 experts need 48 KiB, a million ids of 512 experts 4 MiB).
 * All calls on one GPU share the array: calls that overlap there (different streams or threads) race; calls
 * ordered on one stream do not.  Nothing in the array has to be cleared between calls. */
#define CK_MOE_SORT_NOALLOC_SCRATCH_BYTES (4 * 1024 * 1024)
int ck_moe_sort_noalloc(const void* expert_ids, int ids_are_i32, int64_t* sorted_expert_idxs,
                        int64_t* sorted_scattered_idxs, int64_t* expert_offsets, int64_t M, int64_t E, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Grouped GEMM with row gather / scatter ("scatter2scatter")
 * replaces scattermoe/triton_implementation/ops.py:16-63 (cute::scatter2scatter).
 * For every sorted slot i in [0, num_slots):
 *   out[out_row(i), :] = X[in_row(i), :] @ W[e(i)]         (fp32 accumulation)
 *   e(i)       = expert owning slot i according to expert_offsets
 *   in_row(i)  = i if x_grouped else sorted_scattered_idxs[i] / fan_out
 *   out_row(i) = i if y_grouped else sorted_scattered_idxs[i]
 * X is [*, K] with row stride x_stride (elements, K contiguous); W is a strided view [E, K, N] with
 * element strides (w_stride_e, w_stride_k, w_stride_n), one of w_stride_k / w_stride_n being 1;
 * out is [num_slots, N] with row stride out_stride.  expert_offsets is int64 [E] (inclusive ends).
 * bias is NULL or [E, N] contiguous, of the operands' type: out[out_row(i), :] then also gets bias[e(i), :], added
 * to the fp32 sums before they are rounded - the bias of the reference's per-expert F.linear
 * (scattermoe/torch_implementation.py:35-43; its Triton experts carry none).
 * ------------------------------------------------------------------------------------------- */
int ck_scatter2scatter(const void* X, int64_t x_stride, const void* W, int64_t w_stride_e,
                       int64_t w_stride_k, int64_t w_stride_n, const int64_t* sorted_scattered_idxs,
                       const int64_t* expert_offsets, void* out, int64_t out_stride, int64_t num_slots,
                       int64_t K, int64_t N, int64_t E, int64_t fan_out, int x_grouped, int y_grouped,
                       const void* bias, int dtype, void* stream);

/* The same product with the tail of the tile grid split along the contraction (no counterpart in the reference).
 * A product with few column tiles leaves most CUs idle during its last round of tiles; given a workspace of
 * ck_scatter2scatter_workspace_size() bytes (16-byte aligned; 0: the shape is not eligible - fp32, or K below 4096),
 * the tiles of every XCD's last round are cut into pieces of the contraction range, summed by a second launch on the
 * same stream.  Results differ from ck_scatter2scatter in the order of the fp32 additions only.  workspace == NULL
 * is ck_scatter2scatter.
 * `waves` (here and in the three entry points below) names the loop of the matrix-core kernel, the counterpart of the
 * num_warps / num_stages of the reference's tuned Triton configurations (scattermoe/triton_implementation/
 * kernels.py:152-159): 8 = eight wavefronts per 256 x 256 tile, two per SIMD working in antiphase; 4 = four
 * wavefronts, one per SIMD, each a software pipeline over a 128 x 128 block with its accumulators in the
 * accumulation registers; 0 = the library's choice.  Same tile grid, same results up to the order of the fp32
 * additions inside a matrix instruction's block; anything else is CK_ERR_SHAPE.  A product with a bias takes 8. */
int64_t ck_scatter2scatter_workspace_size(int64_t num_slots, int64_t K, int64_t N, int64_t E, int dtype);
int ck_scatter2scatter_ws(const void* X, int64_t x_stride, const void* W, int64_t w_stride_e, int64_t w_stride_k,
                          int64_t w_stride_n, const int64_t* sorted_scattered_idxs, const int64_t* expert_offsets,
                          void* out, int64_t out_stride, int64_t num_slots, int64_t K, int64_t N, int64_t E,
                          int64_t fan_out, int x_grouped, int y_grouped, const void* bias, int dtype, int waves,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * scatter2scatter with the SwiGLU of the MoE layer in its epilogue.
 * replaces, in one launch each, the pairs of calls the reference layer makes around its activation
 * (scattermoe/triton_implementation/__init__.py:83-87: c_fc then self.act; and, in the backward,
 * ops.py:240-250 of c_proj followed by swiglu_unchunked's backward,
 * swiglu_unchunked/torch_implementation.py:5-7 being the activation):
 *
 *   ck_scatter2scatter_glu:      h[i, :]   = X[in_row(i), :] @ W[e(i)]          W view [E, K, 2I]
 *                                act[i, c] = h[i, c] * silu(h[i, I + c])        c in [0, I)
 *   ck_scatter2scatter_glu_bwd:  d_act[i, :] = DY[i, :] @ W[e(i)]               W view [E, K, I]
 *                                d_h[i, c]     = d_act[i, c] * silu(h[i, I + c])
 *                                d_h[i, I + c] = d_act[i, c] * h[i, c] * silu'(h[i, I + c])
 *
 * Output rows are in sorted-slot order (y_grouped); in the backward so are the rows of DY.  h and d_act are
 * rounded to the storage type before the activation sees them, so the results equal those of the separate
 * calls bit for bit.  Shapes the fused kernels do not take (fp32, I not a multiple of 128 / of 8, odd
 * strides) run as ck_scatter2scatter followed by an element-wise pass, with the same results; d_act then
 * passes through the first half of each d_h row, so d_h must not alias h.
 * Strides are in elements; in_row(i), e(i), expert_offsets as for ck_scatter2scatter.
 * ------------------------------------------------------------------------------------------- */
int ck_scatter2scatter_glu(const void* X, int64_t x_stride, const void* W, int64_t w_stride_e,
                           int64_t w_stride_k, int64_t w_stride_n, const int64_t* sorted_scattered_idxs,
                           const int64_t* expert_offsets, void* h, int64_t h_stride, void* act,
                           int64_t act_stride, int64_t num_slots, int64_t K, int64_t I, int64_t E,
                           int64_t fan_out, int x_grouped, int dtype, int waves, void* stream);
int ck_scatter2scatter_glu_bwd(const void* DY, int64_t dy_stride, const void* W, int64_t w_stride_e,
                               int64_t w_stride_k, int64_t w_stride_n, const int64_t* expert_offsets,
                               const void* h, int64_t h_stride, void* d_h, int64_t d_h_stride,
                               int64_t num_slots, int64_t K, int64_t I, int64_t E, int dtype, int waves,
                               void* stream);

/* Inclusive expert offsets from already-sorted expert ids (int64 [M] -> int64 [E]); used when a caller
 * of cute::scatter2scatter has the sorted ids but not the offsets (ops.py:16-24 takes only the ids). */
int ck_offsets_from_sorted(const int64_t* sorted_expert_idxs, int64_t* expert_offsets, int64_t M, int64_t E,
                           void* stream);

/* ---------------------------------------------------------------------------------------------
 * Per-expert weight gradient ("groupXtY"): DW[e] (K x N) = X_e^T (K x M_e) @ DY_e (M_e x N)
 * replaces scattermoe/triton_implementation/ops.py:67-94 (cute::group_bwd_W).
 * X [M, K] and DY [M, N] are expert-grouped rows (row strides x_stride / dy_stride, unit column stride);
 * DW is a strided view [E, K, N] (element strides dw_stride_e/k/n, one of k/n being 1).  Every element
 * of DW is written: experts with no rows receive zeros, so the caller need not clear DW first.
 * ------------------------------------------------------------------------------------------- */
int ck_group_bwd_W(const void* DY, int64_t dy_stride, const void* X, int64_t x_stride,
                   const int64_t* expert_offsets, void* DW, int64_t dw_stride_e, int64_t dw_stride_k,
                   int64_t dw_stride_n, int64_t M, int64_t K, int64_t N, int64_t E, int dtype, int waves,
                   void* stream);

/* ---------------------------------------------------------------------------------------------
 * Row gather with optional per-row coefficient ("group")
 * replaces scattermoe/triton_implementation/ops.py:98-130 (cute::group).
 *   out[i, :] = A[idx[i] / fan_out, :] * (coeff ? coeff[idx[i]] : 1)     i in [0, num_rows)
 * ------------------------------------------------------------------------------------------- */
int ck_group(const void* A, int64_t a_stride, const int64_t* idx, const void* coeff, void* out,
             int64_t out_stride, int64_t num_rows, int64_t K, int64_t fan_out, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Mixing of each token's k expert outputs with its routing weights, and the routing weights' gradient
 * replaces the two torch.bmm calls of scattermoe/triton_implementation/ops.py:160-164 and :204.
 *   forward : out[t, :]     = sum_j gates[t, j] * expanded[t, j, :]      expanded [T, k, H], gates [T, k]
 *   backward: d_gates[t, j] = sum_h expanded[t, j, h] * grad_out[t, h]
 * gates == NULL in the forward call gives the plain sum over j: the input gradient's
 * `.view(T, k, H).sum(-2)` of ops.py:261.  All tensors dense.
 * ------------------------------------------------------------------------------------------- */
int ck_moe_combine_forward(const void* expanded, const void* gates, void* out, int64_t tokens, int64_t k,
                           int64_t H, int dtype, void* stream);
int ck_moe_combine_backward_gates(const void* expanded, const void* grad_out, void* d_gates, int64_t tokens,
                                  int64_t k, int64_t H, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Routing weights: top-k of the router logits and the softmax over the k selected values
 * replaces the stock torch ops of MoE_Torch._compute_routing_weights / _get_topk
 * (scattermoe/torch_implementation.py:121-132, 193-199: topk or max, .float(), softmax, type_as) and the
 * backward ops autograd derives from them.
 *   forward : logits [tokens, E] (row stride logits_stride, unit column stride) ->
 *             selected [tokens, k] int64: positions of the k largest logits, largest first (ties: the lower
 *             position first; NaN counts as the largest value, as in torch.topk),
 *             weights [tokens, k] (storage type) and weights_f32 [tokens, k]: softmax over the k values in fp32.
 *   backward: d_logits [tokens, E] = softmax backward of d_weights on weights_f32, placed at the selected
 *             positions, zero elsewhere; every element is written.
 * E <= 1024, k <= min(E, 64); weights, weights_f32, selected and d_weights are dense.
 * ------------------------------------------------------------------------------------------- */
int ck_router_topk_softmax_forward(const void* logits, int64_t logits_stride, void* weights, float* weights_f32,
                                   int64_t* selected, int64_t tokens, int64_t E, int64_t k, int dtype, void* stream);
int ck_router_topk_softmax_backward(const void* d_weights, const float* weights_f32, const int64_t* selected,
                                    void* d_logits, int64_t d_logits_stride, int64_t tokens, int64_t E, int64_t k,
                                    int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Router forward in one launch: the router's linear followed by the selection above
 * replaces `self.gate(hidden_states)` (a bias-free linear, scattermoe/torch_implementation.py:122) together
 * with the topk / softmax sequence of :123-132.
 *   logits [tokens, E] = x [tokens, H] * gate_weight [E, H]^T, fp32 accumulation, rounded once to the storage
 *   type and written (row stride logits_stride); selected / weights / weights_f32 as
 *   ck_router_topk_softmax_forward gives them for these stored logits.
 * bf16 and fp16 only (CK_ERR_DTYPE otherwise: the caller uses its linear and ck_router_topk_softmax_forward);
 * H a multiple of 8, x and gate_weight 16-byte aligned with row strides that are multiples of 8 elements and
 * unit column stride; E <= 128, k <= min(E, 64).  The backward is ck_router_topk_softmax_backward followed by the
 * caller's two products with d_logits.
 * ------------------------------------------------------------------------------------------- */
int ck_router_forward(const void* x, int64_t x_stride, const void* gate_weight, int64_t gate_weight_stride,
                      void* logits, int64_t logits_stride, void* weights, float* weights_f32, int64_t* selected,
                      int64_t tokens, int64_t H, int64_t E, int64_t k, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Gradient of the router's weight: d_weight [E, H] = d_logits^T x
 * replaces the weight gradient autograd derives for `self.gate(hidden_states)`
 * (scattermoe/torch_implementation.py:122; an [E, tokens] x [tokens, H] product with few outputs).
 *   d_logits_t [E, tokens]: d_logits transposed, dense; x [tokens, H] with row stride x_stride.
 *   The tokens are cut into pieces whose products are kept in fp32 in the workspace
 *   (ck_router_weight_grad_workspace_size bytes, 16-byte aligned) and added up in a fixed order: one rounding.
 * bf16 and fp16 only (CK_ERR_DTYPE otherwise); tokens and H multiples of 8, E <= 128, d_logits_t and x 16-byte
 * aligned, x_stride a multiple of 8.
 * ------------------------------------------------------------------------------------------- */
int64_t ck_router_weight_grad_workspace_size(int64_t tokens, int64_t H, int64_t E);
int ck_router_weight_grad(const void* d_logits_t, const void* x, int64_t x_stride, void* d_weight,
                          int64_t d_weight_stride, void* workspace, int64_t workspace_bytes, int64_t tokens, int64_t H,
                          int64_t E, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Per-expert bias of the grouped linears
 * replaces the bias term of F.linear(rows_e, W[e], bias[e]) in scattermoe/torch_implementation.py:35-43 (the
 * reference's Triton experts, triton_implementation/__init__.py:24-34, do not read their bias parameter).
 *   forward : y[r(i), :] += bias[e(i), :]   for every expert-sorted position i in [0, num_rows), where e(i) is the
 *             expert whose offset range holds i and r(i) = row_index ? row_index[i] : i (NULL: y is expert-grouped;
 *             sorted_scattered_idxs: y is in (token, slot) order).  In place, fp32 add, one rounding.
 *   backward: d_bias[e, :] = sum of the expert-grouped rows dy[offsets[e-1] .. offsets[e]) (fp32 sum in a fixed
 *             order, one rounding; zeros for an expert without rows).  Every element of d_bias is written.
 * y / dy / bias / d_bias have unit column stride and the given row strides (in elements); E <= 65535 backward.
 * ------------------------------------------------------------------------------------------- */
int ck_expert_bias_forward(void* y, int64_t y_stride, const void* bias, int64_t bias_stride,
                           const int64_t* row_index, const int64_t* expert_offsets, int64_t num_rows, int64_t N,
                           int64_t E, int dtype, void* stream);
int ck_expert_bias_backward(const void* dy, int64_t dy_stride, const int64_t* expert_offsets, void* d_bias,
                            int64_t d_bias_stride, int64_t num_rows, int64_t N, int64_t E, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CUTE_HIP_H */
