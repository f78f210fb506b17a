/*
 * ck_mi355.h -- C ABI of libck_mi355.so: the MoE hot path of cute-kernels on one MI355X (gfx950).
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes only; every pointer is DEVICE memory unless said otherwise;
 *   - the caller allocates every output and every workspace; the library never allocates device memory;
 *   - `stream` is a hipStream_t passed as void*; launches are asynchronous on it, nothing synchronises the host;
 *   - return value 0 = launched; non-zero = rejected (bad argument or launch failure), and
 *     ck_last_error_string() then holds a thread-local message;
 *   - `dtype` codes: CK_F32 = 0, CK_F16 = 1, CK_BF16 = 2;
 *   - activations are row-major and contiguous; expert weights are [E, out_features, in_features] with
 *     in_features contiguous, exactly as the reference stores them
 *     (cute_kernels/kernels/scattermoe/torch_implementation.py:18).
 *
 * Each declaration cites the reference interface it replaces (paths relative to the reference root).
 */
#ifndef CK_MI355_H
#define CK_MI355_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CK_F32 0
#define CK_F16 1
#define CK_BF16 2

#define CK_OK 0
#define CK_ERR_ARG 1
#define CK_ERR_LAUNCH 2

/* Message for the last non-zero return on this thread ("" if none). Host pointer, valid until the next failing call. */
const char* ck_last_error_string(void);
/* ABI revision of the library; bumps when a signature or a struct changes. */
int32_t ck_abi_version(void);
/* Test and measurement hook, no counterpart in the reference: chooses, process-wide, between kernels of this library that
 * compute the same result. The defaults are what the library runs in production; nothing here changes a result beyond
 * the tolerance of the kernels' own tests. Not meant to be changed while other threads issue launches.
 *   "gemm_line_kernel"       (default 1)  0: the 16-bit grouped GEMMs always run on the general kernel
 *   "gemm_register_pipeline" (default 0)  1: the general kernel stages its operands through registers
 *   "gemm_four_waves"        (default 0)  1: the general kernel's direct-to-LDS pipeline with 4 waves instead of 8
 *   "trace_buffer"           (default 0)  device address (as an integer) that builds compiled with -DCK_STAMP write
 *                                         per-wave cycle counts to; product builds never read it
 * Unknown names return CK_ERR_ARG. */
int ck_debug_set_option(const char* name, int64_t value);

/* ---------------------------------------------------------------------------------------------------------------
 * (a) expert histogram + offsets
 * Replaces: continuous_count_cuda(x, output, C, ...) -- cute_kernels/kernels/continuous_count/cuda_implementation/
 *           ops.cpp:7-15, forward.cu:72-178 -- and the bincount(...).cumsum(-1) of
 *           cute_kernels/kernels/scattermoe/triton_implementation/ops.py:19-28.
 * ids: n values, int32 (ids_are_i64 = 0) or int64 (1). Values outside [0, num_bins) are not counted.
 * counts[num_bins] (uint32) is required; ends (inclusive prefix sum) and starts (exclusive) may be NULL.
 * workspace: ck_count_workspace_words(num_bins) uint32 words that are ALL ZERO on entry; the kernel leaves them
 * all zero again on exit, so one zero-initialised buffer per stream can be reused forever.
 * num_bins <= 16384 (same cap as forward.cu:12).
 * ------------------------------------------------------------------------------------------------------------- */
int64_t ck_count_workspace_words(int32_t num_bins);
int ck_count_offsets(const void* ids, int32_t ids_are_i64, int64_t n, int32_t num_bins, uint32_t* counts,
                     uint32_t* ends, uint32_t* starts, uint32_t* workspace, void* stream);

/* ck_count_offsets for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): no counterpart in the reference. Same arguments and results as ck_count_offsets without the
 * workspace: the ticket and accumulators live in a 65,540-byte device array inside the library (one copy per GPU, held
 * until the process ends), looked up once per device. The call clears the words it uses with a small kernel and then
 * runs the same count kernel; it calls no hipMalloc / hipFree. num_bins above 16384 is rejected (CK_ERR_ARG).
 * All calls on one GPU share that array: calls that overlap on one GPU (two streams, two host threads) race. */
int ck_count_offsets_static(const void* ids, int32_t ids_are_i64, int64_t n, int32_t num_bins, uint32_t* counts,
                            uint32_t* ends, uint32_t* starts, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * (b1) router: top-k over logits, softmax over the k selected logits
 * Replaces: MoE_Torch._get_topk + F.softmax(values.float()) --
 *           cute_kernels/kernels/scattermoe/torch_implementation.py:122-135,195-201.
 * logits [T, E] of `dtype`. selected [T, k] int32 (descending by logit; equal logits: lowest expert index first).
 * gates [T, k] fp32 = softmax over the k selected logits. topk_values [T, k] of `dtype` may be NULL.
 * E <= 1024, 1 <= k <= min(E, 32).
 * ------------------------------------------------------------------------------------------------------------- */
int ck_route_topk_softmax(const void* logits, int32_t dtype, int64_t T, int32_t E, int32_t k, int32_t* selected,
                          float* gates, void* topk_values, void* stream);
/* Backward of the above with respect to the logits (autograd of topk + softmax at
 * torch_implementation.py:127-133): d_logits [T, E] of `dtype`, every element written (zeros off the selection).
 * d_gates [T, k] fp32. */
int ck_route_topk_softmax_bwd(const float* gates, const float* d_gates, const int32_t* selected, int64_t T,
                              int32_t E, int32_t k, void* d_logits, int32_t dtype, void* stream);
/* The same when the gates left the router in a 16-bit `dtype` and their gradient d_gates [T, k] came back in it, while
 * the caller also holds that gradient unrounded (d_gates_exact [T, k] fp32, from ck_gate_grad_f32): per element, where
 * d_gates equals d_gates_exact rounded to `dtype` the unrounded value is used, elsewhere (a hook scaled or replaced the
 * gradient) the value that arrived. One launch instead of a compare / reduce / select chain in front of the plain entry
 * point. Follows the same reference lines; the reference itself has only the rounded gradient (ops.py:214). */
int ck_route_topk_softmax_bwd_exact(const float* gates, const float* d_gates_exact, const void* d_gates,
                                    const int32_t* selected, int64_t T, int32_t E, int32_t k, void* d_logits,
                                    int32_t dtype, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * (b2) stable sort of (token, slot) pairs by expert + tile-aligned expert segments
 * Replaces: selected_experts.flatten().sort() and bincount(...).cumsum(-1) --
 *           cute_kernels/kernels/scattermoe/triton_implementation/__init__.py:82-83; the argsort / bincount of
 *           torch_implementation.py:171-193.
 * expert_ids: R = T*k flat ids (int32 or int64), all in [0, E). E <= 4096. An id outside [0, E) is dropped: counts
 *             exclude it, ends[E - 1] < R tells, and the tails of sorted_* stay unwritten (the caller's check).
 * Outputs (all int32 unless noted):
 *   sorted_expert_idxs[R], sorted_scattered_idxs[R]  -- the stable sort and its permutation
 *   counts[E], ends[E], starts[E] (uint32)            -- histogram, inclusive and exclusive prefix sums
 *   seg_starts[E + 1]  -- start row of each expert in the PADDED grouped layout: every expert's segment begins at
 *                         a multiple of `align` rows; seg_starts[E] = number of padded rows in use
 *   row_slot[max_rows] -- padded row p of expert e (seg_starts[e] <= p < seg_starts[e] + counts[e]) holds the flat
 *                         (token, slot) index sorted_scattered_idxs[starts[e] + p - seg_starts[e]]; other rows
 *                         are left unwritten
 *   tile_expert[max_tiles] -- expert that owns rows [t*align, (t+1)*align) of the padded layout, -1 past the end
 * max_rows = ck_sort_max_rows(R, E, align), max_tiles = max_rows / align.
 * workspace: ck_sort_workspace_words(R, E) uint32 words; word 0 must be zero on entry and is zero again on exit.
 * ------------------------------------------------------------------------------------------------------------- */
int64_t ck_sort_max_rows(int64_t R, int32_t E, int32_t align);
int64_t ck_sort_workspace_words(int64_t R, int32_t E);
int ck_sort_by_expert(const void* expert_ids, int32_t ids_are_i64, int64_t R, int32_t E, int32_t align,
                      int32_t* sorted_expert_idxs, int32_t* sorted_scattered_idxs, uint32_t* counts, uint32_t* ends,
                      uint32_t* starts, int32_t* seg_starts, int32_t* row_slot, int32_t* tile_expert,
                      uint32_t* workspace, void* stream);
/* The tile-aligned segment tables from a sort the caller already has -- the three index tensors the reference's expert
 * linears take: sorted_expert_idxs, sorted_scattered_idxs = selected_experts.flatten().sort() and expert_offsets =
 * bincount(...).cumsum(-1) (inclusive ends) -- cute_kernels/kernels/scattermoe/triton_implementation/__init__.py:14-36,82-83,
 * ops.py:295-316. Both index tensors int32 or both int64 (torch.sort returns int64); offsets int32 / uint32 or int64.
 * Outputs as ck_sort_by_expert writes them (counts, seg_starts, row_slot, tile_expert), plus
 *   row_pos[max_rows] -- padded row p of expert e holds sorted position starts[e] + p - seg_starts[e]: the row of an
 *                        UNPADDED grouped tensor [R, *] (the reference's grouped_in / grouped_out layout) that padded row p
 *                        stands for. Used as ck_segments::row_slot with a_gather_div = 1 to read such a tensor, and as
 *                        ck_segments::row_slot_out to write one.
 * One launch, no workspace. A position whose expert id is outside [0, E) or outside its expert's offset range owns no row. */
int ck_segments_from_sorted(const void* sorted_expert_idxs, const void* sorted_scattered_idxs, int32_t idxs_are_i64,
                            const void* expert_offsets, int32_t offsets_are_i64, int64_t R, int32_t E, int32_t align,
                            uint32_t* counts, int32_t* seg_starts, int32_t* row_slot, int32_t* row_pos,
                            int32_t* tile_expert, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * (b3) token-row gather / gated combine
 * Replaces: group(...) / group_triton_kernel -- triton_implementation/ops.py:108-140, kernels.py:225-280 -- and the
 *           bmm-based combine and d_gates of ops.py:173-174,214, and the .sum(-2) of ops.py:273-276.
 * ------------------------------------------------------------------------------------------------------------- */
/* out[n, :] = src[idx[n] / fan_out, :] * (coeff ? coeff[idx[n]] : 1), n < num_rows; src [*, H], out [num_rows, H].
 * coeff has the dtype of src. H * sizeof(dtype) must be a multiple of 16. */
int ck_gather_rows(const void* src, const int32_t* idx, const void* coeff, int32_t fan_out, int64_t num_rows,
                   int32_t H, void* out, int32_t dtype, void* stream);
/* out[t, :] = sum_j (gates ? gates[t, j] : 1) * expanded[t, j, :], fp32 accumulation; expanded [T, k, H].
 * If d_gates_out != NULL (needs grad_out [T, H]): d_gates_out[t, j] = <expanded[t, j, :], grad_out[t, :]> and `out`
 * may be NULL. gates / d_gates_out have the dtype of expanded. */
int ck_combine_rows(const void* expanded, const void* gates, int64_t T, int32_t k, int32_t H, void* out,
                    const void* grad_out, void* d_gates_out, int32_t dtype, void* stream);

/* d_gates[t, j] = <expanded[t, j, :], grad_out[t, :]> in fp32, whatever the dtype of the rows: the d_gates of
 * cute_kernels/kernels/scattermoe/triton_implementation/ops.py:214 (a bmm in the activation dtype there) kept unrounded,
 * so that the softmax backward of the router (ck_route_topk_softmax_bwd, fp32 d_gates) does not subtract rounded
 * numbers. expanded [T * k, H], grad_out [T, H], d_gates [T, k]. */
int ck_gate_grad_f32(const void* expanded, const void* grad_out, int64_t T, int32_t k, int32_t H, float* d_gates,
                     int32_t dtype, void* stream);
/* Padded grouped copy of token rows and (optionally) its transpose, for the grouped GEMMs below:
 *   row p valid : grouped[p, :] = src[row_slot[p] / fan_out, :] * (coeff ? coeff[row_slot[p]] : 1)
 *   row p pad   : zeros
 * fan_out == 0 (coeff must be NULL): src is itself padded-grouped [max_rows, H] and valid row p reads src[p, :].
 * grouped [max_rows, H] may be NULL; grouped_t [H, ld_t] (ld_t >= max_rows) may be NULL. bf16 / f16; fp32 for the
 * row-major copy alone (grouped_t NULL). */
int ck_group_rows_padded(const void* src, const void* coeff, int32_t fan_out, int32_t H, const int32_t* row_slot,
                         const int32_t* seg_starts, const uint32_t* counts, const int32_t* tile_expert,
                         int32_t align, int64_t max_rows, void* grouped, void* grouped_t, int64_t ld_t,
                         int32_t dtype, void* stream);
/* SwiGLU backward over padded grouped rows (formula: cute_kernels/kernels/swiglu/cuda_implementation/backward.cu:27-41),
 * writing what the weight-gradient GEMM consumes in the same pass:
 *   pre [max_rows, 2I] packed [up | gate], d_act [max_rows, I]  ->  d_pre [max_rows, 2I] (valid rows only) and
 *   d_pre_t [2I, ld_t] = d_pre^T with zeros in the pad rows of live tiles (may be NULL). I % 8 == 0. 16-bit dtypes.
 * act_kind: CK_ACT_SWIGLU (act = up * gate * sigmoid(gate)) or CK_ACT_GLU (act = up * sigmoid(gate), torch.nn.GLU on the
 * packed tensor: the activation of the reference's own MoE test, tests/test_commons.py:85). */
int ck_swiglu_bwd_grouped(const void* pre, const void* d_act, int32_t I, const int32_t* seg_starts,
                          const uint32_t* counts, const int32_t* tile_expert, int32_t align, int64_t max_rows,
                          void* d_pre, void* d_pre_t, int64_t ld_t, int32_t act_kind, int32_t dtype, void* stream);
/* Batched 2-D transpose: dst[b, c, r] = src[b, r, c]; src [batch, rows, cols]. 16-bit dtypes only. */
int ck_transpose_batched(const void* src, int64_t batch, int32_t rows, int32_t cols, void* dst, int32_t dtype,
                         void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * (c) scattered grouped GEMMs over tile-aligned expert segments (bf16 / f16 inputs, fp32 accumulation on MFMA)
 * Replaces: scatter2scatter + scatter2scatter_triton_kernel -- triton_implementation/ops.py:31-78, kernels.py:12-133 --
 *           group_bwd_W + groupXtY_triton_kernel -- ops.py:81-105, kernels.py:136-222 -- and the per-expert
 *           F.linear loop of torch_implementation.py:32-49.
 * Shared layout arguments come from ck_sort_by_expert (same `align`; align must be 128 or 256).
 * K and N must be multiples of 8.
 * ------------------------------------------------------------------------------------------------------------- */
typedef struct ck_segments {
  const int32_t* seg_starts;  /* [E + 1] */
  const uint32_t* counts;     /* [E] */
  const int32_t* tile_expert; /* [max_rows / align] */
  const int32_t* row_slot;    /* [max_rows]: the A row a padded row reads (divided by a_gather_div) */
  int64_t max_rows;
  int32_t num_experts;
  int32_t align;
  const int32_t* row_slot_out; /* [max_rows] or NULL (= row_slot): the output row a padded row writes in the scatter
                                  epilogues. Differs from row_slot when input and output are indexed differently, e.g. token
                                  rows in, unpadded grouped rows out (row_pos of ck_segments_from_sorted). */
} ck_segments;

/* Y = A_e * W[e]^T for every expert segment e. W [E, N, K].
 * A rows: a_gather_div > 0 : row p reads a[row_slot[p] / a_gather_div, :]   (a is [*, K], token order)
 *         a_gather_div == 0: row p reads a[p, :]                            (a is padded-grouped [max_rows, K])
 * Epilogue, selected by `epilogue`:
 *   CK_EPI_GROUPED        : y [max_rows, N] padded-grouped (valid rows only); y_t [N, ld_t] transposed copy with
 *                           zeros in pad rows, optional (NULL to skip)
 *   CK_EPI_SCATTER        : y [R, N]: valid row p is written to row row_slot_out[p] (row_slot[p] when that is NULL: back to
 *                           (token, slot) order)
 *                           both: aux_in, if not NULL, is a bias [E, N] whose row e joins the fp32 accumulators of expert
 *                           e's rows before the one rounding (F.linear with a bias, torch_implementation.py:42)
 *   CK_EPI_GELU_TANH      : as CK_EPI_GROUPED (bias included), and aux [max_rows, N] = tanh-approximated GELU of y, computed
 *                           from the rounded y as the activation module applied to y would (torch.nn.GELU("tanh"), the
 *                           non-GLU activation of the reference's layer test, tests/test_commons.py:85-86); no y_t
 *   CK_EPI_SWIGLU         : N = 2*I packed [up | gate] (cute_kernels/kernels/swiglu/__init__.py:121): writes the
 *                           pre-activation to y [max_rows, 2I], act = up*silu(gate) (computed from the rounded
 *                           pre-activation, as the unfused path would) to aux [max_rows, I], and act^T to
 *                           y_t [I, ld_t] (optional)
 *   CK_EPI_SWIGLU_BWD     : the GEMM result is d_act [rows, N = I]; aux_in = saved pre-activation [max_rows, 2I];
 *                           writes d_preact to y [max_rows, 2I] and its transpose to y_t [2I, ld_t] (optional)
 *                           (backward formula: cute_kernels/kernels/swiglu/cuda_implementation/backward.cu:27-41)
 */
#define CK_EPI_GROUPED 0
#define CK_EPI_SCATTER 1
#define CK_EPI_SWIGLU 2
#define CK_EPI_SWIGLU_BWD 3
#define CK_EPI_GLU 5 /* as CK_EPI_SWIGLU with act = up * sigmoid(gate): torch.nn.GLU() on the packed c_fc output */
#define CK_EPI_GELU_TANH 6
#define CK_ACT_SWIGLU 0
#define CK_ACT_GLU 1
#define CK_ACT_GELU_TANH 2
int ck_grouped_gemm(const void* a, int32_t a_gather_div, const void* w, int32_t N, int32_t K,
                    const ck_segments* seg, int32_t epilogue, void* y, void* y_t, int64_t ld_t, void* aux,
                    const void* aux_in, int32_t dtype, void* stream);
/* The same call with a workspace that lets the kernel split the contraction of its last, partial round of tiles. A
 * launch of t tiles runs in ceil(t / 256) rounds on the 256 CUs; when the last round is at most half full (and the
 * launch has at most 64 rounds and at least 16 K steps of 64), each of its tiles is computed by two to four workgroups (as
 * many as fill the chip), an equal share of the contraction each, which exchange fp32 partial tiles through the workspace; the last to arrive adds them in a
 * fixed order (results do not depend on arrival order) and runs the epilogue. Grouped and scatter epilogues of the
 * 256-row-tile kernel; every other case behaves like ck_grouped_gemm. No counterpart in the reference (its launches
 * are not tile-quantised the same way).
 * workspace: ck_grouped_gemm_workspace_bytes() bytes, 16-byte aligned, no initial contents required (the arrival words at
 * its end carry the launch's own epoch, so whatever an earlier or an interrupted launch left there reads as "nobody has
 * arrived"). One buffer per stream: launches that may run concurrently must not share one.
 * workspace NULL or too small: never split. */
int64_t ck_grouped_gemm_workspace_bytes(void);
int ck_grouped_gemm_ws(const void* a, int32_t a_gather_div, const void* w, int32_t N, int32_t K,
                       const ck_segments* seg, int32_t epilogue, void* y, void* y_t, int64_t ld_t, void* aux,
                       const void* aux_in, int32_t dtype, void* stream, void* workspace, int64_t workspace_bytes);
/* Input-gradient form of the grouped GEMM: y[p, :] = a[p, :] @ w[e(p)] with w [E, K, N] row-major, i.e. the weight
 * exactly as the forward pass stores it ([E, out, in] = [E, K, N] here: K = the forward's out, N = its in), read
 * contraction-strided instead of through a transposed copy.
 * Replaces: the dX calls of scatter2scatter on the permuted weight view -- cute_kernels/kernels/scattermoe/
 *           triton_implementation/ops.py:258-292 (expert_weights.permute(0, 2, 1) there; the Triton kernel takes strides).
 * a [max_rows, K] padded grouped rows; epilogue CK_EPI_GROUPED (y [max_rows, N]) or CK_EPI_SCATTER (y [R, N]).
 * Needs seg->align == 256, K % 64 == 0, N % 8 == 0. */
int ck_grouped_gemm_nn(const void* a, const void* w, int32_t N, int32_t K, const ck_segments* seg, int32_t epilogue,
                       void* y, int32_t dtype, void* stream);

/* ck_grouped_gemm_nn with the workspace of ck_grouped_gemm_ws (same rules). */
int ck_grouped_gemm_nn_ws(const void* a, const void* w, int32_t N, int32_t K, const ck_segments* seg, int32_t epilogue,
                          void* y, int32_t dtype, void* stream, void* workspace, int64_t workspace_bytes);

/* The same grouped GEMMs for fp32 tensors (the dtype of the reference's test grid, tests/test_commons.py:26-27): fp32
 * products and fp32 accumulation on v_mfma_f32_32x32x2_f32 (the reference's Triton kernels round fp32 operands to TF32,
 * kernels.py:131,218). y[out_row(p), :] = a[a_row(p), :] @ W_e (+ bias[e, :]) for every valid padded row p:
 *   a_row(p) = row_slot[p] / a_gather_div (a_gather_div > 0, token order) or p (0, padded grouped rows), a [*, K];
 *   W_e = w[e]^T with w [E, N, K] (w_is_kn == 0: the forward linears) or w[e] with w [E, K, N] (w_is_kn != 0: the input
 *   gradient, reading the forward's weight as stored); out_row(p) = row_slot[p] (scatter != 0) or p; bias [E, N] or NULL.
 * Replaces: scatter2scatter for fp32 inputs -- triton_implementation/ops.py:31-78. seg->align % 64 == 0; N, K % 4 == 0. */
int ck_grouped_gemm_f32(const float* a, int32_t a_gather_div, const float* w, int32_t w_is_kn, int32_t N, int32_t K,
                        const ck_segments* seg, int32_t scatter, float* y, const float* bias, void* stream);
/* dw[e] = a[rows of e]^T @ b[rows of e] for fp32 padded-grouped rows a [max_rows, M], b [max_rows, N]; dw [E, M, N], exact
 * zeros for experts without rows. Replaces: group_bwd_W for fp32 inputs -- ops.py:81-105. M, N % 4 == 0. */
int ck_grouped_gemm_dw_f32(const float* a, const float* b, int32_t M, int32_t N, const ck_segments* seg, float* dw,
                           void* stream);

/* dW[e] = A_t[:, seg_e] * B_t[:, seg_e]^T : A_t [M, ld_t], B_t [N, ld_t] are transposed padded-grouped operands with
 * zeros in pad rows; dw [E, M, N]. Experts with no rows get exact zeros (ops.py:252, kernels.py:181). */
int ck_grouped_gemm_dw(const void* a_t, const void* b_t, int64_t ld_t, int32_t M, int32_t N, const ck_segments* seg,
                       void* dw, int32_t dtype, void* stream);

/* The same weight gradient from row-major operands: dW[e] = A[seg_e, :]^T * B[seg_e, :] with a [max_rows, M] and
 * b [max_rows, N] padded-grouped rows (what the other kernels write anyway); no transposed copies. Pad rows may hold
 * anything: they are not read into the product.
 * Replaces: group_bwd_W / groupXtY_triton_kernel, which also reads DY and X row-major --
 *           cute_kernels/kernels/scattermoe/triton_implementation/ops.py:81-105, kernels.py:136-222.
 * dw [E, M, N]; experts with no rows get exact zeros. Needs seg->align % 64 == 0, M % 8 == 0, N % 8 == 0,
 * M >= 256 and N >= 256 (one 256 x 256 tile). */
int ck_grouped_gemm_dw_rows(const void* a, const void* b, int32_t M, int32_t N, const ck_segments* seg, void* dw,
                            int32_t dtype, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * (c, fp8) quantised-expert forward path: e4m3 operands (OCP e4m3fn, the gfx950 format), fp32 accumulation
 * No counterpart in the reference (it has no fp8 code): the semantics are those of the same layer evaluated on the
 * de-quantised operands, cute_kernels/kernels/scattermoe/torch_implementation.py:137-169.
 * ------------------------------------------------------------------------------------------------------------- */
/* Per-row quantisation: scales[r] = max|x[r, :]| / 448 (1 for an all-zero row), q[r, c] = e4m3(x[r, c] * (448 / max)),
 * round to nearest even. x [rows, cols] bf16 / f16, q [rows, cols] bytes, cols % 16 == 0. Used per token for
 * activations and per output channel ([E * out, in] rows) for expert weights. */
int ck_quant_rows_e4m3(const void* x, int64_t rows, int32_t cols, void* q, float* scales, int32_t dtype, void* stream);
/* Y = (A_e * diag(a_scale)) * (W[e] * diag(w_scale[e]))^T over tile-aligned expert segments (align must be 256).
 * a8: e4m3 rows [*, K], gathered like ck_grouped_gemm (a_gather_div); a_scale is indexed by the row of a8 that is read.
 * w8 [E, N, K] e4m3, w_scale [E, N]. K % 128 == 0. Epilogues: CK_EPI_GROUPED (y [max_rows, N]), CK_EPI_SCATTER
 * (y [R, N]), CK_EPI_SWIGLU (N = 2I packed [up | gate]; only the activation is written, to aux [max_rows, I]).
 * Outputs have `out_dtype` (bf16 / f16). */
int ck_grouped_gemm_fp8(const void* a8, const float* a_scale, int32_t a_gather_div, const void* w8,
                        const float* w_scale, int32_t N, int32_t K, const ck_segments* seg, int32_t epilogue, void* y,
                        void* aux, int32_t out_dtype, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * SwiGLU, stand-alone
 * Replaces: swiglu_forward_cuda / swiglu_backward_cuda -- cute_kernels/kernels/swiglu/cuda_implementation/ops.cpp:7-22,
 *           forward.cu:18-94, backward.cu:18-129 (and the strided Triton variants used for the packed form).
 * gate/up/out are [rows, cols] views with row strides in ELEMENTS (so the two halves of a packed tensor can be
 * passed without a copy). Any size is accepted; accesses are 128-bit when every pointer is 16-byte aligned and every
 * row stride and cols are multiples of 16 bytes (a flat tensor, rows == 1, only needs the pointers aligned), element-wise
 * otherwise.
 * ------------------------------------------------------------------------------------------------------------- */
int ck_swiglu_fwd(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out,
                  int64_t out_stride, int64_t rows, int64_t cols, int32_t dtype, void* stream);
int ck_swiglu_bwd(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, const void* d_out,
                  int64_t d_out_stride, void* d_gate, int64_t d_gate_stride, void* d_up, int64_t d_up_stride,
                  int64_t rows, int64_t cols, int32_t dtype, void* stream);
/* Backward of the activation of CK_EPI_GELU_TANH: d_pre[i] = d_act[i] * gelu_tanh'(pre[i]) over n contiguous elements
 * (what autograd derives for torch.nn.GELU("tanh"), the activation of tests/test_commons.py:85-86). bf16 / f16. */
int ck_gelu_tanh_bwd(const void* pre, const void* d_act, void* d_pre, int64_t n, int32_t dtype, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * (d) RMSNorm
 * Replaces: rmsnorm_forward_triton / rmsnorm_backward_triton -- cute_kernels/kernels/rmsnorm/triton_implementation/
 *           forward.py:14-85, backward.py:14-129; numerics follow F.rms_norm (rmsnorm/torch_implementation.py:9-10):
 *           the weight multiply happens in fp32 before the single rounding.
 * x, out, d_out, d_x [B, H] contiguous; weight [H] or NULL; rstd [B] fp32 or NULL (forward: written if non-NULL;
 * backward: read if non-NULL, recomputed from x and eps otherwise).
 * backward: d_weight_partial [ck_rmsnorm_bwd_partial_rows(B), H] fp32 workspace and d_weight [H] fp32 output, both
 * NULL when weight is NULL.
 * ------------------------------------------------------------------------------------------------------------- */
int ck_rmsnorm_fwd(const void* x, const void* weight, float eps, int64_t B, int32_t H, void* out, float* rstd,
                   int32_t dtype, void* stream);
int64_t ck_rmsnorm_bwd_partial_rows(int64_t B);
int ck_rmsnorm_bwd(const void* x, const void* weight, const void* d_out, const float* rstd, float eps, int64_t B,
                   int32_t H, void* d_x, float* d_weight_partial, float* d_weight, int32_t dtype, void* stream);

/* RMSNorm fused ahead of the router: one pass over x that writes y = rmsnorm(x), rstd, and the router logits
 * y @ gate_weight^T computed from the 16-bit y while the rows are in registers (fp32 accumulation, rounded to the rows'
 * dtype); with x8 / scale8, also the e4m3 rows and per-row scales that ck_quant_rows_e4m3 would derive from y.
 * y agrees with ck_rmsnorm_fwd's to within one rounding step of the rows' dtype, not bit for bit: this kernel sums the
 * squares of a row in another order, so rstd may differ in its last bits (about one element of y in a thousand then
 * rounds the other way). Logits, x8 and scale8 are exact functions of the y this kernel writes.
 * Replaces, as one kernel: rmsnorm_forward_triton -- cute_kernels/kernels/rmsnorm/triton_implementation/forward.py:14-53 --
 *           and the router's linear layer, self.gate(hidden_states) -- cute_kernels/kernels/scattermoe/
 *           torch_implementation.py:122-124 (and the per-row quantiser ahead of ck_grouped_gemm_fp8).
 * x, y [B, H]; norm_weight [H] or NULL; gate_weight [E, H]; logits [B, E]; rstd [B] fp32 or NULL; x8 [B, H] bytes and
 * scale8 [B] fp32, both or neither; gate_packed: workspace of 16 * ceil(E / 16) * H elements of the rows' dtype, written by
 * the call (the gate weight in the order the kernel's lanes read it). bf16 / f16. Needs H % 512 == 0, H <= 4096, E <= 128. */
int ck_rmsnorm_route(const void* x, const void* norm_weight, const void* gate_weight, float eps, int64_t B, int32_t H,
                     int32_t E, void* y, float* rstd, void* logits, void* x8, float* scale8, void* gate_packed,
                     int32_t dtype, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Expert biases
 * Replaces: the bias operand of F.linear in Experts_Torch.forward -- cute_kernels/kernels/scattermoe/
 *           torch_implementation.py:20-22,42 (one bias row [out] per expert; the reference's Triton path drops it,
 *           triton_implementation/__init__.py:26-36).
 * ck_add_expert_bias: y[r, :] += bias[e(r), :], y [rows, N], bias [E, N]. Padded grouped rows: pass seg, e(r) is the
 *   expert of the row's tile and pad rows are left alone. Token-order rows: pass row_expert [rows] (negative = skip).
 * ck_expert_bias_grad: d_bias[e, :] = sum of d_y over expert e's rows of the padded grouped layout (fp32 sums).
 * ------------------------------------------------------------------------------------------------------------- */
int ck_add_expert_bias(void* y, int64_t rows, int32_t N, const void* bias, const int32_t* row_expert,
                       const ck_segments* seg, int32_t dtype, void* stream);
int ck_expert_bias_grad(const void* d_y, int32_t N, const ck_segments* seg, void* d_bias, int32_t dtype, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Residual add fused with RMSNorm (the step in front of an MoE block in a transformer layer)
 * Replaces: fused_residual_add_rmsnorm_forward_triton / _backward_triton -- cute_kernels/kernels/
 *           fused_residual_add_rmsnorm/triton_implementation/forward.py:14-104, backward.py:14-149; semantics of
 *           fused_residual_add_rmsnorm_torch (torch_implementation.py:9-19).
 * forward:  added = (x * multiplier) + residual, each step rounded to the tensor dtype (multiplier == 1: no scaling);
 *           out = rmsnorm(added). x, residual, out, added [B, H]; rstd as above.
 * backward: g = d rmsnorm(added)/d added applied to d_out, plus d_added (the gradient arriving through the residual
 *           stream; NULL = none); d_residual = g, d_x = g * multiplier. `added` is the forward's output. With
 *           multiplier == 1 the two gradients are the same values: d_residual may then be the same buffer as d_x, and
 *           the rows are written once (any other multiplier with one buffer is an error).
 * ------------------------------------------------------------------------------------------------------------- */
int ck_fused_residual_add_rmsnorm_fwd(const void* x, const void* residual, const void* weight, float eps,
                                      float multiplier, int64_t B, int32_t H, void* out, void* added, float* rstd,
                                      int32_t dtype, void* stream);
int ck_fused_residual_add_rmsnorm_bwd(const void* added, const void* weight, const void* d_out, const void* d_added,
                                      const float* rstd, float eps, float multiplier, int64_t B, int32_t H, void* d_x,
                                      void* d_residual, float* d_weight_partial, float* d_weight, int32_t dtype,
                                      void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Softmax over the last dimension (what a load-balancing loss applies to the router logits the MoE layer returns)
 * Replaces: softmax_forward_triton / softmax_backward_triton -- cute_kernels/kernels/softmax/triton_implementation/
 *           (launched from kernels/softmax/__init__.py:12-36); semantics of softmax_torch (torch_implementation.py:9-18):
 *           fp32 math, x pre-multiplied by `multiplier` (pass 1 for none).
 * x, out, y, d_y, d_x [B, H] contiguous. backward: d_x = multiplier * y * (d_y - sum_h(d_y * y)).
 * ------------------------------------------------------------------------------------------------------------- */
int ck_softmax_fwd(const void* x, float multiplier, int64_t B, int32_t H, void* out, int32_t dtype, void* stream);
int ck_softmax_bwd(const void* y, const void* d_y, float multiplier, int64_t B, int32_t H, void* d_x, int32_t dtype,
                   void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CK_MI355_H */
