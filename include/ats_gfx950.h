/* libats_gfx950 — C ABI of the MI355X (gfx950) sparse-layer kernels.
 *
 * Every entry point
 *   - takes raw device pointers, sizes and a hipStream_t (passed as void*),
 *   - enqueues work on that stream and returns without synchronising,
 *   - never allocates, frees or retains memory (scratch comes in through a
 *     workspace pointer whose size a *_workspace() call reports),
 *   - returns ATS_OK or a negative error code and never terminates the
 *     process; ats_last_error_string() describes the last failure of the
 *     calling thread.
 *
 * This replaces, for the sparse-layer path, the two native interfaces of the
 * reference (paths relative to the reference checkout):
 *   - the extern "C" launchers of Src/Main_Scripts/core/transformer_ops.cu:331-436
 *     (rms_norm_launcher, rope_precompute_launcher, rope_apply_launcher), which
 *     return void and exit() on error (transformer_ops.cu:321-329);
 *   - the pybind11 module `moe_cuda_ops` of Src/Main_Scripts/core/moe_cuda_ops.cu:436-442
 *     (topk_gating, dispatch_tokens, combine_expert_outputs).
 * Data types: ATS_F32 / ATS_BF16 element tags; all accumulation is float32.
 */
#ifndef ATS_GFX950_H
#define ATS_GFX950_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ATS_OK 0
#define ATS_ERR_INVALID_ARG (-1)
#define ATS_ERR_UNSUPPORTED (-2)
#define ATS_ERR_LAUNCH (-3)
#define ATS_ERR_WORKSPACE (-4)

#define ATS_F32 0
#define ATS_BF16 1

#define ATS_ROUTE_SOFTMAX_TOPK 0 /* softmax over all experts, top-k, renormalise */
#define ATS_ROUTE_TOPK_SOFTMAX 1 /* top-k of the logits, softmax over the k     */

#define ATS_IDX_I32 0
#define ATS_IDX_I64 1

typedef void* ats_stream_t; /* hipStream_t */

/* Library identification and error text (no reference counterpart: the
 * reference prints to stderr and exits, transformer_ops.cu:321-329). */
int ats_version(void);
const char* ats_last_error_string(void);

/* ---- RMSNorm ------------------------------------------------------------
 * Replaces rms_norm_launcher (transformer_ops.cu:333-351); numerics follow
 * RMSNorm.forward of Src/Main_Scripts/core/model.py:263-299:
 *   y = ((float)x * rsqrt(mean(x^2) + eps) * (float)w) cast to x's type.
 * x, y: [rows, hidden] of x_dtype; w: [hidden] of w_dtype or NULL. */
int ats_rmsnorm_fwd(const void* x, const void* w, void* y, int64_t rows, int hidden, float eps,
                    int x_dtype, int w_dtype, ats_stream_t stream);

/* ---- RoPE ---------------------------------------------------------------
 * ats_rope_table replaces rope_precompute_launcher (transformer_ops.cu:353-370)
 * with the float64 evaluation of RotaryEmbedding._build_pytorch_cache
 * (model.py:378-402): angle = (float)pos / scaling * theta^(-2d/dim), cos/sin in
 * float64, stored as float32.  cols == dim writes both (duplicated) halves,
 * cols == dim/2 writes the half table of FusedRoPE (cuda_opt_wrapper.py:350-363). */
int ats_rope_table(float* cos_out, float* sin_out, int seq_len, int dim, int cols, double theta,
                   double scaling_factor, ats_stream_t stream);

/* ats_rope_fwd replaces rope_apply_launcher (transformer_ops.cu:372-392) and
 * follows apply_rotary_pos_emb_optimized (model.py:470-524): rotate-half with
 * separately rounded products and sum, float32 math, one rounding to the
 * element type.  q: [B,Hq,L,D], k: [B,Hkv,L,D] (Hq != Hkv allowed), inputs
 * addressed through element strides (batch, head, position; D contiguous),
 * outputs contiguous; in-place (out == in, contiguous) is allowed.  cos/sin:
 * float32 [table_len, >= D/2 used] with row stride table_stride; position of
 * row l is pos_offset + l and must be < table_len.  k_in may be NULL (Hkv = 0). */
int ats_rope_fwd(const void* q_in, const void* k_in, void* q_out, void* k_out, const float* cos_tab,
                 const float* sin_tab, int table_stride, int table_len, int B, int Hq, int Hkv, int L,
                 int D, int pos_offset, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
                 int64_t k_sh, int64_t k_sl, int dtype, ats_stream_t stream);
/* ats_rope_fwd whose rotated keys, and the values beside them, are appended to a key / value cache instead of
 * going into tensors of their own: the in-place form of torch.cat([past_key, k], dim=2) /
 * torch.cat([past_value, v], dim=2) in GroupedQueryAttention.forward (model.py:700-704) for a cache buffer
 * [B, Hkv, cache_capacity, D] with element strides (cache_sb, cache_sh, cache_sl; D contiguous) that holds
 * cache_pos positions: k (rotated) and v (copied bit for bit, addressed through v_sb / v_sh / v_sl like q and k)
 * land at positions cache_pos .. cache_pos + L - 1; q_out is contiguous [B, Hq, L, D].  The rotation uses
 * position pos_offset + l, independent of cache_pos (the reference rotates a decoding step's rows as positions
 * 0 .. L-1, model.py:690-698). */
int ats_rope_fwd_append(const void* q_in, const void* k_in, const void* v_in, void* q_out, void* k_cache,
                        void* v_cache, const float* cos_tab, const float* sin_tab, int table_stride,
                        int table_len, int B, int Hq, int Hkv, int L, int D, int pos_offset, int64_t q_sb,
                        int64_t q_sh, int64_t q_sl, int64_t k_sb, int64_t k_sh, int64_t k_sl, int64_t v_sb,
                        int64_t v_sh, int64_t v_sl, int64_t cache_sb, int64_t cache_sh, int64_t cache_sl,
                        int64_t cache_pos, int64_t cache_capacity, int dtype, ats_stream_t stream);

/* ---- Router -------------------------------------------------------------
 * logits[T,E] (float32) = x[T,H] . wg[E,H]^T (+ bias[E] if not NULL): the
 * nn.Linear(H, E, bias=False) gate of model.py:1124,1169. */
int ats_router_logits(const void* x, const void* wg, const float* bias, float* logits, int64_t T,
                      int H, int E, int dtype, ats_stream_t stream);

/* Routing.  Replaces moe_cuda_ops.topk_gating (moe_cuda_ops.cu:316-348) with the
 * semantics of the PyTorch paths: variant ATS_ROUTE_SOFTMAX_TOPK = model.py:1200-1217,
 * ATS_ROUTE_TOPK_SOFTMAX = moe_cuda_wrapper.py:229-233.  Selection is by
 * descending logit/temperature, lower expert id first among equal values.
 * Also produces what the auxiliary loss needs (model.py:1244-1263): hist[E]
 * (pre-capacity assignment counts), prob_colsum[E] (sum over tokens of
 * softmax(un-tempered logits)) and aux[1] = min(sum_e hist/(T*k) * colsum/T * E * lbw, 1).
 * idx_out: [T,k] int32; w_out: [T,k] float32.  hist/prob_colsum/aux may be NULL together. */
size_t ats_route_topk_workspace(int64_t T, int E);
int ats_route_topk(const float* logits, int64_t T, int E, int k, float temperature, int variant,
                   int32_t* idx_out, float* w_out, int32_t* hist, float* prob_colsum, float* aux,
                   float load_balancing_weight, void* workspace, size_t workspace_bytes,
                   ats_stream_t stream);

/* ---- Capacity dispatch ---------------------------------------------------
 * Deterministic restatement of the first-come-first-served loop of
 * MoECUDAOps._pytorch_dispatch (moe_cuda_wrapper.py:295-326), replacing
 * moe_cuda_ops.dispatch_tokens (moe_cuda_ops.cu:350-387, atomic order).
 * idx: [T,k] expert ids (int32 or int64).  Outputs (all int32, any may not be NULL):
 *   slot[T*k]       slot inside the expert, -1 when dropped
 *   token_map[E*C]  assignment id t*k+j per slot, -1 when empty
 *   hist[E], kept[E] = min(hist, C), offsets[E+1] = exclusive prefix of kept
 *   row_src[max(1,min(T*k, E*C))]  compact row (offsets[e]+slot) -> assignment id
 *   row_of[T*k]     assignment id -> compact row, -1 when dropped
 * status[1]: 0, or 1 when an expert id was outside [0,E). */
size_t ats_dispatch_plan_workspace(int64_t T, int k, int E);
int ats_dispatch_plan(const void* idx, int idx_dtype, int64_t T, int k, int E, int C, int32_t* slot,
                      int32_t* token_map, int32_t* hist, int32_t* kept, int32_t* offsets,
                      int32_t* row_src, int32_t* row_of, int32_t* status, void* workspace,
                      size_t workspace_bytes, ats_stream_t stream);

/* ats_dispatch_plan without a workspace argument, for callers that cannot allocate.  It has no
 * counterpart in the reference; it is for code under HIP graph capture, tight serving loops and
 * harnesses that forbid hipMalloc, which cannot provide (or size) a workspace.  Same arguments,
 * outputs and results as ats_dispatch_plan; the chunk histograms live in a fixed 4 MiB array in
 * device memory that each GPU the library runs on holds until the process ends, so the plan is
 * limited to ceil(T*k / 256) * E <= 1 048 576 (larger plans return ATS_ERR_WORKSPACE: use
 * ats_dispatch_plan).  The call allocates and frees nothing.  All calls on one GPU share that
 * GPU's array: calls that overlap on one GPU (different streams, or threads) race; calls ordered
 * on one stream are safe, and nothing needs clearing between them.  The first call on a device
 * looks up the array's address (hipGetSymbolAddress) and must therefore come before any capture. */
int ats_dispatch_plan_static(const void* idx, int idx_dtype, int64_t T, int k, int E, int C,
                             int32_t* slot, int32_t* token_map, int32_t* hist, int32_t* kept,
                             int32_t* offsets, int32_t* row_src, int32_t* row_of, int32_t* status,
                             ats_stream_t stream);

/* out[r,:] = src[map[r] / div, :] or zeros when map[r] < 0; r in [0, n_rows).
 * With map = token_map and div = k this fills expert_inputs[E,C,H]
 * (moe_cuda_wrapper.py:306-322); with div = 1 it is a plain row gather. */
int ats_gather_rows(const void* src, const int32_t* map, int div, void* out, int64_t n_rows, int H,
                    int dtype, ats_stream_t stream);

/* row_of[m] = r for every r in [0, n_slots) with m = token_map[r] >= 0; entries
 * of row_of not named by token_map are set to -1.  Lets the combine step work
 * from a bare token_map (moe_cuda_wrapper.py:343-357). */
int ats_invert_token_map(const int32_t* token_map, int64_t n_slots, int32_t* row_of,
                         int64_t n_assign, ats_stream_t stream);

/* ---- Expert FFN (grouped GEMMs) -------------------------------------------
 * SwiGLUExpert.forward (model.py:1071-1088) for all experts in one launch each.
 * Rows of expert e are row_start[e] .. row_start[e]+row_count[e]-1 of the row
 * space (compact: row_start = offsets; padded [E,C,*]: row_start = e*C).
 * gate/up: h[r, i] = silu(a_r . w_gu[e][i,:]) * (a_r . w_gu[e][I+i,:]), where a_r
 * is row r of `a`, or row a_rows[r]/a_row_div of `a` when a_rows != NULL (the
 * permutation gather fused into the operand load; a_num_rows = rows of `a`, every
 * gathered index must be below it; ignored when a_rows == NULL).  w_gu / w_d are device
 * arrays of E pointers to [2I,H] / [H,I] matrices.  h: [rows, I] of dtype;
 * down: y[r,:] = h[r,:] . w_d[e]^T, y of y_dtype (ATS_F32 or dtype).
 * max_rows bounds sum(row_count) (grid sizing only). */
int ats_grouped_gateup_swiglu(const void* a, int64_t a_num_rows, const int32_t* a_rows,
                              int a_row_div, const void* const* w_gu, void* h, const int32_t* row_start,
                              const int32_t* row_count, int E, int64_t max_rows, int H, int I,
                              int dtype, ats_stream_t stream);
int ats_grouped_down(const void* h, const void* const* w_d, void* y, const int32_t* row_start,
                     const int32_t* row_count, int E, int64_t max_rows, int H, int I, int dtype,
                     int y_dtype, ats_stream_t stream);
/* Backward of that pair for a training step: dh = dy . w_d (as the NT product against the
 * transposed weights w_dT[e] = [I, H]) with the gradient of h = silu(g) * u applied in the epilogue:
 * dgu[r, 0:I] = dh * u * (s + g*s*(1-s)), dgu[r, I:2I] = dh * g * s, s = sigmoid(g), g/u read from
 * gu [rows, 2I]; dh itself is never stored.  Same bits as ats_grouped_gemm_nt followed by
 * ats_silu_mul_bwd (reference: SwiGLUFunction.backward, MS/core/cuda_opt_wrapper.py:237-254, after
 * autograd's down_proj gradient).  ..._supported returns 1 for more than 256 rows per expert on
 * average, H a multiple of the 128-byte K slab and one expert's weights within 4 GiB.
 * dgu_t (optional, bfloat16 only; also h_t of ats_grouped_gateup_swiglu_save): the result once more,
 * transposed, in the layout of ats_transpose_grouped_rows -- dgu_t[c, t_col0[e] + m] for row m of
 * expert e, zeros up to the next multiple of 64 columns, row stride ld_t >= ats_wgrad_padded_rows,
 * t_col0 = the k_start of ats_wgrad_plan -- written from the same registers, so that the weight
 * gradient (autograd's dW = dY^T . X for nn.Linear, MS/core/model.py:882-893) needs no transposing
 * pass over this operand.  The columns of experts without rows are not written
 * (ats_transposed_zero_empty_groups clears them). */
int ats_grouped_down_dgrad_dsilu_supported(int E, int64_t max_rows, int H, int I, int dtype);
int ats_grouped_down_dgrad_dsilu(const void* dy, const void* const* w_dT, const void* gu, void* dgu,
                                 const int32_t* row_start, const int32_t* row_count, int E, int64_t max_rows,
                                 int H, int I, int dtype, void* dgu_t, int64_t ld_t, const int32_t* t_col0,
                                 ats_stream_t stream);
/* The same kernel reading the forward's own weights w_d[e] = [H, I] (reduction index H along the rows): no
 * transposed copy of the weights per step, the same bits.  bfloat16 only; ..._supported as above with H a
 * multiple of 64 and I of 8 (reference: autograd's down_proj input gradient, MS/core/model.py:882-893). */
int ats_grouped_down_dgrad_dsilu_nn_supported(int E, int64_t max_rows, int H, int I, int dtype);
int ats_grouped_down_dgrad_dsilu_nn(const void* dy, const void* const* w_d, const void* gu, void* dgu,
                                    const int32_t* row_start, const int32_t* row_count, int E, int64_t max_rows,
                                    int H, int I, int dtype, void* dgu_t, int64_t ld_t, const int32_t* t_col0,
                                    ats_stream_t stream);
/* The same projection for a training step: beside h it writes the gate / up pre-activations
 * gu[r, 0:I] and gu[r, I:2I] ([rows, 2I] of dtype, rounded from the same accumulators), which the
 * backward pass needs; replaces the plain product followed by ats_silu_mul_fwd (reference: the
 * expert's gate_proj / up_proj outputs kept by autograd, MS/core/model.py:882-893).  Available for
 * prefill-sized groups only: ..._save_supported returns 1 when it is (more than 768 rows per expert
 * on average, H a multiple of the 128-byte K slab, `a` and one expert's weights within 4 GiB),
 * otherwise the entry point fails with ATS_ERR_UNSUPPORTED. */
int ats_grouped_gateup_swiglu_save_supported(int64_t a_num_rows, int E, int64_t max_rows, int H, int I,
                                             int dtype);
int ats_grouped_gateup_swiglu_save(const void* a, int64_t a_num_rows, const int32_t* a_rows, int a_row_div,
                                   const void* const* w_gu, void* h, void* gu, const int32_t* row_start,
                                   const int32_t* row_count, int E, int64_t max_rows, int H, int I,
                                   int dtype, void* h_t, int64_t ld_t, const int32_t* t_col0,
                                   ats_stream_t stream);
/* The down projection of weight-streaming (decode) sizes, at most 256 rows per expert, split along
 * K so that enough workgroups stream the weights: slice s of expert e multiplies columns
 * [s*I/k_splits, (s+1)*I/k_splits) and writes float32 parts[s][row_start[e]+m][:H]
 * (parts: [k_splits, part_rows, H]).  The result is the sum over s, taken in slice order by
 * ats_sum_partials or ats_combine_partials.  I must be k_splits whole K slabs (64 bf16 / 32 f32
 * elements).  Same expert loop as ats_grouped_down (moe_cuda_wrapper.py:452-457). */
int ats_grouped_down_splitk(const void* h, const void* const* w_d, float* parts, const int32_t* row_start,
                            const int32_t* row_count, int E, int64_t max_rows, int64_t part_rows, int H,
                            int I, int k_splits, int dtype, ats_stream_t stream);
/* A gate/up projection of a few rows cut along K (ats_grouped_down_splitk run on the [2I, H] weight):
 * parts [n_parts, rows, 2I] float32, gate columns first; out[r,c] = silu(sum_s gate) * (sum_s up), rounded
 * once to out_dtype -- SwiGLUExpert.forward (model.py:1071-1088) on the summed accumulators.  I % 4 == 0. */
int ats_swiglu_partials(const float* parts, int n_parts, int64_t part_stride, void* out, int64_t rows, int I,
                        int out_dtype, ats_stream_t stream);
/* out[i] = sum_s parts[s*part_stride + i], i < n, added in slice order in float32 and rounded once
 * to out_dtype (n and part_stride multiples of 4). */
int ats_sum_partials(const float* parts, int n_parts, int64_t part_stride, void* out, int64_t n,
                     int out_dtype, ats_stream_t stream);

/* ---- Combine --------------------------------------------------------------
 * Token-major restatement of MoECUDAOps._pytorch_combine (moe_cuda_wrapper.py:328-359),
 * replacing moe_cuda_ops.combine_expert_outputs (moe_cuda_ops.cu:389-423, atomic adds):
 * out[t,:] = sum over the kept choices j of token t, in ascending row (= ascending
 * expert id) order, of w[t,j] * y[row_of[t*k+j], :]; float32 products and sums
 * rounded separately; zeros for a token with no kept choice.
 * If residual != NULL, out[t,:] = residual[t,:] + that sum. */
int ats_combine(const void* y, const int32_t* row_of, const float* w, const void* residual,
                void* out, int64_t T, int k, int H, int y_dtype, int out_dtype, ats_stream_t stream);
/* ats_combine whose token-major result is added onto rows of a larger tensor instead of being stored:
 * out[out_rows[t], :] += round(sum_j w[t,j] * y[row_of[t*k+j], :]) for out_rows[t] >= 0 (distinct rows), the
 * sum rounded to out_dtype first as the stored result would be; the bits of ats_combine followed by
 * ats_scatter_add_rows.  For a block that runs the experts on a subset of the tokens and adds the result
 * onto the residual stream at their positions.  k <= 8, H % 8 == 0, 16-byte aligned operands. */
int ats_combine_scatter_add(const void* y, const int32_t* row_of, const float* w, const int32_t* out_rows,
                            void* out, int64_t T, int k, int H, int y_dtype, int out_dtype, ats_stream_t stream);
/* ats_combine over the partial results of ats_grouped_down_splitk: expert row r is
 * sum_s parts[s*part_stride + r*H + :] (slice order, float32), rounded to out_dtype as the
 * unsplit projection rounds its result, then weighted and summed as above.  k <= 8, H % 8 == 0. */
int ats_combine_partials(const float* parts, int n_parts, int64_t part_stride, const int32_t* row_of,
                         const float* w, const void* residual, void* out, int64_t T, int k, int H,
                         int out_dtype, ats_stream_t stream);

/* ---- Mixture-of-Depths helpers -------------------------------------------
 * score[t] = x[t,:] . w[:] (+ bias[0]); optionally prob[t] = sigmoid(score/temperature)
 * (MoDRouter.forward, model.py:926-936). */
int ats_row_dot(const void* x, const void* w, const float* bias, float* score, float* prob,
                float temperature, int64_t T, int H, int dtype, ats_stream_t stream);
/* The same pass also writes the rows to copy_out [T, H] (optional, must not alias x): the residual
 * output of a Mixture-of-Depths block starts as a copy of its input (tokens that skip the block pass
 * through, model.py:1366-1404), and the scores read every row anyway. */
int ats_row_dot_copy(const void* x, const void* w, const float* bias, float* score, float* prob,
                     float temperature, void* copy_out, int64_t T, int H, int dtype, ats_stream_t stream);
/* Per sequence, positions of the `keep` largest scores (lower position first
 * among equals), written in ascending order as flat token ids b*L+pos:
 * sel[B*keep] int32.  L <= 8192. */
int ats_select_topk_per_sequence(const float* score, int B, int L, int keep, int32_t* sel,
                                 ats_stream_t stream);
/* base[rows[i], :] += delta[i, :] for i in [0, n) (rows distinct). */
int ats_scatter_add_rows(void* base, const int32_t* rows, const void* delta, int64_t n, int H,
                         int dtype, ats_stream_t stream);

/* mask[i] = 1.0f if v[i] >= (kth smallest of v, 1-based) else 0.0f: the inference
 * branch of MoDRouter.forward (model.py:984-990, kthvalue threshold).
 * workspace: at least 4 bytes of device memory, 8-byte aligned; when it holds 16 or
 * more, the int64 at byte offset 8 receives the number of ones in the mask (the
 * "computed tokens" statistic of model.py:990-995).  With the ats_kth_value_workspace(n) bytes
 * (16, or 4112 from 16384 values on) the radix select runs over many workgroups, one launch per
 * digit, instead of in one workgroup; n < 2^31. */
size_t ats_kth_value_workspace(int64_t n);
int ats_kth_value_mask(const float* v, int64_t n, int64_t kth, float* mask, void* workspace,
                       size_t workspace_bytes, ats_stream_t stream);

/* Training branch of MoDRouter.forward (model.py:941-952): mask[i] = 1.0f at exactly min(k, n) positions, the
 * k largest of v (among equal values the lower index first; torch.topk leaves that order to the library),
 * else 0.0f; ste (may be null) receives the straight-through weights (mask - v) + v, float32 in the
 * reference's order of operations.  workspace: ats_kth_value_workspace(n) bytes, 8-byte aligned.  n < 2^31. */
int ats_topk_mask_ste(const float* v, int64_t n, int64_t k, float* mask, float* ste, void* workspace,
                      size_t workspace_bytes, ats_stream_t stream);
/* Backward of that branch, which the reference leaves to autograd over model.py:923-952:
 * grad_logits[i] = (grad_weights[i] + grad_probs[i]) * p (1 - p) / temperature with p = prob[i] (either
 * gradient may be null), grad_bias[0] (may be null) = their sum, added in a fixed order.  The gradients of
 * the router's weight and of x follow from grad_logits through ats_router_bwd_dw / ats_router_bwd_dx
 * with one "expert". */
int ats_mod_route_bwd(const float* grad_weights, const float* grad_probs, const float* prob,
                      float temperature, float* grad_logits, float* grad_bias, int64_t n, ats_stream_t stream);

/* out = gate * silu(up), elementwise over n values: replaces swiglu_launcher
 * (transformer_ops.cu:394-409), the activation of the dense FusedSwiGLU wrapper
 * (cuda_opt_wrapper.py:476-478; note the convention differs from the experts'). */
int ats_swiglu_mul(const void* gate, const void* up, void* out, int64_t n, int dtype, ats_stream_t stream);

/* ---- Backward pass ---------------------------------------------------------
 * The reference trains through this path with PyTorch autograd (model.py) and,
 * for its fused ops, with explicit autograd Functions (cuda_opt_wrapper.py:85-254).
 * These entry points are the gradients of the forward entry points above.
 *
 * RMSNormFunction.backward (cuda_opt_wrapper.py:119-142): with g = dy*w,
 * r = rsqrt(mean(x^2)+eps):  dx = r*g - x*r^3*mean(g*x),  dw[h] = sum_rows dy*x*r
 * (float32, fixed summation order).  dw may be NULL; otherwise workspace must hold
 * ats_rmsnorm_bwd_workspace(rows, hidden) bytes, 16-byte aligned. */
size_t ats_rmsnorm_bwd_workspace(int64_t rows, int hidden);
int ats_rmsnorm_bwd(const void* x, const void* w, const void* dy, void* dx, float* dw, int64_t rows,
                    int hidden, float eps, int x_dtype, int w_dtype, void* workspace,
                    size_t workspace_bytes, ats_stream_t stream);
/* RoPEFunction.backward (cuda_opt_wrapper.py:180-207): the inverse rotation
 * (sin negated); arguments as ats_rope_fwd with gradients in place of q/k. */
int ats_rope_bwd(const void* dq_out, const void* dk_out, void* dq, void* dk, const float* cos_tab,
                 const float* sin_tab, int table_stride, int table_len, int B, int Hq, int Hkv, int L,
                 int D, int pos_offset, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
                 int64_t k_sh, int64_t k_sl, int dtype, ats_stream_t stream);
/* out = silu(a) * b on row-strided [rows, cols] operands (strides in elements), and its
 * gradient da = dout*b*(s + a*s*(1-s)), db = dout*a*s, s = sigmoid(a)
 * (SwiGLUFunction.backward, cuda_opt_wrapper.py:237-254; SwiGLUExpert, model.py:1071-1088:
 * a = gate half, b = up half of the [rows, 2I] projection).  rows_dev (optional device scalar)
 * lowers the row count to min(rows, *rows_dev), e.g. the number of kept rows of a dispatch plan. */
int ats_silu_mul_fwd(const void* a, int64_t lda, const void* b, int64_t ldb, void* out, int64_t ldo,
                     int64_t rows, const int32_t* rows_dev, int cols, int dtype, ats_stream_t stream);
int ats_silu_mul_bwd(const void* a, int64_t lda, const void* b, int64_t ldb, const void* dout,
                     int64_t ldd, void* da, int64_t ldda, void* db, int64_t lddb, int64_t rows,
                     const int32_t* rows_dev, int cols, int dtype, ats_stream_t stream);
/* Gradient of ats_combine: for expert row r with m = token_map[r] >= 0, t = m / k:
 * dy[r,:] = w[m] * dout[t,:], dw[m] = dout[t,:] . y[r,:]; rows with m < 0 and the dw of
 * dropped assignments are zero.  dw: [T*k] float32. */
int ats_combine_bwd(const void* dout, const void* y, const int32_t* token_map, const float* w, void* dy,
                    float* dw, int64_t n_rows, int64_t T, int k, int H, int y_dtype, int out_dtype,
                    ats_stream_t stream);
/* Gradient of the routing rule w.r.t. the router logits (mode 0: softmax -> top-k ->
 * renormalise, model.py:1200-1217; mode 1: top-k -> softmax, moe_cuda_wrapper.py:229-233)
 * plus, when usage != NULL, of the load-balancing loss (model.py:1244-1263) taken on
 * logits_aux: the factor aux_scale * (aux_scale_dev ? *aux_scale_dev : 1) must equal
 * dL/daux * E * load_balancing_weight / T (0 where the loss is clamped); usage[e] as in the
 * forward (a constant).  logits_route are the logits the routing saw (with noise, if any). */
int ats_route_bwd(const float* logits_route, const float* logits_aux, const int32_t* idx, const float* w,
                  const float* dw, const float* usage, float aux_scale, const float* aux_scale_dev,
                  float temperature, int mode, float* dlogits, int64_t T, int E, int k,
                  ats_stream_t stream);
/* Gradient of ats_router_logits: out[t,:] = base[t,:] + dlogits[t,:] . Wg (base NULL or == out),
 * dWg[e,:] = sum_t dlogits[t,e] * x[t,:] (float32, fixed order). */
int ats_router_bwd_dx(const float* dlogits, const void* wg, const void* base, void* out, int64_t T, int E,
                      int H, int dtype, ats_stream_t stream);
size_t ats_router_bwd_dw_workspace(int64_t T, int E, int H);
int ats_router_bwd_dw(const float* dlogits, const void* x, float* dwg, int64_t T, int E, int H, int dtype,
                      void* workspace, size_t workspace_bytes, ats_stream_t stream);
/* Transposes that make the contraction dimension contiguous for the backward GEMMs:
 * E matrices [R, C] -> [C, R]; and grouped rows [*, C] (row r of expert e, optionally
 * gathered as in ats_grouped_gateup_swiglu) -> [C, ld_out] where expert e owns the columns
 * k_start[e] .. k_start[e]+k_count[e]-1, k_count[e] = max(64, roundup(row_count[e], 64)),
 * zero padded (ats_wgrad_plan writes k_start/k_count; ld_out >= ats_wgrad_padded_rows).
 * aligned_bases != 0 promises that every matrix in both pointer tables is 16-byte aligned. */
int ats_transpose_batched(const void* const* in_ptrs, void* const* out_ptrs, int E, int R, int C, int dtype,
                          int aligned_bases, ats_stream_t stream);
int64_t ats_wgrad_padded_rows(int64_t max_rows, int E);
int ats_wgrad_plan(const int32_t* row_count, int E, int32_t* k_start, int32_t* k_count, ats_stream_t stream);
int ats_transpose_grouped_rows(const void* in, int64_t ld_in, int C, const int32_t* gather, int gather_div,
                               const int32_t* row_start, const int32_t* row_count, int E, int64_t max_rows,
                               void* out, int64_t ld_out, int dtype, ats_stream_t stream);
/* Clears the 64 columns that every expert without rows owns in a transposed matrix [C, ld] of that layout. */
int ats_transposed_zero_empty_groups(void* out, int64_t ld, int C, const int32_t* row_count,
                                     const int32_t* k_start, int E, int dtype, ats_stream_t stream);
/* General grouped product with K contiguous in both operands:
 * out[row_start[e]+m, n] = sum_k A_e[m,k] * B_e[n,k], m < row_count[e], n < N.
 * A_e = rows row_start[e].. of `a` (optionally gathered through a_rows), or a_ptrs[e] with rows
 * counted from 0; B_e = b_ptrs[e] ([b_rows >= N, ldb]); K_e = k_count[e] when given.
 * Serves the training forward (gate/up pre-activations), dgrad (B = transposed weights)
 * and wgrad (A, B = transposed activations, one "expert" per weight matrix). */
int ats_grouped_gemm_nt(const void* a, const void* const* a_ptrs, int64_t lda, int64_t a_num_rows,
                        const int32_t* a_rows, int a_row_div, const void* const* b_ptrs, int64_t ldb,
                        int64_t b_rows, void* out, int64_t ldo, const int32_t* row_start,
                        const int32_t* row_count, const int32_t* k_count, int E, int64_t max_rows, int N,
                        int K, int dtype, int out_dtype, ats_stream_t stream);
/* Grouped product against weights stored with the reduction index along their rows:
 * out[row_start[e]+m, n] = sum_k A_e[m,k] * B_e[k,n], B_e = b_ptrs[e] ([K, ldb >= N]).
 * The data gradient of a linear layer, dX = dY . W with W = [out_features, in_features] as the forward holds it
 * (autograd's input gradient of nn.Linear, MS/core/model.py:882-893), without a transposed copy of W; same bits
 * as ats_grouped_gemm_nt on the transposed copy.  bfloat16 operands, prefill-sized groups only: ..._supported
 * returns 1 for more than 192 rows per expert on average, K a multiple of 64, N and ldb multiples of 8 and one
 * expert's weights within 4 GiB; otherwise transpose (ats_transpose_batched) and call ats_grouped_gemm_nt. */
int ats_grouped_gemm_nn_supported(int E, int64_t max_rows, int N, int K, int64_t ldb, int dtype);
int ats_grouped_gemm_nn(const void* a, int64_t lda, int64_t a_num_rows, const int32_t* a_rows, int a_row_div,
                        const void* const* b_ptrs, int64_t ldb, void* out, int64_t ldo, const int32_t* row_start,
                        const int32_t* row_count, int E, int64_t max_rows, int N, int K, int dtype, int out_dtype,
                        ats_stream_t stream);

/* ---- Causal grouped-query attention (forward) -----------------------------------
 * Replaces GroupedQueryAttention._standard_attention / _flash_attention
 * (Src/Main_Scripts/core/model.py:757-839): softmax(q.k^T * scale + causal mask) . v with float32
 * scores and softmax, probabilities rounded to bf16, output laid out [B, L, Hq*D] (the layout o_proj
 * consumes).  bf16 only, D = 64 or 128, Hq a multiple of Hkv (query head h reads kv head h / (Hq/Hkv)).
 * q: [B,Hq,L,D] contiguous; k: the Lk rows of a (batch, head) follow one another (D elements each) from
 * base + b*k_sb + h*k_sh, so a [B,Hkv,Lk,D] tensor or the first Lk rows of a larger cache buffer
 * [B,Hkv,capacity,D] is read in place; Lk >= L; v: rows of D contiguous elements addressed as
 * base + b*v_sb + j*v_sl + h*v_sh, so a [B,Hkv,Lk,D] tensor, a cache buffer or a view of a fused
 * projection output [B,Lk,Hkv,D] is read in place (element strides, multiples of 8).  With Lk > L the first Lk - L keys are a
 * cache in front of the queries (model.py:700-704): query i sits at position i + Lk - L and sees keys up
 * to there.  The reference's masked path only runs that case for L = 1 (its [L, L] mask does not
 * broadcast otherwise); its flash path aligns the diagonal the same way.
 * key_bias (optional): [B,Lk] float32 added to the scaled scores of a key for every query and head; the
 * reference's padding mask is (1 - attention_mask) * -1e4 (model.py:819-824).
 * lse (optional): [B,Hq,L] float32 log-sum-exp of the scaled (and biased) scores per query.
 * workspace (optional): with few query rows against many keys (decoding a handful of sequences) one workgroup
 * per (batch, head group) cannot fill the chip; given ats_attention_fwd_workspace(...) bytes of scratch the
 * keys are cut into ranges that run side by side and a second kernel merges their partial softmax results
 * (same values up to float32 rounding of the merge).  The size query returns 0 where that does not apply;
 * NULL / too small a workspace selects the single-pass kernel. */
size_t ats_attention_fwd_workspace(int B, int Hq, int Hkv, int L, int Lk, int D);
int ats_attention_fwd(const void* q, const void* k, int64_t k_sb, int64_t k_sh, const void* v, int64_t v_sb,
                      int64_t v_sl, int64_t v_sh, const float* key_bias, void* out, float* lse, int B, int Hq,
                      int Hkv, int L, int Lk, int D, float scale, void* workspace, size_t workspace_bytes,
                      ats_stream_t stream);
/* The same with the two options of the reference's masked path that the plain entry point leaves out
 * (model.py:819-833):
 *   bias_qk (optional): float32 [L, Lk] matrices added to the scaled scores of (query, key); a [B,1,L,Lk]
 *     attention mask is (1 - mask) * -1e4.  The matrix of (batch b, query head h) starts at
 *     bias_qk + b * bias_sb + h * bias_sh floats: bias_sb = 0 shares one matrix over the batch, bias_sh = 0
 *     over the heads ([B,1,L,Lk] masks), bias_sh = L * Lk gives every head its own ([B,H,L,Lk] masks).
 *   dropout_p in [0, 1): each attention weight is dropped with this probability and the kept ones are scaled
 *     by 1 / (1 - p) before they meet V (nn.Dropout on the weights while training); the log-sum-exp is that of
 *     the undropped scores.  Keep / drop is a function of (dropout_seed, batch, head, query, key) only, so
 *     ats_attention_bwd_ex given the same seed sees the same mask; it is not torch's generator stream.
 * With either option a per-key bias must be folded into bias_qk by the caller (key_bias must be NULL), and the
 * single-pass kernel without the software pipeline runs.  Neither option set: identical to ats_attention_fwd. */
int ats_attention_fwd_ex(const void* q, const void* k, int64_t k_sb, int64_t k_sh, const void* v, int64_t v_sb,
                         int64_t v_sl, int64_t v_sh, const float* key_bias, const float* bias_qk, int64_t bias_sb,
                         int64_t bias_sh, float dropout_p, uint64_t dropout_seed, void* out, float* lse, int B, int Hq,
                         int Hkv, int L, int Lk, int D, float scale, void* workspace, size_t workspace_bytes,
                         ats_stream_t stream);

/* ---- Causal grouped-query attention (backward) ----------------------------------
 * The reference leaves this gradient to autograd (model.py:757-839 under torch.autograd); the kernels
 * recompute the probabilities from the forward's log-sum-exp and form
 *   dV = P^T.dO, dP = dO.V^T, dS = P*(dP - delta)*scale, dQ = dS.K, dK = dS^T.Q
 * without atomics (one kernel owns query rows, one owns key rows and sums over the query heads of
 * its kv head).  ats_attention_delta: delta[B,Hq,L] = sum_d dO*O with out, dout [B,L,Hq*D].
 * ats_attention_bwd: q [B,Hq,L,D], k, v [B,Hkv,Lk,D], dout [B,L,Hq*D] contiguous; lse, delta [B,Hq,L];
 * key_bias as in the forward (optional); dq, dk, dv shaped like q, k, v. */
int ats_attention_delta(const void* out, const void* dout, float* delta, int B, int Hq, int L, int D,
                        ats_stream_t stream);
int ats_attention_bwd(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                      const float* delta, const float* key_bias, void* dq, void* dk, void* dv, int B, int Hq, int Hkv,
                      int L, int Lk, int D, float scale, ats_stream_t stream);
/* Backward with the options of ats_attention_fwd_ex (same bias_qk, dropout_p and dropout_seed as the forward
 * call whose lse is passed; delta from ats_attention_delta on the forward's output as usual). */
int ats_attention_bwd_ex(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                         const float* delta, const float* key_bias, const float* bias_qk, int64_t bias_sb,
                         int64_t bias_sh, float dropout_p, uint64_t dropout_seed, void* dq, void* dk, void* dv, int B,
                         int Hq, int Hkv, int L, int Lk, int D, float scale, ats_stream_t stream);
/* ats_attention_bwd_ex without the separate ats_attention_delta launch: the dQ kernel, whose lanes hold the dO
 * rows already, forms delta from them and the forward's output `out` [B,L,Hq*D] and writes it to delta_ws
 * [B,Hq,L] (float32, caller's), where the dK/dV kernel behind it reads it.  Same gradient as autograd's for
 * model.py:757-839; delta is summed in another order than ats_attention_delta sums it (float32 rounding). */
int ats_attention_bwd_out(const void* q, const void* k, const void* v, const void* out, const void* dout,
                          const float* lse, float* delta_ws, const float* key_bias, const float* bias_qk,
                          int64_t bias_sb, int64_t bias_sh, float dropout_p, uint64_t dropout_seed, void* dq, void* dk,
                          void* dv, int B, int Hq, int Hkv, int L, int Lk, int D, float scale, ats_stream_t stream);

/* ---- Float32 attention: the row softmax between two grouped products --------------
 * _standard_attention on float32 tensors (model.py:807-839) materialises the scores; so does this path:
 * scores = q.k^T per (batch, head) through ats_grouped_gemm_nt, ats_attention_softmax_f32 in place, then
 * weights.v through ats_grouped_gemm_nt again (the host mirror composes them, ops.attention_f32).
 * scores: [B * Hq, Lp, ld] float32, row r of head e at (e * Lp + r) * ld; rows >= L and columns >= Lk are
 * padding (written as zeros; Lp, ld multiples of 4 for the products).  Applied in the reference's order: scale,
 * causal fill with -1e4 (query i sees keys up to i + Lk - L), + key_bias [B, Lk], + bias_qk (both optional,
 * bias_sb / bias_sh as in ats_attention_fwd_ex), float32 softmax; with dropout_p > 0 weights_drop receives the weights
 * after dropout (same keep / drop function as ats_attention_fwd_ex) and scores keeps the undropped ones.
 * ats_attention_softmax_bwd_f32: dp = gradient of the dropped weights on entry, gradient of the raw scores on
 * return: P * (dP' - sum_j P dP') * scale, dP' = keep * dP / (1 - p). */
int ats_attention_softmax_f32(float* scores, float* weights_drop, int B, int Hq, int L, int Lp, int Lk, int ld,
                              float scale, const float* key_bias, const float* bias_qk, int64_t bias_sb,
                              int64_t bias_sh, float dropout_p, uint64_t dropout_seed, ats_stream_t stream);
int ats_attention_softmax_bwd_f32(const float* weights, float* dp, int B, int Hq, int L, int Lp, int Lk, int ld,
                                  float scale, float dropout_p, uint64_t dropout_seed, ats_stream_t stream);

/* ---- Training-step ops beside the sparse layer --------------------------------
 * Fused cross-entropy + accuracy.  Replaces fused_cross_entropy_accuracy_launcher
 * (Src/Main_Scripts/training/fused_loss.cu:179-214); numerics follow FusedLoss._pytorch_fallback
 * (Src/Main_Scripts/training/cuda_kernels.py:191-249).  A token is ignored when its label equals
 * pad_id or lies outside [0, V).  Per token: loss_tok = logsumexp(z) - z[label] (10.0 if not
 * finite), lse, correct (arg-max == label, lower index among equal logits), valid.
 * sums[5] = {sum w*loss, sum w, sum loss, sum correct, valid count} over valid tokens
 * (w = weights[t], 1 when weights == NULL), added in a fixed order.  logits: [T, V] of dtype. */
int ats_cross_entropy_fwd(const void* logits, const int64_t* labels, int64_t pad_id, const float* weights,
                          float* loss_tok, float* lse, float* correct, float* valid, float* sums, int64_t T,
                          int V, int dtype, ats_stream_t stream);
/* Gradient of sums[0] / max(sums[1], 1e-8) w.r.t. the logits, times the device scalar scale[0]:
 * dlogits[t,v] = scale * w_t * valid_t / max(sums[1], 1e-8) * (exp(z - lse_t) - [v == label_t]).
 * (The reference's fused loss returns a value without a graph; its fallback uses autograd.) */
int ats_cross_entropy_bwd(const void* logits, const int64_t* labels, const float* lse, const float* valid,
                          const float* weights, const float* sums, const float* scale, void* dlogits, int64_t T,
                          int V, int dtype, ats_stream_t stream);
/* Multi-tensor gradient norm and clipping.  Replaces fused_grad_clip_launcher
 * (Src/Main_Scripts/training/fused_grad_clip.cu:117-175) without its synchronisation and atomics.
 * grad_ptrs/sizes: n_tensors tensors of one dtype; chunk_start[n_tensors+1]: running count of
 * ats_grad_clip_chunk_elems()-sized chunks (built by the host), n_chunks = chunk_start[n_tensors];
 * partial: n_chunks floats of scratch.  norm_out[0] = sqrt(extra_sumsq[0] + sum of squares),
 * norm_out[1] = that sum (so groups of different dtype can be chained through extra_sumsq).
 * do_clip: 0 = norm only; 1 = norm, then grads *= max_norm / (norm + 1e-6) if that is < 1;
 * 2 = scale only, with the norm already in norm_out[0]. */
int ats_grad_clip_chunk_elems(void);
int ats_grad_norm_clip(void* const* grad_ptrs, const int64_t* sizes, const int32_t* chunk_start, int n_tensors,
                       int n_chunks, int dtype, const float* extra_sumsq, float* partial, float* norm_out,
                       float max_norm, int do_clip, ats_stream_t stream);

/* ---- The reference's own launcher names ---------------------------------------
 * Exact float32 signatures of Src/Main_Scripts/core/transformer_ops.cu:331-409, so that the ctypes
 * loader of Src/Main_Scripts/core/cuda_opt_wrapper.py:50-79 binds this library unchanged (call sites
 * cuda_opt_wrapper.py:98-108, 156-169, 219-228, 337-344).  Thin aliases of ats_rmsnorm_fwd,
 * ats_rope_table (half-width table), ats_rope_fwd (in place, q and k with the same head count, as
 * that signature has it; the caller guarantees position_offset + seq_len <= max_seq_len) and
 * ats_swiglu_mul.  They return void like the originals but never exit(): the status of the calling
 * thread's last legacy call is ats_legacy_last_status(), its text ats_last_error_string().
 * swiglu_fused_launcher (transformer_ops.cu:411-434; no call site in the reference's Python) is the
 * product x . gate_weight^T times silu(x . up_weight^T) with float32 weights [intermediate, hidden]; like
 * the original it accepts the biases and does not apply them.  It owns a stream-ordered scratch
 * allocation of 2 * total_tokens * intermediate_size floats. */
void rms_norm_launcher(const float* input, const float* weight, float* output, int batch_seq,
                       int hidden_size, float eps, ats_stream_t stream);
void rope_precompute_launcher(float* cos_cache, float* sin_cache, int max_seq_len, int head_dim,
                              float theta, ats_stream_t stream);
void rope_apply_launcher(float* q, float* k, const float* cos, const float* sin, int batch_size,
                         int num_heads, int seq_len, int head_dim, int position_offset,
                         ats_stream_t stream);
void swiglu_launcher(const float* gate, const float* up, float* output, int total_tokens,
                     int intermediate_size, ats_stream_t stream);
void swiglu_fused_launcher(const float* input, const float* gate_weight, const float* up_weight,
                           const float* gate_bias, const float* up_bias, float* output, int total_tokens,
                           int hidden_size, int intermediate_size, bool use_bias, ats_stream_t stream);
/* The training-step launchers the reference's second loader binds (Src/Main_Scripts/training/cuda_kernels.py:
 * 60-78, call sites 154-164 and 340-346), with the signatures of training/fused_loss.cu:183-193 and
 * training/fused_grad_clip.cu:117-123.  Aliases of ats_cross_entropy_fwd and ats_grad_norm_clip that own
 * their scratch memory (stream-ordered allocations), as the originals do: loss_out = sum of the token losses,
 * accuracy_out = number of correct arg-max predictions (float), valid_tokens_out = valid tokens (int64);
 * fused_grad_clip_launcher returns the total norm (which synchronises the stream, as in the original) after
 * scaling the float32 gradients by max_norm / (norm + 1e-6) when that is below 1. */
void fused_cross_entropy_accuracy_launcher(const float* logits, const int64_t* labels, int64_t pad_token_id,
                                           float* loss_out, float* accuracy_out, int64_t* valid_tokens_out,
                                           int total_tokens, int vocab_size, ats_stream_t stream);
float fused_grad_clip_launcher(float** grad_ptrs_device, int* grad_sizes_device, int num_tensors, float max_norm,
                               ats_stream_t stream);
int ats_legacy_last_status(void);

/* ---- Host-side views of the grouped-GEMM tile schedule (no device work) ----
 * No reference counterpart; used to test the block -> (expert, m-tile, n-tile, K slice)
 * map on the CPU.  row_count_host is a host array; aligned = 1 rounds every group's tile
 * count up to a multiple of SM; k_slices >= 1.  decode returns 1 and fills
 * out4 = {expert, m_tile, n_tile, slice} when the block owns a tile, else 0.  grid_blocks
 * takes max_rows and E already multiplied by the number of K slices. */
int ats_debug_decode_tile(int64_t block, const int32_t* row_count_host, int E, int BM, int n_tiles,
                          int SM, int SN, int aligned, int k_slices, int32_t* out4);
int64_t ats_debug_grid_blocks(int64_t max_rows, int E, int BM, int n_tiles, int SM, int SN, int aligned);
/* The same map as the GEMM kernels evaluate it on the device (a wave-parallel search): out4_dev
 * [n_blocks, 4] int32 receives {expert, m_tile, n_tile, slice} per block id, -1s where the block
 * owns no tile.  row_count_dev is a device array. */
int ats_debug_decode_tiles_device(const int32_t* row_count_dev, int E, int BM, int n_tiles, int SM, int SN,
                                  int aligned, int k_slices, int64_t n_blocks, int32_t* out4_dev,
                                  ats_stream_t stream);

/* ---- Calibration loop for the benchmark ----
 * No reference counterpart (the reference's benchmark, Src/Main_Scripts/core/cuda_debug_script.py,
 * reports times only).  Launches 256 workgroups of 8 waves (one per compute unit) that issue `iters` rounds of independent
 * bf16 MFMAs on operands held in registers: shape 0 = v_mfma_f32_32x32x16_bf16, 1 =
 * v_mfma_f32_16x16x32_bf16; random_operands 0 = all-zero bits, 1 = normal deviates of standard
 * deviation 0.5.  *flop_out (host) receives the flop count of the launch; clocks_dev (device, two uint64,
 * may be null) receives the core-clock cycles and the 100 MHz ticks that workgroup 0 spent in the loop.
 * The caller times the launch with events on `stream`. */
int ats_calibrate_mfma(int shape, int random_operands, int iters, uint64_t* clocks_dev, double* flop_out,
                       ats_stream_t stream);
/* Plain streaming copy of `bytes` (a multiple of 16; both pointers 16-byte aligned): the yardstick that the
 * benchmark prints beside the bandwidth-bound kernels.  No reference counterpart. */
int ats_calibrate_copy(const void* src, void* dst, size_t bytes, ats_stream_t stream);
/* Plain streaming read of `bytes` (a multiple of 16; src 16-byte aligned; sink: 4 writable device bytes that are
 * not written in practice): the yardstick that the benchmark prints beside the weight-streaming kernels of the
 * decode-sized workloads.  No reference counterpart. */
int ats_calibrate_read(const void* src, size_t bytes, void* sink, ats_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ATS_GFX950_H */
