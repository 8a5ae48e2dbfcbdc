/*
 * piper_amd.h -- C ABI of libpiper_amd.so: the per-device compute of one Piper stage
 * (MoE expert region + ZeRO bucket path) as hand-written gfx950 HIP kernels.
 *
 * Conventions for every entry point
 *   - all pointers are DEVICE pointers unless the parameter is documented "host";
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *   - nothing synchronises the host, nothing allocates: scratch memory is passed
 *     in by the caller and sized by the matching *_workspace_bytes query;
 *   - the return value is 0 on success, a negative PK_ERR_* code for an argument
 *     error (nothing was launched), or a positive hipError_t value;
 *   - `dtype` arguments use the PK_F32 / PK_BF16 codes below;
 *   - row-major, contiguous tensors; T tokens, H hidden, E experts, K top-k,
 *     I expert intermediate size, A = T*K routed rows.
 *
 * The reference (github.com/uw-syfi/piper) is pure Python, so there is no FFI to
 * mirror symbol-for-symbol; each entry point names the reference ATen sequence it
 * replaces (file:line under the reference tree).
 */
#ifndef PIPER_AMD_H
#define PIPER_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PK_OK 0
#define PK_ERR_ARG (-1)         /* null pointer / negative size / bad enum            */
#define PK_ERR_SHAPE (-2)       /* shape not supported by the kernels (see each call) */
#define PK_ERR_ALIGN (-3)       /* pointer or leading dimension not 16-byte aligned   */
#define PK_ERR_WORKSPACE (-4)   /* workspace too small                                */
#define PK_ERR_UNSUPPORTED (-5) /* dtype / option combination not built               */

#define PK_F32 0
#define PK_BF16 1

#define PK_MAX_EXPERTS 1024
#define PK_MAX_TOPK 64


typedef void* pk_stream_t;

#define PK_API __attribute__((visibility("default")))

/* Library version (major*10000 + minor*100 + patch) and a static message for a
 * negative status code. */
PK_API int pk_version(void);
PK_API const char* pk_status_string(int status);

/* Optional set-up for the CURRENT device: resolves the device addresses of the library's own
 * device arrays (the scheduling counters of the grouped GEMMs, the scratch of
 * pk_sort_by_expert_static) and reads the device's CU count.  Every entry point does this by
 * itself on its first call on a device; a caller that records launches into a HIP graph calls
 * pk_init() (or makes one ordinary call of each entry point it will record) on that device BEFORE
 * the capture starts, because symbol look-ups are not legal while a stream is capturing.
 * No counterpart in the reference (its operators are ATen calls). */
PK_API int pk_init(void);

/* ------------------------------------------------------------------ routing */

/* logits[T,E] (f32) = x[T,H] (x_dtype) . w_gate[E,H]^T (f32) + gate_bias[E] (f32, may be NULL),
 * fp32 products and accumulation.  The hidden dimension is split over workgroups into
 * `workspace` (pk_gate_workspace_bytes) and summed in a fixed order; without a workspace it
 * runs unsplit.  Replaces the gate Linear inside `self.router(x, expert_bias)`
 * (examples/models/qwen3.py:237-241; MoEArgs.gate_bias at :45). */
PK_API int64_t pk_gate_workspace_bytes(int64_t T, int64_t H, int64_t E);
PK_API int pk_gate_logits(const void* x, int x_dtype, const float* w_gate, const float* gate_bias,
                   float* logits, int64_t T, int64_t H, int64_t E, void* workspace,
                   int64_t workspace_bytes, pk_stream_t stream);

/* Softmax over experts in fp32, top-K selection, optional renormalisation of the K
 * selected scores (route_norm) and scaling (route_scale).
 *   selection key: the fp32 logit; larger first; equal logits -> lower expert index first
 *   (-0.0 == +0.0; NaN sorts as largest, as torch.sort does).
 *   top_scores[T,K] f32, top_idx[T,K] i32 in selection order (best first).
 * Replaces the softmax/top-k/renorm part of the router call (qwen3.py:237-241,
 * score_func="softmax", route_norm/route_scale at qwen3.py:43-44,172-173).
 * Limits: 1 <= K <= min(E, PK_MAX_TOPK), E <= PK_MAX_EXPERTS. */
PK_API int pk_route_topk(const float* logits, int64_t T, int64_t E, int64_t K, int route_norm,
                  float route_scale, float* top_scores, int32_t* top_idx, pk_stream_t stream);

/* Backward of pk_route_topk: d_logits[T,E] (f32, fully written) from d_top_scores[T,K]. */
PK_API int pk_route_topk_bwd(const float* logits, const int32_t* top_idx, const float* d_top_scores,
                      int64_t T, int64_t E, int64_t K, int route_norm, float route_scale,
                      float* d_logits, pk_stream_t stream);

/* Backward of pk_gate_logits.
 *   d_x_f32[T,H]   (f32)  = d_logits . w_gate                (written, not accumulated)
 *   d_w_gate[E,H]  (f32) += or = d_logits^T . x              (accumulate != 0 adds)
 *   d_gate_bias[E] (f32) += or = column sums of d_logits     (may be NULL)
 * d_x_f32 or d_w_gate may be NULL to skip that product.  The token reduction of d_w_gate is
 * split over workgroups into `workspace` (pk_gate_bwd_workspace_bytes) and summed in a fixed
 * order; without a workspace it runs unsplit (slower, same result up to fp32 rounding). */
PK_API int64_t pk_gate_bwd_workspace_bytes(int64_t T, int64_t H, int64_t E);
PK_API int pk_gate_logits_bwd(const float* d_logits, const void* x, int x_dtype, const float* w_gate,
                       float* d_x_f32, float* d_w_gate, float* d_gate_bias, int accumulate,
                       int64_t T, int64_t H, int64_t E, void* workspace, int64_t workspace_bytes,
                       pk_stream_t stream);

/* Stable counting sort of the A = T*K flat slots (slot = t*K + k) by expert id.
 *   counts[E]   i32  tokens per expert                          (histogram)
 *   starts[E+1] i32  exclusive prefix sum, starts[E] = A        (qwen3_bmm_experts_patch.py:27)
 *   perm[A]     i32  sorted position -> flat slot  ("token_indices_experts_sorted")
 *   inv_perm[A] i32  flat slot -> sorted position
 *   order[E]    i32  (may be NULL) experts by descending row count, ties by index; a
 *                    scheduling hint for pk_grouped_swiglu_wgrad under skewed routing
 * Within an expert, slots stay in ascending order (= torch.argsort(stable=True)).
 * Replaces the reorderer call (qwen3.py:243-247).  Expert ids must lie in [0,E). */
PK_API int64_t pk_sort_workspace_bytes(int64_t A, int64_t E);
PK_API int pk_sort_by_expert(const int32_t* top_idx, int64_t A, int64_t E, int32_t* counts,
                      int32_t* starts, int32_t* perm, int32_t* inv_perm, int32_t* order,
                      void* workspace, int64_t workspace_bytes, pk_stream_t stream);

/* pk_sort_by_expert for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * inputs, outputs and result as pk_sort_by_expert; the per-chunk histograms live in a fixed array
 * inside the library (PK_SORT_STATIC_WORDS int32 per GPU, held until the process ends) instead of a
 * caller workspace, and nothing is allocated.  Limit: ceil(A / 512) * E <= PK_SORT_STATIC_WORDS,
 * otherwise PK_ERR_WORKSPACE and nothing is launched.  All calls on one GPU share the array: calls
 * that overlap on one GPU (different streams or threads) race; calls on one stream are ordered.
 * The array needs no clearing between calls (every word a call reads it has written before). */
#define PK_SORT_STATIC_WORDS (256 * 1024)
PK_API int pk_sort_by_expert_static(const int32_t* top_idx, int64_t A, int64_t E, int32_t* counts,
                             int32_t* starts, int32_t* perm, int32_t* inv_perm, int32_t* order,
                             pk_stream_t stream);

/* starts[E+1] (i32) from counts[E] given as int32 (counts_is_i64 == 0) or int64.
 * For callers that hand pk_grouped_swiglu_* a `num_tokens_per_expert` tensor
 * (qwen3_bmm_experts_patch.py:24-27). */
PK_API int pk_counts_to_starts(const void* counts, int counts_is_i64, int64_t E, int32_t* starts,
                        pk_stream_t stream);

/* ------------------------------------------------- permute / unpermute+combine */

/* routed[p,:] = x[perm[p] / K, :] for p in [0,A).   (qwen3.py:250) */
PK_API int pk_permute_fwd(const void* x, int dtype, const int32_t* perm, void* routed, int64_t A,
                   int64_t H, int64_t K, pk_stream_t stream);

/* d_x[t,:] = sum_k d_routed[inv_perm[t*K+k], :]  (+ addend_f32[t,:] when not NULL), fp32
 * accumulation in ascending k, rounded once to `dtype`.  Deterministic replacement for the
 * index_put(accumulate) autograd emits for qwen3.py:250. */
PK_API int pk_permute_bwd(const void* d_routed, int dtype, const int32_t* inv_perm,
                   const float* addend_f32, void* d_x, int64_t T, int64_t H, int64_t K,
                   pk_stream_t stream);

/* out[t,:] = sum_k top_scores[t,k] * y_sorted[inv_perm[t*K+k], :], fp32 accumulation in
 * ascending k, rounded once to `dtype`.  Fuses the unpermute scatter and the fp32 bmm
 * combine (qwen3.py:265-283).  residual (optional, [T,H] in `dtype`) is added to the rounded
 * sum, which fuses the block's `x + moe(...)` (qwen3.py:313-314). */
PK_API int pk_combine_fwd(const void* y_sorted, int dtype, const int32_t* inv_perm,
                   const float* top_scores, const void* residual, void* out, int64_t T, int64_t H,
                   int64_t K, pk_stream_t stream);

/* Backward of pk_combine_fwd, per sorted row p (slot = perm[p], t = slot / K):
 *   d_y_sorted[p,:]     = top_scores[slot] * d_out[t,:]          (dtype)
 *   d_top_scores[slot]  = sum_h d_out[t,h] * y_sorted[p,h]       (f32) */
PK_API int pk_combine_bwd(const void* d_out, const void* y_sorted, int dtype, const int32_t* perm,
                   const float* top_scores, void* d_y_sorted, float* d_top_scores, int64_t A,
                   int64_t H, int64_t K, pk_stream_t stream);

/* buf[r, 0:width] = 0 for r in [*first_row, rows); first_row is a DEVICE pointer (for example
 * starts + E, so nothing is read back).  The reference's bmm_experts returns zeros in the rows of
 * its input that no expert owns (`out = x.new_zeros(...)`, qwen3_bmm_experts_patch.py:43), which
 * the grouped kernels never touch. */
PK_API int pk_zero_rows_from(void* buf, int dtype, const int32_t* first_row, int64_t rows, int64_t width,
                      pk_stream_t stream);

/* ------------------------------------------------------ RMSNorm in front of the region
 * The block's ffn_norm (qwen3.py:313-314; torchtitan builds it as RMSNorm(dim, eps=norm_eps),
 * eps 1e-6 in the Qwen3 configs, qwen3.py:28): y = x * rsqrt(mean_h(x^2) + eps) * weight, computed
 * in fp32 and rounded once.  x, weight, y in `dtype`; rstd [T] f32 (optional) is what the
 * backward needs. */
PK_API int pk_rmsnorm_fwd(const void* x, int dtype, const void* weight, float eps, void* y, float* rstd,
                   int64_t T, int64_t H, pk_stream_t stream);
/* Backward.  d_x = rstd * (s - xh * mean_h(s * xh)) with xh = x * rstd, s = d_y * weight;
 * d_x_addend (optional, [T,H] in `dtype`, e.g. the gradient of the residual branch) is added to
 * the rounded result.  d_weight (optional, [H] in `dtype`) = sum_t d_y * xh, summed in a fixed
 * order through `workspace` (pk_rmsnorm_bwd_workspace_bytes); accumulate adds to what is there.
 * Rows of up to 8192 (bf16) / 4096 (f32) elements with 16-byte aligned operands run in one
 * pass with d_weight partials in registers; other shapes take a slower generic pair of kernels. */
PK_API int64_t pk_rmsnorm_bwd_workspace_bytes(int64_t T, int64_t H);
PK_API int pk_rmsnorm_bwd(const void* d_y, const void* x, int dtype, const void* weight, const float* rstd,
                   const void* d_x_addend, void* d_x, void* d_weight, int accumulate, int64_t T,
                   int64_t H, void* workspace, int64_t workspace_bytes, pk_stream_t stream);

/* ------------------------------------------------------ grouped SwiGLU experts
 * Expert e owns rows [starts[e], starts[e+1]) of every [A, *] operand.
 * Weights: w1 (gate) [E,I,H], w3 (up) [E,I,H], w2 (down) [E,H,I]
 * (BmmExperts, qwen3_bmm_experts_patch.py:90-110).
 * Together these replace _run_bmm_experts (qwen3_bmm_experts_patch.py:11-50) and the
 * autograd graph torch builds for it (src/executors.py:257-296).
 * bf16 runs on MFMA tiles when H % 128 == 0, I % 128 == 0 and every operand is 16-byte aligned,
 * and on a shape-unrestricted FMA kernel (still HIP, same results to rounding) otherwise; f32 runs on a
 * tiled FMA kernel with no shape restriction.
 * On the MFMA path an operand whose rows are gathered through a row map (x_rows, d_out) is addressed with
 * 32-bit byte offsets from its first row: the rows that the map can name (ceil(A / row_map_div) of them)
 * must span less than 4 GiB, otherwise the call returns PK_ERR_SHAPE and launches nothing.
 */

/* Forward.  x_rows[A_x,H]: when row_map is NULL, row p of the A operand is x_rows[p]
 * (x already expert-sorted, the reference boundary); otherwise it is
 * x_rows[row_map[p] / row_map_div] (permute fused into the operand load; pass perm and K).
 *   g[A,I] = x . w1[e]^T,  u[A,I] = x . w3[e]^T   (saved for backward)
 *   h[A,I] = silu(g) * u
 *   y[A,H] = h . w2[e]^T */
PK_API int pk_grouped_swiglu_fwd(const void* x_rows, const int32_t* row_map, int64_t row_map_div,
                          const void* w1, const void* w2, const void* w3,
                          const int32_t* starts, void* g, void* u, void* h, void* y,
                          int64_t A, int64_t H, int64_t I, int64_t E, int dtype,
                          pk_stream_t stream);

/* Input gradient (Piper's BWD_I task, src/executors.py:353-411).
 *   d_h = d_y . w2[e];  d_g = d_h * u * silu'(g);  d_u = d_h * silu(g)   -> d_g, d_u [A,I]
 *   d_x_sorted[A,H] = d_g . w1[e] + d_u . w3[e] */
PK_API int pk_grouped_swiglu_dgrad(const void* d_y, const void* w1, const void* w2, const void* w3,
                            const void* g, const void* u, const int32_t* starts, void* d_g,
                            void* d_u, void* d_x_sorted, int64_t A, int64_t H, int64_t I,
                            int64_t E, int dtype, pk_stream_t stream);

/* The two halves of pk_grouped_swiglu_dgrad as separate launches, so that a caller can start
 * the weight gradient (which needs d_g, d_u but not d_x) as soon as the first half is queued. */
PK_API int pk_grouped_swiglu_dgrad_dh(const void* d_y, const void* w2, const void* g, const void* u,
                               const int32_t* starts, void* d_g, void* d_u, int64_t A, int64_t H,
                               int64_t I, int64_t E, int dtype, pk_stream_t stream);
PK_API int pk_grouped_swiglu_dgrad_dx(const void* d_g, const void* d_u, const void* w1, const void* w3,
                               const int32_t* starts, void* d_x_sorted, int64_t A, int64_t H,
                               int64_t I, int64_t E, int dtype, pk_stream_t stream);

/* Input gradient of the experts with the weighted combine folded in: what pk_combine_bwd followed
 * by pk_grouped_swiglu_dgrad_dh computes (the backward of qwen3.py:268-289 up to the SwiGLU
 * pre-activations), without materialising d_y = score * d_out[token] per routed row.
 *   sorted row r belongs to flat slot m = row_map[r] (token m / row_map_div), score scores[m]
 *   a[r]        = d_out[m / row_map_div] . w2[e]^T                     (fp32, never stored)
 *   d_scores[m] = < a[r], silu(g[r]) * u[r] >                          ([T*K] f32, every slot written)
 *   d_g, d_u    = SwiGLU backward of (scores[m] * a[r])                ([A,I], dtype)
 *   hs[r]       = scores[m] * silu(g[r]) * u[r]                        ([A,I], dtype)
 * hs replaces h and d_out replaces d_y in the weight gradient (pk_grouped_swiglu_wgrad_scaled):
 * d_w2[e] = sum_r d_out[token_r]^T . hs[r].  The matrix-core path needs a workspace of
 * pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes (partial score gradients per 64 columns,
 * summed in a fixed order). */
PK_API int64_t pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes(int64_t A, int64_t I);
PK_API int pk_grouped_swiglu_dgrad_dh_scaled(const void* d_out, const int32_t* row_map, int64_t row_map_div,
                                      const float* scores, const void* w2, const void* g,
                                      const void* u, const int32_t* starts, void* d_g, void* d_u,
                                      void* hs, float* d_scores, void* workspace,
                                      int64_t workspace_bytes, int64_t A, int64_t H, int64_t I,
                                      int64_t E, int dtype, pk_stream_t stream);

/* Weight gradient (Piper's BWD_W task, src/executors.py:413-476).
 *   d_w2[e] (+)= d_y[rows_e]^T . h[rows_e]          [H,I]
 *   d_w1[e] (+)= d_g[rows_e]^T . x[rows_e]          [I,H]
 *   d_w3[e] (+)= d_u[rows_e]^T . x[rows_e]          [I,H]
 * x rows are addressed as in the forward (row_map / row_map_div).  expert_order (may be NULL)
 * is the `order` output of pk_sort_by_expert; it only changes which compute units work on
 * which expert, never the result.  accumulate != 0 adds
 * to the existing contents (gradient accumulation over microbatches,
 * src/executors.py:333-343); otherwise every element is overwritten, with zeros for
 * an expert that received no rows. */
PK_API int pk_grouped_swiglu_wgrad(const void* d_y, const void* h, const void* d_g, const void* d_u,
                            const void* x_rows, const int32_t* row_map, int64_t row_map_div,
                            const int32_t* starts, const int32_t* expert_order, void* d_w1,
                            void* d_w2, void* d_w3,
                            int accumulate, int64_t A, int64_t H, int64_t I, int64_t E,
                            int dtype, pk_stream_t stream);

/* The same weight gradients from the outputs of pk_grouped_swiglu_dgrad_dh_scaled: d_out [T,H]
 * is addressed through row_map / row_map_div like x, hs [A,I] takes the place of h. */
PK_API int pk_grouped_swiglu_wgrad_scaled(const void* d_out, const void* hs, const void* d_g, const void* d_u,
                                   const void* x, const int32_t* row_map, int64_t row_map_div,
                                   const int32_t* starts, const int32_t* expert_order, void* d_w1,
                                   void* d_w2, void* d_w3,
                                   int accumulate, int64_t A, int64_t H, int64_t I, int64_t E,
                                   int dtype, pk_stream_t stream);

/* The same pair with one operand of every weight-gradient GEMM K-contiguous (the fused region's
 * path for bf16 with H % 256 == 0 and I % 256 == 0).  pk_grouped_swiglu_dgrad_dh_scaled_t writes
 * d_g, d_u [A,I] as above and, instead of hs, the three transposed copies
 *   d_gT, d_uT, hsT  [ldt / 32][I][32]  (dtype): the routed rows are laid out along a padded row
 *   axis of length ldt on which row r of expert e has index padded_start(e) + r,
 *   padded_start(e) = (starts[e] & ~63) + 64*e; the value of column i at padded index q sits at
 *   [q / 32][i][q % 32] (for every block of 32 padded rows the I columns, each with its 32 row
 *   values contiguous: the producer writes and the weight-gradient kernels read whole kilobytes).
 *   The padded rows from an expert's last row up to the next multiple of 32 (the end of its last
 *   block) are zero, and pk_grouped_swiglu_wgrad_scaled_t relies on that; all other padded rows
 *   between experts are neither written nor read.
 * ldt >= pk_grouped_swiglu_transposed_ld(A, H, I, E, dtype) and a multiple of 64; that query returns
 * 0 when the shape or dtype has no such path (use the entry points above then).
 * d_g and d_u (the row-major outputs) may both be NULL in pk_grouped_swiglu_dgrad_dh_scaled_t: they
 * are then not written, and pk_grouped_swiglu_dgrad_dx_t computes d_x_sorted = d_g . w1[e] + d_u . w3[e]
 * (the second half of the input gradient, as pk_grouped_swiglu_dgrad_dx) from the transposed copies,
 * so that the SwiGLU backward stores each of d_g, d_u once instead of twice.
 * pk_grouped_swiglu_wgrad_scaled_t computes the same d_w1, d_w2, d_w3 as
 * pk_grouped_swiglu_wgrad_scaled from d_out, x (through row_map / row_map_div) and the transposed
 * copies.  Both replace the autograd of qwen3_bmm_experts_patch.py:39-41 like the pair above.
 * Restriction of pk_grouped_swiglu_wgrad_scaled_t: the last 32-row block of an expert multiplies
 * the zeros of the transposed copy with the rows of x / d_out that the row map names behind the
 * expert's last row (rows of the next expert's tokens).  Zero times a finite value is zero; zero
 * times Inf or NaN is NaN.  A non-finite row of x or d_out can therefore reach the weight gradients
 * of the expert in front of the one it was routed to, which pk_grouped_swiglu_wgrad_scaled (rows
 * past an expert's end read as zeros) confines to its own experts. */
PK_API int64_t pk_grouped_swiglu_transposed_ld(int64_t A, int64_t H, int64_t I, int64_t E, int dtype);
PK_API int pk_grouped_swiglu_dgrad_dh_scaled_t(const void* d_out, const int32_t* row_map, int64_t row_map_div,
                                        const float* scores, const void* w2, const void* g,
                                        const void* u, const int32_t* starts, void* d_g, void* d_u,
                                        void* d_gT, void* d_uT, void* hsT, int64_t ldt, float* d_scores,
                                        void* workspace, int64_t workspace_bytes, int64_t A, int64_t H,
                                        int64_t I, int64_t E, int dtype, pk_stream_t stream);
/* HOST, tuning hint: 1 when leaving out the row-major d_g / d_u and running
 * pk_grouped_swiglu_dgrad_dx_t is the faster pair for this shape (long experts), 0 when the
 * row-major pair is (or the shape has no transposed path). */
PK_API int pk_grouped_swiglu_dx_from_transposed_pays(int64_t A, int64_t H, int64_t I, int64_t E, int dtype);
PK_API int pk_grouped_swiglu_dgrad_dx_t(const void* d_gT, const void* d_uT, int64_t ldt, const void* w1, const void* w3,
                                 const int32_t* starts, void* d_x_sorted, int64_t A, int64_t H, int64_t I,
                                 int64_t E, int dtype, pk_stream_t stream);
PK_API int pk_grouped_swiglu_wgrad_scaled_t(const void* d_out, const void* hsT, const void* d_gT, const void* d_uT,
                                     int64_t ldt, const void* x, const int32_t* row_map, int64_t row_map_div,
                                     const int32_t* starts, const int32_t* expert_order, void* d_w1,
                                     void* d_w2, void* d_w3, int accumulate, int64_t A, int64_t H,
                                     int64_t I, int64_t E, int dtype, pk_stream_t stream);

/* Diagnostic, HOST only (touches no device): index of the set of scheduling counters that the
 * persistent grouped GEMMs use for launches with this key.  The library keeps PK_SCHED_SETS sets per
 * device and gives every (stream, capture sequence) pair a set of its own, so that launches that can
 * overlap never share counters: launches on one stream are ordered, and launches recorded into a
 * HIP graph (capture_sequence != 0: 1 + the id hipStreamGetCaptureInfo reports) keep the set of
 * their capture for the life of the graph.  thread_key is 0 except for hipStreamPerThread, which
 * names a different stream in every host thread.  With more than PK_SCHED_SETS keys on a device the
 * sets are shared round-robin, and two launches that share one must not overlap.  No counterpart
 * in the reference. */
#define PK_SCHED_SETS 1024
PK_API int pk_sched_slot_index(int device, uint64_t stream_handle, uint64_t capture_sequence, uint64_t thread_key);

/* ------------------------------------------------------------- ZeRO bucket path */

/* HOST function.  offsets[i] (in elements) of n tensors laid out back to back, each start
 * rounded up to `align_bytes` (a power of two, multiple of elem_size; 1 reproduces the
 * reference's unaligned running sum, src/actor.py:545-554).  Returns the padded total
 * (also a multiple of the alignment), or a negative PK_ERR_*.  numels/offsets: host. */
PK_API int64_t pk_bucket_plan(const int64_t* numels, int64_t n, int64_t elem_size,
                       int64_t align_bytes, int64_t* offsets);

/* Multi-tensor copy/cast/accumulate into a flat bucket, one launch per
 * 120 tensors (more are split over several launches):  flat[offsets[i] : offsets[i]+numels[i]] (+)= cast(src[i]).
 *   srcs: HOST array of n device pointers (NULL entries are skipped: "grad is None");
 *   offsets, numels: HOST arrays (elements);  src_dtype -> dst_dtype any of f32/bf16.
 * Replaces the per-tensor `flat[o:o+n].add_(g.reshape(-1).to(f32))` loop
 * (src/runtime.py:275-282) and the torch.cat flatten (src/actor.py:534). */
PK_API int pk_bucket_pack(const void* const* srcs, const int64_t* offsets, const int64_t* numels,
                   int64_t n, int src_dtype, void* flat, int dst_dtype, int accumulate,
                   pk_stream_t stream);

/* Inverse of pk_bucket_pack without accumulation: dst[i][:] = cast(flat[offsets[i] : ...]).
 * Only needed when parameters are NOT views of the bucket (src/runtime.py:329-339 keeps
 * them as views, in which case unflatten is free). */
PK_API int pk_bucket_unpack(const void* flat, int flat_dtype, void* const* dsts, const int64_t* offsets,
                     const int64_t* numels, int64_t n, int dst_dtype, pk_stream_t stream);

/* flat[0:n] = 0 for an f32 bucket (src/runtime.py:223-229). */
PK_API int pk_bucket_zero(float* flat, int64_t n, pk_stream_t stream);

/* One fused AdamW step over a whole fp32 bucket, torch.optim.AdamW operation order
 * (decoupled decay, lerp first moment, bias-corrected step):
 *   p *= 1 - lr*wd;  m += (g-m)*(1-b1);  v = v*b2 + (1-b2)*g*g;
 *   p -= (lr / (1-b1^step)) * m / (sqrt(v)/sqrt(1-b2^step) + eps)
 * grad is f32 (the bucket) and is scaled by grad_scale first (1.0f = off).
 * shadow (may be NULL): the updated p rounded to `shadow_dtype`, written in the same pass --
 * this is the bucket the bf16 parameter views alias, so "unflatten" costs nothing.
 * zero_grad != 0 also clears grad in the same pass.
 * Replaces `shard_param.grad = ...; shard_optim.step()` (src/runtime.py:470-473) and
 * `bucket.optimizer.step()` (src/executors.py:1024-1025). */
PK_API int pk_adamw_fused(float* master, float* exp_avg, float* exp_avg_sq, float* grad, void* shadow,
                   int shadow_dtype, int64_t n, float lr, float beta1, float beta2, float eps,
                   float weight_decay, int64_t step, float grad_scale, int zero_grad,
                   pk_stream_t stream);

/* pk_bucket_pack of the LAST microbatch's gradients folded into pk_adamw_fused: the gradient of
 * bucket element offsets[i] + j is flat_grad[offsets[i] + j] (fp32, what earlier microbatches packed;
 * flat_grad may be NULL = zero) plus grads[i][j] (grad_dtype; grads[i] may be NULL = the tensor
 * received no gradient in the last microbatch), added in fp32 exactly as pk_bucket_pack with
 * accumulate would have stored it, so master, moments and the bf16 parameter bucket come out
 * bit-identical to pk_bucket_pack(accumulate) followed by pk_adamw_fused, while the fp32 gradient
 * bucket is neither written nor read again (28 bytes per element with one microbatch, against 6 + 30).
 * grads / offsets / numels are HOST arrays of n entries as in pk_bucket_pack; every tensor is
 * stepped, with or without a gradient of its own.  Bucket elements that belong to no tensor
 * (alignment padding) are left as they are; in a bucket built by pk_bucket_plan they hold zeros in
 * every buffer and an AdamW step leaves such elements at zero.  zero_grad != 0 clears the flat_grad
 * elements of the tensors.  shadow (may be NULL) must be bf16.  Replaces the last call of
 * ParamStorage.accumulate_zero_param_grads_to_flat (src/runtime.py:249-282) together with
 * step_zero_shard_optimizers (src/runtime.py:454-484). */
PK_API int pk_adamw_fused_packed(float* master, float* exp_avg, float* exp_avg_sq, float* flat_grad,
                          const void* const* grads, const int64_t* offsets, const int64_t* numels, int64_t n,
                          int grad_dtype, void* shadow, int shadow_dtype, float lr, float beta1, float beta2,
                          float eps, float weight_decay, int64_t step, float grad_scale, int zero_grad,
                          pk_stream_t stream);

/* ------------------------------------------------------------- kernel timing
 * Measurement aid with no counterpart in the reference: when enabled, every kernel launch of
 * the library is bracketed by two hipEventRecord calls on its stream.  pk_timing_collect
 * waits for the recorded events, writes up to max_records (kernel id, milliseconds) pairs in
 * launch order, forgets them and returns how many launches were recorded. */
PK_API int pk_timing_enable(int on);
PK_API int64_t pk_timing_collect(int32_t* ids, float* ms, int64_t max_records);
/* Restrict the bracketing to launches of one kernel id (as returned in `ids`); a negative id times
 * every kernel again.  Two event records per launch cost the stream a few microseconds, which
 * adds up over the ~20 launches of a step: a throughput measurement times only what it needs. */
PK_API int pk_timing_select(int kernel_id);
PK_API const char* pk_timing_kernel_name(int id);

#ifdef __cplusplus
}
#endif
#endif /* PIPER_AMD_H */
