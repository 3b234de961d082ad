/* picomoe -- C ABI of the MI355X (gfx950) kernels for picotron's single-GPU (EP=1) MoE hot path.
 *
 * Conventions (every entry point):
 *   - plain device pointers, explicit sizes, row-major contiguous tensors unless a stride is given;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); work is only enqueued,
 *     nothing synchronises, allocates or keeps a pointer past the call;
 *   - returns 0 on success, PICOMOE_ERR_ARG for a shape / dtype / alignment the kernels do not
 *     accept, PICOMOE_ERR_TOO_LARGE for one whose tile count does not fit the kernels' 32-bit tile numbering
 *     (expert FFN: about (n_rows / 64 + experts) x max(hidden, 2 inter) / 64 >= 2^31), or PICOMOE_ERR_HIP_BASE +
 *     hipError_t when the launch itself failed;
 *   - `dtype` is PICOMOE_F32 or PICOMOE_BF16 (the dtype of the token features / weights).
 *
 * Each declaration cites the reference code it replaces (paths inside the picotron checkout,
 * `EP/` = picotron/expert_parallel/).
 */
#ifndef PICOMOE_H
#define PICOMOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PICOMOE_OK 0
#define PICOMOE_ERR_ARG 1
#define PICOMOE_ERR_TOO_LARGE 2
#define PICOMOE_ERR_HIP_BASE 1000

#define PICOMOE_F32 0
#define PICOMOE_BF16 1

#define PICOMOE_ABI_VERSION 6

/* ABI version of the loaded library (compare with PICOMOE_ABI_VERSION). */
int picomoe_abi_version(void);

/* Static, human-readable text for a return code of any entry point. */
const char* picomoe_error_string(int code);

/* ---- FP8 E4M3 dispatch quantise / dequantise ---------------------------------------------------
 * Replaces EP/ep_communications.py:63-68 (_per_token_quant_fp8): per row, amax = max|x| floored at
 * 1e-4 and scale = amax/448, both rounded to x's dtype; q = e4m3fn_rne(clamp(float(x)/scale, +-448)).
 * x [n_rows, hidden] (dtype), q [n_rows, hidden] bytes, scale [n_rows] fp32. */
int picomoe_fp8_quant(const void* x, int dtype, int64_t n_rows, int64_t hidden, uint8_t* q, float* scale,
                      void* stream);

/* Replaces EP/ep_communications.py:100: out = dtype(q) * dtype(scale), rounded to dtype. */
int picomoe_fp8_dequant(const uint8_t* q, const float* scale, int64_t n_rows, int64_t hidden, void* out, int dtype,
                        void* stream);

/* The FP8 dispatch of one rank in one pass.  Replaces, together, the quantise and the dequantise around the exchange
 * (EP/ep_communications.py:89-100; with one rank there is no exchange) and the two gathers that expand the tokens to
 * routed rows and sort them by expert (EP/expert_parallel.py:216-217, :340): every token row is read once and
 * x_sorted[inv_order[t * top_k + j]] = dequantise(quantise(tokens[t])) for j < top_k, with the arithmetic of
 * picomoe_fp8_quant and picomoe_fp8_dequant (same codes, same scales, same rounding).  inv_order [n_tokens * top_k] is
 * the plan's (sorted position of each routed row; negative or >= n_out = not kept: skipped); x_sorted [n_out, hidden]
 * in dtype.  Optional, both or neither of a pair: q_sorted [n_out, hidden] codes + scale_sorted [n_out] fp32 in the same
 * order (the operands of picomoe_ffn_gate_up_fp8); q [n_tokens, hidden] + scale [n_tokens] in token order (the wire
 * format of :63-68).  top_k <= 16. */
int picomoe_dispatch_fp8(const void* tokens, int dtype, int64_t n_tokens, int64_t hidden, const int32_t* inv_order, int top_k,
                         int64_t n_out, void* x_sorted, uint8_t* q_sorted, float* scale_sorted, uint8_t* q, float* scale,
                         void* stream);

/* ---- Router --------------------------------------------------------------------------------------
 * Replaces EP/expert_parallel.py:175-184 (MoELayer._route after the gate Linear): probs =
 * softmax_fp32(logits [n_tokens, num_experts]); picks = top_k of (probs + expert_bias) ordered by
 * descending score, lower expert id first on equal scores; weights = probs at the picks, divided by
 * their sum when norm_topk != 0 and top_k > 1, cast to dtype.  num_experts <= 1024, top_k <= 16.
 * Optional outputs (NULL to skip): probs [n_tokens, num_experts] fp32; counts [num_experts] int32
 * (picks per expert are ADDED with integer atomics: zero it first); colsum_partial
 * [picomoe_route_partials(...), num_experts] fp32 partial column sums of probs (EP/expert_parallel.py:196-203). */
int picomoe_route_partials(int64_t n_tokens, int num_experts);
int picomoe_route_fwd(const void* logits, int dtype, int64_t n_tokens, int num_experts, int top_k,
                      const float* expert_bias, int norm_topk, int64_t* topk_idx, void* topk_w, float* probs,
                      int* counts, float* colsum_partial, void* stream);

/* Backward of the above plus the aux-loss term (autograd of EP/expert_parallel.py:175-184 and :202-204):
 * d_logits = softmax_bwd(d_probs) with d_probs gathering d_topk_w (through the renormalisation) and
 * d_aux[0] * aux_coef * f_e / n_tokens, f_e = counts[e] * E / (top_k * n_tokens).  d_topk_w, d_aux, counts
 * may be NULL. */
int picomoe_route_bwd(const float* probs, const int64_t* topk_idx, const void* d_topk_w, int dtype, int64_t n_tokens,
                      int num_experts, int top_k, int norm_topk, const float* d_aux, const int* counts, float aux_coef,
                      void* d_logits, void* stream);

/* Replaces EP/expert_parallel.py:199-212 (MoELayer._balance): aux_out[0] = aux_coef * sum_e f_e * mean_t probs[t,e]
 * (skipped when aux_out is NULL) and expert_bias[e] += bias_rate * sign(mean(counts) - counts[e]) in place
 * (skipped when expert_bias is NULL or bias_rate == 0). */
int picomoe_balance(const int* counts, const float* colsum_partial, int n_partials, int64_t n_tokens, int num_experts,
                    int top_k, float aux_coef, float bias_rate, float* aux_out, float* expert_bias, void* stream);

/* Backward of the router's gate Linear, EP/expert_parallel.py:65 and :174 (`self.gate = nn.Linear(hidden, num_experts,
 * bias=False)`, `router_logits = self.gate(tokens)`: autograd's d_tokens = d_logits @ gate.weight and d_weight =
 * d_logits.T @ tokens), together with autograd's sum of the tokens' gradient paths (through the router and through the
 * experts), in one read of each operand: d_x[t] = addend[t] + d_logits[t] @ gate_w and, when d_w is given,
 * d_w[e] = sum_t d_logits[t, e] * tokens[t] (fp32 sums in a fixed order, rounded once).  d_logits [n_tokens, num_experts],
 * gate_w and d_w [num_experts, hidden], addend (NULL = zeros), tokens and d_x [n_tokens, hidden], all in dtype; the product
 * d_logits @ gate_w is rounded to dtype before the sum with the addend, as a GEMM followed by an add rounds.
 * Either output may be NULL.  num_experts <= 16 for d_x alone (tokens, d_w, workspace NULL) and <= 8 with d_w, which needs `workspace` of
 * picomoe_gate_bwd_workspace_bytes(...) bytes (0 = this gate has no fused weight gradient; -1 = bad arguments); hidden a
 * multiple of 16 bytes and at most 2^22, pointers 16-byte aligned: PICOMOE_ERR_ARG otherwise (a caller keeps the library GEMMs for wider
 * routers). */
int64_t picomoe_gate_bwd_workspace_bytes(int dtype, int64_t n_tokens, int num_experts, int64_t hidden);
int picomoe_gate_bwd(const void* d_logits, const void* gate_w, const void* addend, const void* tokens, int dtype,
                     int64_t n_tokens, int num_experts, int64_t hidden, void* d_x, void* d_w, void* workspace,
                     int64_t workspace_bytes, void* stream);

/* ---- Permute / unpermute (the EP=1 form of dispatch / combine) ---------------------------------------
 * Replaces EP/expert_parallel.py:30-35 and :335-339 (stable argsort by expert, its inverse, bincount) and
 * EP/capacity_moe.py:44-57, :109-110 (_slot_assignment and the drop-mode keep mask).
 * expert_idx [n_rows] int64.  Rows are ranked inside their expert in ascending row order (within[r]); with
 * capacity > 0 only rows whose rank lies in [round_index*capacity, (round_index+1)*capacity) are kept (round 0
 * alone is the drop mode; successive rounds are the static-memory dropless loop, EP/capacity_moe.py:108-110).
 * Kept rows are laid out expert after expert:
 * inv_order[r] = sorted position of row r, or -1 when dropped; order[pos] = row at position pos (-1 past the
 * last kept row); counts [E] int64 = rows per expert before dropping; kept_counts [E] int64 = rows kept this
 * round; within [n_rows] int32 optional.  workspace: picomoe_permute_workspace_bytes() bytes. */
int64_t picomoe_permute_workspace_bytes(int64_t n_rows, int num_experts);
int picomoe_permute_plan(const int64_t* expert_idx, int64_t n_rows, int num_experts, int64_t capacity,
                         int64_t round_index, int32_t* order, int32_t* inv_order, int64_t* counts, int64_t* kept_counts, int32_t* within, void* workspace,
                         void* stream);

/* The same plan for callers that cannot allocate or pass a workspace (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The block histograms and segment starts
 * live in a fixed array of PICOMOE_PLAN_STATIC_BYTES (1 MiB) of device memory inside the library, one per GPU, held
 * until the process ends; the call allocates and frees nothing.  Inputs whose
 * picomoe_permute_workspace_bytes(n_rows, num_experts) exceeds that -- (ceil(n_rows / 1024) + 1) * num_experts * 4
 * bytes, e.g. more than 261120 rows at 1024 experts or 33 million rows at 8 -- are refused with PICOMOE_ERR_TOO_LARGE.
 * Every call on a GPU uses that GPU's one array: calls that overlap in time on one GPU (different streams or threads)
 * race; calls on one stream are ordered.  Nothing in the array has to be cleared between calls (each call writes every
 * entry before reading it).  Results are identical to picomoe_permute_plan's.
 * picomoe_permute_plan_static_init() is its set-up, also without a counterpart in the reference: it looks up the
 * address of the current device's array (one runtime symbol query, no allocation, no launch) and keeps it.  Call it
 * once per device, with that device current, before the first picomoe_permute_plan_static of a stream capture;
 * without it the first plan call on a device does the lookup itself, which an eager call may and a captured one should
 * not.  Calling it again is free. */
#define PICOMOE_PLAN_STATIC_BYTES (1 << 20)
int64_t picomoe_permute_plan_static_max_bytes(void);
int picomoe_permute_plan_static_init(void);
int picomoe_permute_plan_static(const int64_t* expert_idx, int64_t n_rows, int num_experts, int64_t capacity,
                                int64_t round_index, int32_t* order, int32_t* inv_order, int64_t* counts, int64_t* kept_counts,
                                int32_t* within, void* stream);

/* Replaces the gathers tokens[token_idx] (EP/expert_parallel.py:216-217) and x[order] (:340) in one pass:
 * out[i] = src[row_map[i] / div] for i < n_out (row_map NULL = identity, negative entries are skipped). */
int picomoe_gather_rows(const void* src, const int32_t* row_map, int div, int64_t n_out, int64_t hidden, int dtype,
                        void* out, void* stream);

/* Replaces y_sorted[inv_order] + _combine_topk (EP/expert_parallel.py:341, :219-224) and the weighted index_add
 * of EP/capacity_moe.py:158-160: out[t] = sum_j weights[t,j] * y[inv_order[t*top_k+j]] over the rows that were
 * kept; products rounded to dtype, fp32 sum rounded once.  weights NULL = plain sum (the gradient of the
 * expand/permute gather). */
int picomoe_combine_fwd(const void* y, const int32_t* inv_order, const void* weights, int64_t n_tokens, int top_k,
                        int64_t hidden, int dtype, void* out, void* stream);

/* Backward of the above: d_y[inv_order[t*k+j]] = weights[t,j] * d_out[t]; d_weights[t,j] = <d_out[t], y[...]>
 * (0 for dropped rows).  Rows of d_y that no kept row maps to are left untouched. */
int picomoe_combine_bwd(const void* d_out, const void* y, const int32_t* inv_order, const void* weights, int64_t n_tokens,
                        int top_k, int64_t hidden, int dtype, void* d_y, void* d_weights, void* stream);

/* ---- Expert FFN: grouped SwiGLU GEMMs -----------------------------------------------------------------
 * Rows are grouped by expert, expert e owning the next counts[e] rows (counts [E] int64 on the device, read by
 * the kernels: no host copy).  n_rows = rows allocated in the row-major activations (>= sum of counts).
 * gate_w / up_w [E, inter, hidden], down_w [E, hidden, inter], all contiguous, in dtype.  fp32 accumulation.
 *
 * picomoe_ffn_gate_up replaces the gate||up grouped GEMM + silu_and_mul (EP/megakernel.py:302-304;
 * model.py:258): act [n_rows, inter] = silu(x . gate_w[e]^T) * (x . up_w[e]^T); inter13 [n_rows, 2*inter]
 * (optional) receives [g | u] for the backward pass. */
int picomoe_ffn_gate_up(const void* x, const int64_t* counts, int num_experts, int64_t n_rows, int64_t hidden,
                        int64_t inter, const void* gate_w, const void* up_w, int dtype, void* act, void* inter13,
                        void* workspace, int64_t workspace_bytes, void* stream);
/* The same gate||up GEMM + silu_and_mul on FP8 MFMA, fed by the FP8 dispatch: xq [n_rows, hidden] E4M3 codes with one
 * fp32 scale per row (what _per_token_quant_fp8 ships, EP/ep_communications.py:63-68, instead of the dequantised rows
 * of :100), gate_wq / up_wq [E, inter, hidden] codes with one fp32 scale per output row ([E * inter], quantised the
 * same way, e.g. with picomoe_fp8_quant on the [E * inter, hidden] view).  g = (xq . gate_wq[e]^T) * x_scale * scale,
 * fp32 accumulation; act / inter13 in bf16.  hidden % 256 == 0 and inter % 128 == 0, else PICOMOE_ERR_ARG.  The
 * reference has no FP8 GEMM: results are compared with the bf16 GEMM on the dequantised rows at rtol 5e-2. */
int picomoe_ffn_gate_up_fp8(const void* xq, const float* x_scale, const int64_t* counts, int num_experts, int64_t n_rows,
                            int64_t hidden, int64_t inter, const void* gate_wq, const void* up_wq, const float* gate_scale,
                            const float* up_scale, void* act, void* inter13, void* stream);
/* Replaces the down grouped GEMM with its optional row-weight epilogue (EP/megakernel.py:305, :95-96). */
int picomoe_ffn_down(const void* act, const int64_t* counts, int num_experts, int64_t n_rows, int64_t hidden, int64_t inter,
                     const void* down_w, const void* row_weight, int dtype, void* y, void* workspace, int64_t workspace_bytes,
                     void* stream);
/* The same down GEMM on FP8 MFMA: actq [n_rows, inter] E4M3 codes of the SwiGLU output with one fp32 scale per row
 * (picomoe_fp8_quant of act), down_wq [E, hidden, inter] codes with one fp32 scale per output row ([E * hidden]);
 * y [n_rows, hidden] bf16 = (actq . down_wq[e]^T) * act_scale * down_scale, fp32 accumulation, times the optional bf16
 * row_weight as in picomoe_ffn_down (EP/megakernel.py:305, :95-96).  hidden % 256 == 0 and inter % 128 == 0, else
 * PICOMOE_ERR_ARG.  No counterpart in the reference (it has no FP8 GEMM): compared with the bf16 GEMM at rtol 5e-2. */
int picomoe_ffn_down_fp8(const void* actq, const float* act_scale, const int64_t* counts, int num_experts, int64_t n_rows,
                         int64_t hidden, int64_t inter, const void* down_wq, const float* down_scale, const void* row_weight,
                         void* y, void* stream);
/* Replaces da = dy @ down_w[e] and _silu_and_mul_bwd (EP/megakernel.py:344-345, :187-197) in one kernel:
 * d_inter13 [n_rows, 2*inter] = [dg | du]; act_out (optional) = silu(g) * u rebuilt from inter13. */
int picomoe_ffn_dgrad_act(const void* dy, const int64_t* counts, int num_experts, int64_t n_rows, int64_t hidden,
                          int64_t inter, const void* down_w, const void* inter13, int dtype, void* d_inter13, void* act_out,
                          void* workspace, int64_t workspace_bytes, void* stream);
/* Replaces dx = d_inter13 @ w13[e] (EP/megakernel.py:346) without the concatenated w13. */
int picomoe_ffn_dgrad_x(const void* d_inter13, const int64_t* counts, int num_experts, int64_t n_rows, int64_t hidden,
                        int64_t inter, const void* gate_w, const void* up_w, int dtype, void* dx, void* workspace,
                        int64_t workspace_bytes, void* stream);
/* Device scratch the four row-grouped calls above (gate_up, down, dgrad_act, dgrad_x) can use (the library allocates nothing
 * itself, the boundary rule of the reference's kernels being torch-owned memory: EP/megakernel.py:294-306 allocates every buffer
 * with torch.empty).  With `workspace` of at least this many bytes the bf16 kernels cut the tiles of the last, partly filled
 * round of blocks into 2 or 4 ranges of K that run side by side, park the fp32 partial tiles there and add them up in a second
 * small kernel, which also applies the epilogue (SwiGLU, SwiGLU backward, row weight); with NULL (or fewer bytes) every tile is
 * computed whole.  Results agree to the rounding of the fp32 partial sums.  Calls that overlap in time on different streams need
 * a workspace each; calls of one stream can share one. */
int64_t picomoe_ffn_workspace_bytes(void);
/* Which kernels the five expert-FFN entry points run for a dtype and layer widths (a query, no launch):
 * PICOMOE_FFN_BF16_MFMA -- bf16, hidden and inter multiples of 64 and >= 128: 256 x 256 tiles on v_mfma_f32_16x16x32_bf16;
 * PICOMOE_FFN_F32_MFMA  -- fp32, hidden and inter multiples of 4 and >= 32: 128 x 128 tiles on v_mfma_f32_32x32x2_f32
 *                          (full fp32 products: the reference runs fp32 inputs on its matrix units too, EP/megakernel.py:162);
 * PICOMOE_FFN_GENERIC   -- everything else: 64 x 64 tiles of scalar fp32 FMAs, correct for any shape and far slower.
 * picomoe_ffn_wgrad picks by its own p_dim / q_dim / strides in the same way. */
#define PICOMOE_FFN_GENERIC 0
#define PICOMOE_FFN_BF16_MFMA 1
#define PICOMOE_FFN_F32_MFMA 2
int picomoe_ffn_kernel_family(int dtype, int64_t hidden, int64_t inter);
/* Replaces _grouped_wgrad (EP/megakernel.py:209-291): out [E, p_dim, q_dim] with out[e] = lhs_e^T @ rhs_e over the
 * rows of expert e; lhs [n_rows, >=p_dim] with row stride ld_lhs, rhs likewise (so the two halves of d_inter13
 * are addressed in place).  Empty experts get zeros. */
int picomoe_ffn_wgrad(const void* lhs, int64_t ld_lhs, const void* rhs, int64_t ld_rhs, const int64_t* counts,
                      int num_experts, int64_t n_rows, int64_t p_dim, int64_t q_dim, int dtype, void* out, void* stream);

/* ---- Diagnostics -----------------------------------------------------------------------------------------
 * No counterpart in the reference and not part of the MoE path: a loop of nothing but MFMAs, to measure what the matrix
 * pipes sustain under this GPU's power limit -- the ceiling the grouped-GEMM kernels are compared with next to the
 * datasheet peak.  n_blocks blocks of 8 wavefronts (one block per CU fills the chip with two wavefronts per SIMD), each
 * wavefront multiplying the same operand fragments into 32 independent accumulator blocks `iters` times.  The fragments
 * are read once from `operands` (operand_bytes >= 16, 16-byte aligned; indices wrap), so the caller chooses the bit
 * patterns: random values draw more power than zeros.  `sink` may be NULL.  burst_iters > 0 (a divisor of iters) makes
 * every block pause for idle_us (<= 1000) after each burst_iters iterations, all its wavefronts together: the rate inside
 * the bursts against the rate of the uninterrupted loop says how much of a pause comes back as a higher clock, i.e. what
 * a phase without MFMAs costs a kernel whose clock the power limit sets.  burst_iters == 0: no pauses.
 * picomoe_diag_mfma_loop_flop returns the FLOP one such launch performs (-1 for an unknown shape). */
#define PICOMOE_DIAG_BF16_16X16X32 0 /* v_mfma_f32_16x16x32_bf16 */
#define PICOMOE_DIAG_BF16_32X32X16 1 /* v_mfma_f32_32x32x16_bf16 */
#define PICOMOE_DIAG_FP8_16X16X128 2 /* v_mfma_f32_16x16x128_f8f6f4 on E4M3 codes */
int64_t picomoe_diag_mfma_loop_flop(int shape, int64_t iters, int n_blocks);
int picomoe_diag_mfma_loop(const void* operands, int64_t operand_bytes, int shape, int64_t iters, int64_t burst_iters,
                           int64_t idle_us, int n_blocks, float* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PICOMOE_H */
