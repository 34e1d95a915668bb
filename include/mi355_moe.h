/*
 * mi355_moe.h -- C ABI of the MI355X (gfx950) MoE-block kernels.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the null stream) and returns 0 on success or a
 * negative MI355_E* code; mi355_moe_last_error() then describes the failure
 * (thread-local text).  No entry point synchronises the host with the device and
 * none allocates device memory: outputs and workspaces are caller-owned.
 * All kernels of one call run on the given stream in program order.
 *
 * The reference (TorchLLMTuner) has no FFI: its MoE block is a composition of
 * PyTorch ops.  Each declaration therefore cites the reference lines whose
 * arithmetic it replaces (paths relative to the reference checkout).
 *
 * Shape legend: T tokens, D model dim, E experts, K experts per token, N = T*K
 * assignment slots (flat index t*K + k), F expert hidden dim, R rows of the
 * expert-major buffer, El = number of local experts (hi - lo).
 */
#ifndef MI355_MOE_H
#define MI355_MOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_MOE_ABI_VERSION 3

/* element types of activation / weight buffers.
 * MI355_F64 is accepted where the reference's fp64 runs pass through this boundary
 * (tests/unit_tests/cpu/test_expert_compile_segments.py:13-40 runs the experts in fp64):
 * the row movers, the combine, the grouped experts and grouped linear maps compute in fp64
 * throughout; the router gate takes fp64 tokens and weights and converts them to fp32 on
 * the way in, as RouterGateLinearFunction does (linear.py:123-125), and writes its
 * gradients back in the operands' types.  Every other entry point takes fp32 or bf16
 * and returns MI355_EINVAL for fp64. */
#define MI355_F32 0
#define MI355_BF16 1
#define MI355_F64 2

/* score functions: llmtuner/models/common/moe/routing.py:270-277 */
#define MI355_SCORE_SIGMOID 0
#define MI355_SCORE_SOFTMAX 1
#define MI355_SCORE_SQRTSOFTPLUS 2

/* selection modes: routing.py:291-303 */
#define MI355_SELECT_TOPK 0     /* biased top-k, optionally group-limited   */
#define MI355_SELECT_FIXED 1    /* fixed_router: (t + k) % E, weights 1/K   */
#define MI355_SELECT_BALANCED 2 /* _debug_force_load_balance: (t*K + k) % E */

/* error codes */
#define MI355_OK 0
#define MI355_EINVAL (-1)  /* bad argument (shape, dtype, alignment, null)  */
#define MI355_ELAUNCH (-2) /* a HIP launch or runtime call failed           */
#define MI355_EUNSUP (-3)  /* valid request this build does not implement   */

int mi355_moe_abi_version(void);
const char* mi355_moe_last_error(void);

/* ------------------------------------------------------------------ router */

/*
 * logits_TE[t][e] = sum_d x[t][d] * w[e][d]  (+ logit_bias[e]), fp32 output and
 * fp32 accumulation whatever the storage types.
 * Replaces RouterGateLinearFunction.forward and RouterGateLinear.forward,
 * llmtuner/models/common/linear.py:107-131,179-183.
 * x: (T,D) x_dtype row-major; w: (E,D) w_dtype; logit_bias: (E) fp32 or NULL.
 * workspace: mi355_router_gate_fwd_workspace_bytes(T,D,E) bytes (for the same T, D, E)
 * or NULL.  With a workspace, bf16 x, fp32 w and D, E multiples of 64, each fp32 weight
 * is written as three bf16 pieces (24 mantissa bits) and the product runs as three bf16
 * MFMAs with fp32 accumulation (from 1024 tokens on in 128-token tiles with the
 * contraction split over workgroups, partial sums added in a fixed order); otherwise the
 * strided fp32-MFMA kernel is used.
 */
int64_t mi355_router_gate_fwd_workspace_bytes(int64_t T, int64_t D, int64_t E);
int mi355_router_gate_fwd(const void* x, int x_dtype, const void* w, int w_dtype,
                          const float* logit_bias, float* logits_TE, void* workspace,
                          int64_t T, int64_t D, int64_t E, void* stream);

/*
 * dx[t][d] = sum_e dlogits[t][e] * w[e][d]   (written in x_dtype; NULL = skip)
 * dw[e][d] = sum_t dlogits[t][e] * x[t][d]   (written in w_dtype; NULL = skip)
 * both accumulated in fp32.  Replaces RouterGateLinearFunction.backward,
 * linear.py:133-151.  workspace: mi355_router_gate_bwd_workspace_bytes() bytes
 * (bf16 weight pieces, split-K partial sums for dw); NULL selects the strided
 * fp32-MFMA kernels and is only valid when dw is NULL or T is small.
 */
int64_t mi355_router_gate_bwd_workspace_bytes(int64_t T, int64_t D, int64_t E);
int mi355_router_gate_bwd(const float* dlogits_TE, const void* x, int x_dtype,
                          const void* w, int w_dtype, void* dx, void* dw,
                          void* workspace, int64_t T, int64_t D, int64_t E,
                          void* stream);

/*
 * Scores, expert choice, gather, norm and scale in one pass over the logits.
 * Replaces TokenChoiceTopKRouter.forward after the gate, routing.py:270-324:
 * score function (:270-277), biased top-k (:168-192) or group-limited top-k
 * (:194-239; group score = sum of the group's top-2, top num_limited groups kept,
 * the rest masked to -inf), unbiased gather, route_norm with +1e-20, route_scale
 * (:311-315), and the fixed / balanced debug routings (:291-309, :146-166).
 * Selection order is "higher choice score first, ties to the lower expert id";
 * ids are emitted in that order.  Without a bias and without groups the choice is made
 * on the logits (every score function is non-decreasing in its logit), so it does not
 * depend on the last ulp of exp(): for equal logits in, the ids equal those of any
 * correct top-k over the scores wherever the scores themselves do not tie.
 * expert_bias: (E) fp32 or NULL.  num_groups = 0 disables grouping.
 * scores_TE: optional (T,E) fp32 output of the score function (NULL = skip).
 * routing_map_TE: optional (T,E) bytes, 1 where the token chose the expert (the bool
 * routing map of routing.py:320-324; NULL = skip).
 */
int mi355_router_select_fwd(const float* logits_TE, const float* expert_bias,
                            float* weights_TK, int64_t* ids_TK, float* scores_TE,
                            uint8_t* routing_map_TE, int64_t T, int64_t E, int64_t K,
                            int score_func, int route_norm, float route_scale,
                            int num_groups, int num_limited, int select_mode,
                            void* stream);

/*
 * The same selection for a quantile-balanced router in training
 * (QuantileBalancedTopKRouter._select_experts, routing.py:399-430: one biased
 * top-(K+1), sorted): plain top-k over scores + expert_bias, and additionally
 * cutoff_T[t] = the (K+1)-th largest biased score of token t, the value the required
 * biases of mi355_quantile_observe are measured against.  Needs K < E.
 */
int mi355_router_select_cutoff_fwd(const float* logits_TE, const float* expert_bias,
                                   float* weights_TK, int64_t* ids_TK, float* scores_TE,
                                   float* cutoff_T, int64_t T, int64_t E, int64_t K,
                                   int score_func, int route_norm, float route_scale,
                                   void* stream);

/*
 * Required-bias histogram of quantile-balanced routing, _observe_quantile_histogram,
 * routing.py:433-461: for every token t that is not padding and every expert e,
 *   bin = clamp(floor((cutoff_T[t] - scores_TE[t][e] - (min(bias) - 1)) / width), 0, B-1),
 *   width = (max(bias) - min(bias) + 2) / B,   histogram_EB[e][bin] += 1.
 * histogram_EB: (E,B) int64, accumulated into (the caller zeroes it once per
 * optimizer step).  padding_mask_T: (T) bytes, non-zero = padding, or NULL.
 * The fp32 operations are the reference's in its order; integer atomics make the
 * result independent of scheduling.
 */
int mi355_quantile_observe(const float* scores_TE, const float* cutoff_T,
                           const float* expert_bias_E, const uint8_t* padding_mask_T,
                           int64_t* histogram_EB, int64_t T, int64_t E, int64_t B,
                           void* stream);

/*
 * Next mean-centred expert bias from the histogram,
 * QuantileBalancer.estimate_expert_bias, routing.py:557-610: per expert the K/E
 * quantile of its required-bias distribution (target rank ceil(count*K/E), linear
 * interpolation inside the crossing bin with an integral numerator), experts without
 * observations held at their current position, result minus its mean, times the bin
 * width.  An all-zero histogram returns expert_bias_E unchanged, bit for bit.
 * next_bias_E may not alias expert_bias_E.  workspace: 8*E bytes.
 */
int mi355_quantile_estimate(const int64_t* histogram_EB, const float* expert_bias_E,
                            float* next_bias_E, void* workspace, int64_t E, int64_t K,
                            int64_t B, void* stream);

/*
 * dlogits_TE from dweights_TK (and, optionally, a dense gradient dscores_TE on the
 * full score map, e.g. from an auxiliary loss; NULL = none): the backward of the
 * gather / norm / scale / score chain that autograd derives for routing.py:270-315.
 * For MI355_SELECT_FIXED the weights are constants and only dscores_TE flows.
 */
int mi355_router_select_bwd(const float* logits_TE, const int64_t* ids_TK,
                            const float* dweights_TK, const float* dscores_TE,
                            float* dlogits_TE, int64_t T, int64_t E, int64_t K,
                            int score_func, int route_norm, float route_scale,
                            int select_mode, void* stream);

/*
 * Per-forward load-balance loss on the dense score map and the routing map:
 *   f_e = E * counts_e / max(sum counts, 1e-12),  counts_e = sum_t map[t][e]
 *   p_e = sum_t s[t][e] / max(sum_e s[t][e], 1e-12)   (padding tokens contribute 0)
 *   loss = sum_e f_e * p_e            (the value is T * L_bal; the caller's 1/tokens
 *                                      normalisation makes it coeff * L_bal)
 * Replaces MicrobatchWiseLoadBalanceLoss.forward up to inject(),
 * llmtuner/models/common/moe/auxiliary_loss.py:147-162 (single process: no token-axis
 * reduction).  routing_map_TE: (T,E) bytes, non-zero = chosen; padding_mask_T: (T) bytes
 * or NULL; loss: 1 float; f_E: (E) floats kept for the backward; workspace:
 * mi355_balance_loss_workspace_bytes().  E <= 1024.
 * The backward writes d loss / d scores * grad_loss[0] into dscores_TE (the map carries no
 * gradient): (f_j - sum_e f_e s'_e) / S_t, zero rows for padding tokens.
 */
int64_t mi355_balance_loss_workspace_bytes(int64_t T, int64_t E);
int mi355_balance_loss_fwd(const float* scores_TE, const uint8_t* routing_map_TE,
                           const uint8_t* padding_mask_T, float* loss, float* f_E,
                           void* workspace, int64_t T, int64_t E, void* stream);
int mi355_balance_loss_bwd(const float* scores_TE, const float* f_E,
                           const uint8_t* padding_mask_T, const float* grad_loss,
                           float* dscores_TE, int64_t T, int64_t E, void* stream);

/* ------------------------------------------------------- permutation plan */

/*
 * Expert-major layout of the N = T*K assignment slots, stable in the flat slot
 * index (bit-identical to argsort(ids.flatten(), stable=True)).
 * Replaces LocalTokenDispatcher._local_reorder's index work,
 * llmtuner/parallel/expert_parallel/token_dispatch.py:180-186, the routing-map
 * count layer.py:278, GroupedExperts' cumsum experts.py:204, and -- with
 * align > 1 -- the padded layout of TorchAOTokenDispatcher._permute,
 * torchao_dispatch.py:143-175 (contract:
 * tests/unit_tests/cpu/models/test_moe_token_dispatch.py:154-179): each local
 * expert's segment is padded up to a multiple of `align` rows; an empty expert gets
 * no padding.
 *
 * Only experts in [local_lo, local_hi) receive rows (one rank's share of an
 * expert-parallel layout, token_dispatch.py:367-371); other slots get row -1 but
 * are still counted.
 *
 * Outputs (all caller-allocated, int32):
 *   counts_E      (E)     slots per expert, over all experts
 *   seg_offsets   (El+1)  first row of each local segment; [El] = total rows used
 *   seg_counts    (2*El)  [0,El): real (unpadded) rows per local segment;
 *                 [El,2*El): the local expert indices ordered by descending row
 *                 count, ties to the lower index -- the order in which the
 *                 weight-gradient kernels below walk the experts, so that the
 *                 longest contractions start first under skewed routing
 *   row_of_slot   (N)     row of slot t*K+k, or -1 when not local
 *   slot_of_row   (row_capacity) slot held by each row, -1 for padding / unused
 *   token_of_row  (row_capacity) token held by each row (slot / K), -1 for padding /
 *                 unused; optional (NULL = skip): the gather index of the fused expert
 *                 kernels below
 *   tile_expert, tile_row0 (tile_capacity each) and num_tiles (1): the list of
 *       row tiles covering the real rows of every segment (local expert index and
 *       first row of each tile).  A segment of c rows has ceil(c / tile_m) tiles, all
 *       of the same height ceil(c / that number) rounded up to 16 rows (at most
 *       tile_m; the last one ends with the segment): equal tiles of an expert run in
 *       step and share its weights in L2, a short rest tile would not
 * row_capacity  >= N + El*(align-1) is always enough;
 * tile_capacity >= N/tile_m + El + 1 is always enough.
 * workspace: mi355_permute_plan_workspace_bytes(T,K,E) bytes.
 * A slot whose id lies outside [0,E) is not counted and gets row -1 (its token simply
 * misses that expert); nothing is read or written out of bounds.  E <= 2048.
 */
int64_t mi355_permute_plan_workspace_bytes(int64_t T, int64_t K, int64_t E);
int mi355_permute_plan(const int64_t* ids_TK, int64_t T, int64_t K, int64_t E,
                       int64_t local_lo, int64_t local_hi, int64_t align,
                       int64_t tile_m, int32_t* counts_E, int32_t* seg_offsets,
                       int32_t* seg_counts, int32_t* row_of_slot,
                       int32_t* slot_of_row, int32_t* token_of_row, int64_t row_capacity,
                       int32_t* tile_expert, int32_t* tile_row0, int32_t* num_tiles,
                       int64_t tile_capacity, void* workspace, void* stream);

/*
 * mi355_permute_plan without a workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid it).  No
 * counterpart in the reference.  Same arguments, outputs and results as mi355_permute_plan;
 * the scratch (slot ranks, per-workgroup histograms) lives in an array inside the library,
 * mi355_permute_plan_static_max_bytes() = 8 MiB per GPU, held until the process ends.
 * Returns MI355_EINVAL without launching when mi355_permute_plan_workspace_bytes(T,K,E)
 * exceeds that (e.g. N = T*K = 2^20 slots with E <= 128 fits; N = 131072, E = 256 fits).
 * Calls no hipMalloc / hipFree and no allocating library routine.  All calls on one GPU share
 * that GPU's array: calls that overlap on one GPU (two streams or threads) race -- serialise
 * them, or use mi355_permute_plan with separate workspaces.  The first call on a device looks
 * the array's address up and must not run under stream capture (it returns MI355_EINVAL
 * there): call once, uncaptured, beforehand -- T = 0 will do.
 */
int64_t mi355_permute_plan_static_max_bytes(void);
int mi355_permute_plan_static(const int64_t* ids_TK, int64_t T, int64_t K, int64_t E,
                              int64_t local_lo, int64_t local_hi, int64_t align,
                              int64_t tile_m, int32_t* counts_E, int32_t* seg_offsets,
                              int32_t* seg_counts, int32_t* row_of_slot,
                              int32_t* slot_of_row, int32_t* token_of_row,
                              int64_t row_capacity, int32_t* tile_expert,
                              int32_t* tile_row0, int32_t* num_tiles,
                              int64_t tile_capacity, void* stream);

/*
 * Segment offsets, counts and the tile list for rows that are ALREADY expert-major
 * with `counts[e]` rows per local expert (no padding): the layout
 * GroupedExperts.forward receives, llmtuner/models/common/moe/experts.py:152-204
 * (offsets_E = cumsum(counts), :204).  counts: (El) int32; negative counts are
 * treated as 0 and segments are clamped to the row_capacity rows that exist.
 * seg_counts is (2*El) int32 as in mi355_permute_plan (counts, then the experts by
 * descending count).  tile_capacity >= row_capacity/tile_m + El is always enough.
 */
int mi355_segments_from_counts(const int32_t* counts, int64_t El, int64_t tile_m,
                               int64_t row_capacity, int32_t* seg_offsets, int32_t* seg_counts,
                               int32_t* tile_expert, int32_t* tile_row0,
                               int32_t* num_tiles, int64_t tile_capacity, void* stream);

/*
 * rows[row_of_slot[t*K+k]] = x[t] for every slot with a row (each token row is read once
 * and stored K times), zero for padding rows; rows at or beyond seg_offsets[El] are left
 * untouched.  Replaces the gather x[token_indices], token_dispatch.py:197-199, and the
 * sentinel-row padding of the padded layout.  slot_of_row may be NULL when the plan has no
 * padding rows (align = 1); with it, total_rows points at seg_offsets[El] on the device.
 */
int mi355_permute_rows_fwd(const void* x, int dtype, const int32_t* row_of_slot,
                           const int32_t* slot_of_row, const int32_t* total_rows,
                           void* rows, int64_t T, int64_t D, int64_t K,
                           int64_t row_capacity, void* stream);

/*
 * dx[t] = sum_k drows[row_of_slot[t*K+k]] (slots with row -1 contribute nothing),
 * summed in fp32 (fp64 rows: in fp64) in ascending k, written in `dtype`.  This is the backward of the
 * row gather (autograd's index_put accumulate for token_dispatch.py:199; the
 * duplicate-row contract is tests/unit_tests/cpu/kernel/test_kernel_contracts.py:
 * 114-127).
 */
int mi355_permute_rows_bwd(const void* drows, int dtype, const int32_t* row_of_slot,
                           void* dx, int64_t T, int64_t D, int64_t K, void* stream);

/* ------------------------------------------------------------------ combine */

/*
 * out[t] = sum_k weights[t][k] * y[row_of_slot[t*K+k]], contributions taken in
 * ascending row order (the order index_add visits them in).  Replaces
 * LocalTokenDispatcher.combine, token_dispatch.py:255-275, and the padding strip
 * of TorchAOTokenDispatcher._unpermute, torchao_dispatch.py:177-185.
 * round_terms != 0 reproduces the reference's default rounding (each weighted row
 * rounded to the y dtype before the sum, accumulate_in_fp32 = False); 0 keeps the
 * products in fp32 (accumulate_in_fp32 = True).  The sum itself is always fp32 and
 * rounded once to `dtype`.
 */
int mi355_combine_fwd(const void* y, int dtype, const float* weights_TK,
                      const int32_t* row_of_slot, void* out, int64_t T, int64_t D,
                      int64_t K, int round_terms, void* stream);

/*
 * dy[row] = weights[t][k] * dout[t]   for every slot with a row (rows that hold
 *           padding are zeroed up to *total_rows)
 * dweights[t][k] = sum_d y[row][d] * dout[t][d]   (0 for slots without a row)
 * The autograd-derived backward of token_dispatch.py:263-274.
 */
int mi355_combine_bwd(const void* dout, const void* y, int dtype,
                      const float* weights_TK, const int32_t* row_of_slot,
                      const int32_t* slot_of_row, const int32_t* total_rows,
                      void* dy, float* dweights_TK, int64_t T, int64_t D, int64_t K,
                      int64_t row_capacity, void* stream);

/* ---------------------------------------------------- grouped SwiGLU experts */

/*
 * For every tile-listed row r of local expert e:
 *   gate[r] = rows[r] . w1[e]^T,  up[r] = rows[r] . w3[e]^T      (R,F)
 *   h[r]    = silu(gate[r]) * up[r]                              (R,F)
 *   y[r]    = h[r] . w2[e]^T                                     (R,D)
 * with gate, up, the SiLU value, the product and y each rounded to `dtype`
 * (the reference's rounding points).  Replaces GroupedExperts._compute,
 * llmtuner/models/common/moe/experts.py:204-209, its _grouped_mm (:211-285) and
 * SwiGLU.forward, llmtuner/models/common/activation.py:36-37.
 * w1,w3: (El,F,D); w2: (El,D,F), all `dtype`, row-major.
 * token_of_row (optional): when given, `rows` is the UNPERMUTED (T,D) token matrix and
 * row r reads rows[token_of_row[r]] -- the gather of token_dispatch.py:197-199 fused
 * into the operand loads, so the (R,D) expert-major copy is never written.  bf16 with
 * D and F multiples of 64 only (MI355_EUNSUP otherwise).  num_tokens = T bounds the
 * index: entries are clamped to [0, T) on the device (a corrupt index reads a wrong row,
 * never out of bounds), and the call returns MI355_EINVAL without launching when
 * token_of_row is given with T < 1 or with T*D*2 >= 2^32 bytes (the gather addresses its
 * source with 32-bit byte offsets).  Ignored when token_of_row is NULL.
 * gate/up/h are saved for the backward (each (row_capacity,F)).  A caller that will never
 * run the backward may pass gate = up = NULL (both): for bf16 with D and F multiples of 64
 * (>= 384) those two outputs are then not written at all; for any other dtype or shape
 * that is MI355_EINVAL (the other paths use the buffers as intermediates).
 * The kernels walk the plan's tile list in tiles of mi355_grouped_tile_m(dtype) rows
 * (256), so the list must have been built with that value.
 */
int64_t mi355_grouped_tile_m(int dtype);
int mi355_grouped_swiglu_fwd(const void* rows, const int32_t* token_of_row, int64_t num_tokens,
                             const void* w1, const void* w3, const void* w2, int dtype,
                             const int32_t* seg_offsets,
                             const int32_t* seg_counts, const int32_t* tile_expert,
                             const int32_t* tile_row0, const int32_t* num_tiles,
                             int64_t tile_capacity, void* gate, void* up, void* h,
                             void* y, int64_t El, int64_t D, int64_t F,
                             int64_t row_capacity, void* stream);

/*
 * Backward of the above (autograd-derived in the reference):
 *   dh = dy . w2[e];  dgate = dh * up * silu'(gate);  dup = dh * silu(gate)
 *   drows = dgate . w1[e] + dup . w3[e]
 *   dw2[e] = dy_e^T . h_e;  dw1[e] = dgate_e^T . rows_e;  dw3[e] = dup_e^T . rows_e
 * dgate/dup are caller-provided scratch of (row_capacity,F) each.  Weight
 * gradients are written (not accumulated) in `dtype`; experts with no rows get
 * zeros.  Any of drows/dw1/dw3/dw2 may be NULL to skip it.  token_of_row and num_tokens
 * have the meaning they have in the forward (`rows` = the (T,D) token matrix); drows is always
 * expert-major (row_capacity,D) and goes through mi355_permute_rows_bwd.
 */
int mi355_grouped_swiglu_bwd(const void* dy, const void* rows,
                             const int32_t* token_of_row, int64_t num_tokens, const void* w1,
                             const void* w3, const void* w2, const void* gate,
                             const void* up, const void* h, int dtype,
                             const int32_t* seg_offsets, const int32_t* seg_counts,
                             const int32_t* tile_expert, const int32_t* tile_row0,
                             const int32_t* num_tiles, int64_t tile_capacity,
                             void* dgate, void* dup, void* drows, void* dw1,
                             void* dw3, void* dw2, int64_t El, int64_t D, int64_t F,
                             int64_t row_capacity, void* stream);

/*
 * The backward of "experts, then combine" as one call, for the case the layer actually
 * runs: out[t] = sum_k weights[t][k] * y[row(t,k)] with y from mi355_grouped_swiglu_fwd
 * called with token_of_row (x = the (T,D) token matrix).  It computes what
 * mi355_combine_bwd followed by mi355_grouped_swiglu_bwd compute (the autograd-derived
 * backward of GroupedExperts.forward, experts.py:204-209 and :211-285, and of
 * LocalTokenDispatcher.combine, token_dispatch.py:255-275) without ever writing the
 * expert-major gradient dy = weights * dout or reading y:
 *   dh[r]   = row_scale[r] * (dout[token_of_row[r]] . w2[e])     (scaled in the epilogue)
 *   hs[r]   = row_scale[r] * h[r],  h recomputed from gate and up (h need not be kept)
 *   dw2[e]  = dout[token_of_row]_e^T . hs_e
 *   dot_partial[r][j] = sum over the j-th 128 columns f of (dout[token_of_row[r]] . w2[e])[f] * h[r][f]
 * and dgate, dup, drows, dw1, dw3 as in mi355_grouped_swiglu_bwd.  The gradient of
 * weights[t][k] is the sum over j of dot_partial[row(t,k)][j] (mi355_combine_scores_bwd).
 * Two bf16 roundings move compared with the two-call form (dh is rounded once, after the
 * scaling, instead of dy and dh each; dW2 rounds weights*h instead of weights*dout); both
 * stay inside the bf16 tolerance of the path.
 * bf16 only, D and F multiples of 64 and >= 384; token_of_row is required here and
 * num_tokens = T bounds it as in mi355_grouped_swiglu_fwd (dout and x are both (T,D)):
 * mi355_grouped_combine_bwd_slots returns the number of partials per row (the second
 * dimension of dot_partial), or 0 when this entry point does not cover the case (then use
 * the two-call form).  row_scale (row_capacity floats) comes from mi355_combine_row_scale:
 * row_scale[r] = weights[slot_of_row[r]], 0 for rows that hold padding.
 * dgate, dup, hs: caller-provided (row_capacity,F) each; dot_partial (row_capacity,slots) fp32.
 * stages: 0 for the whole backward, or a mask of MI355_STAGE_DH ... MI355_STAGE_DW3 (below) to
 * launch only those kernels on the same buffers (profilers, callers that schedule the stages).
 */
int64_t mi355_grouped_combine_bwd_slots(int dtype, int64_t D, int64_t F);
int mi355_grouped_swiglu_combine_bwd(const void* dout, const void* x, const int32_t* token_of_row,
                                     int64_t num_tokens, const float* row_scale, const void* w1, const void* w3,
                                     const void* w2, const void* gate, const void* up, int dtype,
                                     const int32_t* seg_offsets, const int32_t* seg_counts,
                                     const int32_t* tile_expert, const int32_t* tile_row0,
                                     const int32_t* num_tiles, int64_t tile_capacity, void* dgate,
                                     void* dup, void* hs, float* dot_partial, void* drows,
                                     void* dw1, void* dw3, void* dw2, int64_t El, int64_t D,
                                     int64_t F, int64_t row_capacity, int stages, void* stream);
int mi355_combine_row_scale(const float* weights_TK, const int32_t* slot_of_row, float* row_scale,
                            int64_t T, int64_t K, int64_t row_capacity, void* stream);
/* dweights[t][k] = sum_j dot_partial[row_of_slot[t*K+k]][j], summed in ascending j; 0 for
 * slots without a row. */
int mi355_combine_scores_bwd(const float* dot_partial, int64_t slots, const int32_t* row_of_slot,
                             float* dweights_TK, int64_t T, int64_t K, int64_t row_capacity,
                             void* stream);

/*
 * One of the seven bf16 MFMA kernels behind the two calls above, by itself, on the
 * same buffers: for profilers and for callers that schedule the stages themselves.
 * No counterpart in the reference.  bf16 only, D and F multiples of 64.
 */
#define MI355_STAGE_GATEUP 1 /* gate, up, h   <- rows, w1, w3 */
#define MI355_STAGE_DOWN 2   /* y             <- h, w2        */
#define MI355_STAGE_DH 4     /* dgate, dup    <- dy, w2, gate, up */
#define MI355_STAGE_DX 8     /* drows         <- dgate, dup, w1, w3 */
#define MI355_STAGE_DW2 16   /* dw2           <- dy, h        */
#define MI355_STAGE_DW1 32   /* dw1           <- dgate, rows  */
#define MI355_STAGE_DW3 64   /* dw3           <- dup, rows    */
int mi355_grouped_swiglu_stage(int stage, const void* dy, const void* rows,
                               const int32_t* token_of_row, int64_t num_tokens, const void* w1,
                               const void* w3, const void* w2, void* gate, void* up,
                               void* h, void* y, const int32_t* seg_offsets,
                               const int32_t* seg_counts, const int32_t* tile_expert,
                               const int32_t* tile_row0, const int32_t* num_tiles,
                               int64_t tile_capacity, void* dgate, void* dup, void* drows,
                               void* dw1, void* dw3, void* dw2, int64_t El, int64_t D,
                               int64_t F, int64_t row_capacity, void* stream);

/*
 * One grouped linear map over expert-major rows, the reference's pluggable
 * GroupedExperts._grouped_mm(x_TD, weight_EOI, offsets_E)
 * (llmtuner/models/common/moe/experts.py:211-216, :256-285):
 *   y[r] = x[r] . w[e(r)]^T      x (rows, I), w (El, O, I) row-major, y (rows, O)
 * over the segments of a plan / of mi355_segments_from_counts, fp32 accumulation, one rounding
 * to `dtype` (fp32, bf16 or fp64; x, w and y share it).  It is what GroupedExperts is built from when
 * its gated activation is not SwiGLU (llmtuner/models/common/activation.py:40-64, SituGLU):
 * gate = linear(x, w1), up = linear(x, w3), h = activation(gate, up), y = linear(h, w2).
 * bf16 with I and O multiples of 64 (>= 384) runs the MFMA kernels of the SwiGLU path (the down
 * projection's kernel forward, the dH product with a plain epilogue for dx, the dW2 kernel for
 * dw); everything else the strided fp32-MFMA GEMM.  Rows outside the listed segments are not
 * written.  The backward (autograd of the above): dx[r] = dy[r] . w[e(r)], dw[e] = sum over the
 * segment of dy[r]^T x[r]; dx or dw may be NULL; an expert without rows gets a zero dw.
 */
int mi355_grouped_linear_fwd(const void* x, const void* w, int dtype, const int32_t* seg_offsets,
                             const int32_t* seg_counts, const int32_t* tile_expert,
                             const int32_t* tile_row0, const int32_t* num_tiles,
                             int64_t tile_capacity, void* y, int64_t El, int64_t I, int64_t O,
                             int64_t row_capacity, void* stream);
int mi355_grouped_linear_bwd(const void* dy, const void* x, const void* w, int dtype,
                             const int32_t* seg_offsets, const int32_t* seg_counts,
                             const int32_t* tile_expert, const int32_t* tile_row0,
                             const int32_t* num_tiles, int64_t tile_capacity, void* dx, void* dw,
                             int64_t El, int64_t I, int64_t O, int64_t row_capacity, void* stream);

/*
 * RMS normalisation over the last axis, the `rms_norm` entry of the reference's kernel
 * registry (llmtuner/kernel/ops/rms_norm.py:10-31; reference math
 * llmtuner/kernel/cpu/basic.py:17-25 = torch.nn.functional.rms_norm): the norm the decoder
 * layer applies right before the MoE block (models/qwen/qwen3/model.py:452).
 *   r[t] = 1/sqrt(mean_d x[t][d]^2 + epsilon);   y[t][d] = (x[t][d] * r[t]) * weight[d]
 * computed in fp32 and rounded once to `dtype` (fp32 or bf16; x, weight and y share it).
 * rstd: optional (rows) fp32 output of r, the only thing the backward keeps.
 */
int mi355_rms_norm_fwd(const void* x, const void* weight, int dtype, void* y, float* rstd,
                       int64_t rows, int64_t D, float epsilon, void* stream);

/*
 * Backward of the above (autograd-derived in the reference), g = dy * weight, xh = x * r:
 *   dx[t][d] = r[t] * (g[t][d] - xh[t][d] * mean_d(g[t][.] * xh[t][.]))
 *   dweight[d] = sum_t dy[t][d] * xh[t][d]      (fixed summation order, no atomics)
 * dx or dweight may be NULL to skip it.  workspace (for dweight):
 * mi355_rms_norm_bwd_workspace_bytes(rows, D) bytes.
 */
int64_t mi355_rms_norm_bwd_workspace_bytes(int64_t rows, int64_t D);
int mi355_rms_norm_bwd(const void* dy, const void* x, const void* weight, const float* rstd,
                       int dtype, void* dx, void* dweight, void* workspace, int64_t rows,
                       int64_t D, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_MOE_H */
