/*
 * C ABI of the MI355X (gfx950) fused top-k MoE kernels.
 *
 * The reference reaches this path through a Python operator interface and has
 * no C ABI of its own; every entry point below names the reference function it
 * stands in for (paths relative to the reference root).  A binding only needs
 * raw device pointers, sizes and a HIP stream: there are no framework types in
 * any signature.
 *
 * Conventions
 *   - every pointer is a device pointer unless the comment says "host";
 *   - `stream` is a `hipStream_t` passed as `void*` (NULL = the null stream);
 *   - kernels are enqueued on `stream`; no entry point synchronises, allocates
 *     or frees device memory; scratch is passed in by the caller and sized with
 *     the matching `*_workspace_bytes` function;
 *   - return value: 0 on success, a negative MTS_ERR_* for a contract violation
 *     (nothing was launched), a positive `hipError_t` if a launch failed;
 *   - T tokens, K experts per token, E experts, H model width, I expert width,
 *     TK = T*K routes; "entry" = t*K+k; "row" = position in the expert-sorted
 *     order; tensors are dense row-major.
 */
#ifndef MTS_MOE_H
#define MTS_MOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MTS_VERSION 4

/* element types of activations / weights / weight gradients */
#define MTS_BF16 0
#define MTS_F32 1
#define MTS_F16 2

#define MTS_OK 0
#define MTS_ERR_NULL (-1)        /* a required pointer is NULL                      */
#define MTS_ERR_SHAPE (-2)       /* sizes out of the supported range                */
#define MTS_ERR_DTYPE (-3)       /* unknown or unsupported element type             */
#define MTS_ERR_WORKSPACE (-4)   /* workspace too small                             */
#define MTS_ERR_ALIGN (-5)       /* a pointer or leading dimension is not 16-byte aligned */

#define MTS_MAX_EXPERTS 1024          /* router post-process, capacity mask                      */
#define MTS_MAX_MOE_EXPERTS 65534     /* routing metadata and the grouped GEMMs (the reference's
                                         limit, minitrain/kernels/triton/fused_moe.py:55-70)      */
#define MTS_MAX_TOP_K 8

int mts_version(void);
const char* mts_error_string(int code);

/* ---- router post-process ------------------------------------------------
 * Replaces TorchOpsBackend.router_postprocess (minitrain/kernels/torch_ops.py:87-120)
 * and _router_forward_kernel (minitrain/kernels/triton/router.py:62-152).
 * logits [T,E] f32 -> weights [T,K] f32, indices [T,K] i32 (rank order, ties to
 * the lower expert index), prob_mean [E], z_loss [1], entropy [1].
 * The statistics are reduced in a fixed order (no float atomics).
 * counts [E] i32 and load_balance [1] may be NULL.  They stand in for the router
 * module's bookkeeping around the operator (minitrain/model/moe_router.py:82-90):
 * routes per expert (its torch.bincount) and E * sum_e (counts_e / (T*K)) * prob_mean_e
 * (its auxiliary loss).
 * load_stats [E+7] f32 may be NULL; it holds the module's load metrics
 * (moe_router.py:113-135) for dropless routing: [0,E) the fraction of the routes each
 * expert takes, [E] the largest and [E+1] the smallest route count, [E+2] the
 * population standard deviation of the fractions times E, [E+3] the largest fraction
 * times E, [E+4] the number of experts without a route, [E+5] 0 (no route dropped),
 * [E+6] entropy / log E (entropy itself for E = 1).
 * weights_act [T,K] in act_dtype (MTS_BF16 or MTS_F16) may be NULL; it is the copy of
 * `weights` the router module makes for the MoE block (`expert_weights.to(
 * hidden_states.dtype)`, moe_router.py:139-140), rounded to nearest even.             */
int64_t mts_router_workspace_bytes(int64_t T, int E);
int mts_router_fwd(const float* logits, int64_t T, int E, int K, int normalize,
                   float* weights, int32_t* indices, float* prob_mean, float* z_loss,
                   float* entropy, int32_t* counts, float* load_balance, float* load_stats,
                   void* weights_act, int act_dtype, void* workspace, int64_t workspace_bytes,
                   void* stream);

/* Replaces _router_backward_kernel (minitrain/kernels/triton/router.py:155-259).
 * g_weights [T,K], g_prob_mean [E], g_z_loss [1] -> dlogits [T,E]; each of the
 * gradient inputs may be NULL, which stands for zeros (an output that took no part in
 * the loss).  g_load_balance [1] is the gradient of the load-balancing term; it
 * reaches the logits through prob_mean only (the route fractions counts/(T*K)
 * carry no gradient) and needs the counts the forward call wrote.
 * g_weights_act [T,K] in act_dtype is the gradient that arrived at the activation-dtype
 * copy of the weights; it is widened and added to g_weights (either may be NULL).     */
int mts_router_bwd(const float* logits, const float* weights, const int32_t* indices,
                   const float* g_weights, const void* g_weights_act, int act_dtype,
                   const float* g_prob_mean, const float* g_z_loss,
                   const float* g_load_balance, const int32_t* counts, int64_t T, int E, int K,
                   int normalize, float* dlogits, void* stream);

/* ---- router projection ----------------------------------------------------
 * Replaces the fp32 router GEMM of TopKRouter.forward and its autograd backward
 * (minitrain/model/moe_router.py:64-76: `hidden_states.float()` followed by
 * `F.linear(router_input, weight.float())`): logits[t,e] = sum_h float(x[t,h]) * w_r[e,h],
 * fp32 products and sums, x [T,H] read in act_dtype (no fp32 copy), w_r [E,H] f32.
 * E <= 16, H a multiple of 4 and at most 4096, E * H <= 32768 (W_r sits in LDS).   */
int mts_router_logits_fwd(const void* x, const float* w_r, int64_t T, int H, int E,
                          int act_dtype, float* logits, void* stream);

/* dx[t,h] = sum_e dlogits[t,e] * w_r[e,h] (written in act_dtype, the cast the autograd
 * of `.float()` applies), d_w_r[e,h] = sum_t dlogits[t,e] * float(x[t,h]) (f32; partial
 * sums per block of rows in the workspace, added in a fixed order).              */
int64_t mts_router_logits_bwd_workspace_bytes(int64_t T, int H, int E);
int mts_router_logits_bwd(const float* dlogits, const void* x, const float* w_r, int64_t T,
                          int H, int E, int act_dtype, void* dx, float* d_w_r,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* ---- the layer's head in two launches ---------------------------------------
 * mts_router_logits_fwd + mts_router_fwd + mts_moe_route as one chain (router projection,
 * post-process and routing metadata of minitrain/model/moe_router.py:64-90 and
 * triton/fused_moe.py:74-154): the post-process runs on the logits while they are still in
 * registers, the routes per expert it counts per block are the chunk histogram of the
 * routing metadata; in the second launch every scatter block adds up those counts itself and
 * one more block reduces the statistics.  Outputs as in
 * those three calls (logits [T,E] f32 are written for the backward pass; weights_act,
 * load_balance and load_stats may be NULL).  E <= 16, H a multiple of 4 and at most 4096, E * H <= 32768,
 * K <= min(E, MTS_MAX_TOP_K).  The statistics are summed in a fixed order of their own: they agree
 * with mts_router_fwd to rounding, indices and the permutation agree exactly.              */
int64_t mts_moe_head_workspace_bytes(int64_t T, int K, int E);
int mts_moe_head_fwd(const void* x, const float* w_r, int64_t T, int H, int E, int K, int normalize,
                     int act_dtype, float* logits, float* weights, int32_t* indices, void* weights_act,
                     float* prob_mean, float* z_loss, float* entropy, int32_t* counts,
                     float* load_balance, float* load_stats, int32_t* expert_start, int32_t* s_scatter,
                     int32_t* s_reverse, int32_t* x_gather, void* workspace, int64_t workspace_bytes,
                     void* stream);

/* mts_router_bwd chained into mts_router_logits_bwd: every block of the projection's backward
 * kernel first forms the logit gradients of its rows from the post-process's saved tensors
 * (same arithmetic as mts_router_bwd), so dlogits never goes through memory.  dx [T,H] in
 * act_dtype, d_w_r [E,H] f32.  Gradient inputs may be NULL (zeros) as for mts_router_bwd.      */
int64_t mts_moe_head_bwd_workspace_bytes(int64_t T, int H, int E);
int mts_moe_head_bwd(const void* x, const float* w_r, const float* logits, const float* weights,
                     const int32_t* indices, const int32_t* counts, const float* g_weights,
                     const void* g_weights_act, const float* g_prob_mean, const float* g_z_loss,
                     const float* g_load_balance, int64_t T, int H, int E, int K, int normalize,
                     int act_dtype, void* dx, float* d_w_r, void* workspace, int64_t workspace_bytes,
                     void* stream);

/* ---- routing metadata ---------------------------------------------------
 * Replaces compute_routing_metadata (minitrain/kernels/triton/fused_moe.py:74-154)
 * and its three kernels (fused_moe_kernels.py:25-234): per-expert counts [E],
 * expert_start [E+1], the stable expert-major permutation (s_scatter [TK]: row ->
 * entry, s_reverse [TK]: entry -> row, x_gather [TK]: row -> token) and, when
 * tile_row_start/tile_expert/tile_count are not NULL, the list of block_m-row
 * tiles (capacity min(TK, ceil(TK/block_m)+E-1) each, tile_count [1]).
 * s_scatter, s_reverse and x_gather may all be NULL: then only counts and
 * expert_start (and the tile list) are written, which is what the router module
 * needs in place of its torch.bincount (minitrain/model/moe_router.py:82).
 * A negative index marks a dropped route (see mts_moe_capacity_mask): it is not
 * counted and gets no row, its s_reverse entry is -1, and expert_start[E] is the
 * number of kept routes; every kernel below works on the kept rows only, combine
 * and the routing-weight gradient skip the -1 entries.
 * Returns MTS_ERR_SHAPE if E > MTS_MAX_MOE_EXPERTS (beyond MTS_MAX_EXPERTS the three kernels run
 * once per window of MTS_MAX_EXPERTS experts); indices >= E are a caller error:
 * they are clamped into range (memory-safe, result undefined).                  */
int64_t mts_moe_route_workspace_bytes(int64_t T, int K, int E);
int mts_moe_route(const int32_t* top_k_index, int64_t T, int K, int E, int block_m,
                  int32_t* counts, int32_t* expert_start, int32_t* s_scatter,
                  int32_t* s_reverse, int32_t* x_gather, int32_t* tile_row_start,
                  int32_t* tile_expert, int32_t* tile_count, void* workspace,
                  int64_t workspace_bytes, void* stream);

/* mts_moe_route without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops and harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The chunk counters live in an array inside the library's device
 * image, MTS_ROUTE_STATIC_BYTES per GPU the library is used on, held until the process ends; the
 * call allocates and frees nothing.  Same arguments, results and errors as mts_moe_route
 * otherwise; MTS_ERR_WORKSPACE when mts_moe_route_workspace_bytes(T, K, E) exceeds
 * MTS_ROUTE_STATIC_BYTES (T*K*E <= 2^28, e.g. 4 M routes over 64 experts).  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (different streams) race; calls
 * on one stream, or ordered by events, do not.  The first call on a device looks the array's
 * address up (hipGetSymbolAddress), so make one call per device outside a graph capture.   */
#define MTS_ROUTE_STATIC_BYTES (4 << 20)
int mts_moe_route_static(const int32_t* top_k_index, int64_t T, int K, int E, int block_m,
                         int32_t* counts, int32_t* expert_start, int32_t* s_scatter,
                         int32_t* s_reverse, int32_t* x_gather, int32_t* tile_row_start,
                         int32_t* tile_expert, int32_t* tile_count, void* stream);

/* ---- capacity-limited dispatch --------------------------------------------
 * The selection rule of TopKRouter._capacity_mask (minitrain/model/moe_router.py:
 * 29-61): per expert, the `capacity` routes with the largest router weight are
 * kept, equal weights in ascending flat entry (t*K+k) order.  keep [T*K] gets 1/0
 * per entry; kept_index [T*K] (may be NULL) gets the expert index of a kept route
 * and -1 for a dropped one, which is the form mts_moe_route takes for a compacted
 * dispatch (the compaction the reference reserves its expert_capacity_factor for,
 * minitrain/model/config.py:24-28); accepted_counts [E] = min(count_e, capacity).
 * top_k_weights are the fp32 router weights.  The caller computes capacity =
 * max(min_capacity, ceil(factor*T*K/E)) (moe_router.py:38-42).                 */
int64_t mts_moe_capacity_workspace_bytes(int64_t T, int K, int E);
int mts_moe_capacity_mask(const int32_t* top_k_index, const float* top_k_weights, int64_t T, int K,
                          int E, int64_t capacity, uint8_t* keep, int32_t* kept_index,
                          int32_t* accepted_counts, void* workspace, int64_t workspace_bytes,
                          void* stream);

/* ---- weight staging -----------------------------------------------------
 * src [E,R,C] of src_dtype -> dst of dst_dtype, [E,R,C] (transpose=0) or [E,C,R]
 * (transpose=1).  Stands in for the in-kernel weight casts of the reference
 * (fused_moe_kernels.py:343,351) and stages the transposed operands of the
 * backward GEMMs.  The GEMM entry points below take their weight operands in the
 * activation dtype: bf16 weights with bf16 activations, fp32 with fp32.       */
int mts_moe_stage_weights(const void* src, int src_dtype, void* dst, int dst_dtype, int E,
                          int64_t R, int64_t C, int transpose, void* stream);

/* The same casts for fp32 master weights (the reference's single-GPU training contract,
 * minitrain/train/trainer.py:95-98: fp32 parameters under bf16 autocast) as ONE launch for both
 * expert weights: w1 (n1 values) -> w1_out, w2 (n2 values) -> w2_out, both of dst_dtype
 * (MTS_BF16 or MTS_F16), same layout; n1 and n2 multiples of 8, all pointers 16-byte aligned.
 * The backward GEMMs read the same copies, so a layer step casts each weight once.        */
int mts_moe_cast_weights_pair(const float* w1, void* w1_out, int64_t n1, const float* w2,
                              void* w2_out, int64_t n2, int dst_dtype, void* stream);

/* ---- forward ------------------------------------------------------------
 * Replaces _fused_up_proj_swiglu_kernel (fused_moe_kernels.py:264-367):
 * for every row r (token x_gather[r], expert e): [g;u] = W1[e] x ; a = silu(g)*u.
 * x [T,H], w1 [E,2I,H], pre_act [TK,2I], post_act [TK,I], all of act_dtype
 * (MTS_BF16, MTS_F16: MFMA kernels, H and I multiples of 8; MTS_F32: plain fp32 kernels).
 * weights (flat [T*K], act_dtype) and s_scatter (row -> entry) are optional as a pair.  With
 * them post_act[r] = s_r * silu(g) * u, s_r = weights[s_scatter[r]] (fp32 product, one
 * rounding): the down projection then yields s_r * y[r], the combine is the unweighted sum
 * (mts_moe_combine with weights == NULL), and the same buffer is the `weighted_act` operand of
 * the dW2 GEMM (the reference recomputes it in the backward kernel, fused_moe_kernels.py:587-588), so
 * mts_moe_bwd_dy1 need not write it again.                                         */
int mts_moe_fwd_gateup_swiglu(const void* x, const void* w1, const int32_t* x_gather,
                              const int32_t* expert_start, const void* weights,
                              const int32_t* s_scatter, int64_t T, int K, int E, int H,
                              int I, int act_dtype, void* pre_act, void* post_act,
                              void* stream);

/* Replaces _fused_down_proj_kernel (fused_moe_kernels.py:369-437):
 * y[r] = W2[e] a[r];  post_act [TK,I], w2 [E,H,I] -> y [TK,H].                */
int mts_moe_fwd_down(const void* post_act, const void* w2, const int32_t* expert_start,
                     int64_t TK, int E, int H, int I, int act_dtype, void* y, void* stream);

/* The two launches above as ONE (the pair of launches in _FusedMoEFunction.forward,
 * minitrain/kernels/triton/fused_moe.py:203-249): same arguments, same tiles, bit-identical pre_act,
 * post_act and y.  On their own both GEMMs end in a round of tiles that fills a fraction of the chip;
 * in one launch the down tiles take the CUs as the gate/up tiles leave them (forward GEMMs -5 %).
 * A down tile reads post_act rows that gate/up tiles of the same launch write: the m-tiles of both
 * parts go to the XCDs in the same contiguous ranges, so writers and readers of a row share an L2, and
 * a counter per m-tile in `workspace` tells the readers when the rows are complete.
 *   mts_moe_fwd_joint_supported: 1 where the launch exists (bf16 / fp16, H and I multiples of 64, one
 *     expert's W1 no larger than an XCD's L2); elsewhere mts_moe_fwd_gateup_down returns MTS_ERR_SHAPE.
 *   workspace: mts_moe_fwd_joint_workspace_bytes(TK, E) bytes of int32, 16-byte aligned, ALL ZERO on the
 *     first call.  A launch that ran through leaves it all zero, so calls that follow one another on a
 *     stream share one workspace (larger and smaller problems alike); calls that may overlap need one each.
 *   status: word 0 of the workspace stays 0.  A block that waited longer than 200 ms for its rows gives
 *     up and sets bit 0 (every other wait then ends at once: no launch hangs); a block that finds rows
 *     written on another XCD than its own sets bit 1.  Either way the outputs of that call are invalid
 *     and the workspace must be cleared before it is used again.  Reading the word is the caller's
 *     business (after a synchronisation, or from a copy made on the stream).                          */
int mts_moe_fwd_joint_supported(int act_dtype, int H, int I);
int64_t mts_moe_fwd_joint_workspace_bytes(int64_t TK, int E);
int mts_moe_fwd_gateup_down(const void* x, const void* w1, const void* w2, const int32_t* x_gather,
                            const int32_t* expert_start, const void* weights,
                            const int32_t* s_scatter, int64_t T, int K, int E, int H, int I,
                            int act_dtype, void* pre_act, void* post_act, void* y,
                            int32_t* workspace, int64_t workspace_bytes, void* stream);

/* Replaces _token_gather_weighted_sum_kernel (fused_moe_kernels.py:451-498):
 * out[t] = addend[t] + sum_k w[t,k] * y[s_reverse[t*K+k]]  (fp32 sum, one rounding);
 * weights == NULL gives the unweighted sum used for dx; addend [T,H] (act_dtype) may be NULL
 * (zeros): it is the other gradient that reaches x, the router projection's (the sum autograd
 * forms for minitrain/model/blocks.py:89-96, where x feeds both the router and the experts). */
int mts_moe_combine(const void* y, const void* weights, const void* addend, const int32_t* s_reverse,
                    int64_t T, int K, int H, int act_dtype, void* out, void* stream);

/* ---- backward -----------------------------------------------------------
 * Replaces _moe_bwd_down_proj_kernel (fused_moe_kernels.py:500-600):
 * A = W2[e]^T dO[t];  dS = <A,a>;  weighted_act = s*a;  [dg;du] = d(s*A)/d[g;u].
 * The weight operand comes in one of two layouts: w2_as_stored = 1, w2 is W2 itself
 * [E,H,I] in the activation dtype, or w2_as_stored = 0, it is the transposed copy [E,I,H]
 * made by mts_moe_stage_weights.  mts_moe_bwd_weights_as_stored(act_dtype, H, I) says
 * whether this entry point and mts_moe_bwd_dx take the stored layout (bf16, H and 2I
 * multiples of 64); otherwise they return MTS_ERR_SHAPE for it.  ds_partial is
 * [TK, mts_moe_ds_partials(I)] f32 scratch reduced by mts_moe_bwd_ds (fixed order, no
 * atomics).  weighted_act may be NULL: it is then not written (the caller holds s*a already,
 * see mts_moe_fwd_gateup_swiglu).  schedule may be NULL; otherwise (16-bit activations,
 * mts_moe_bwd_schedule_bytes(E) > 0 bytes, 16-byte aligned) one more block of the launch
 * writes the schedule of mts_moe_bwd_joint there, see mts_moe_bwd_schedule.            */
int mts_moe_ds_partials(int I);
int mts_moe_bwd_weights_as_stored(int act_dtype, int H, int I);
int mts_moe_bwd_dy1(const void* d_out, const void* w2, int w2_as_stored, const void* pre_act,
                    const void* weights, const int32_t* x_gather, const int32_t* s_scatter,
                    const int32_t* expert_start, int64_t T, int K, int E, int H, int I,
                    int act_dtype, void* d_pre_act, void* weighted_act, float* ds_partial,
                    int32_t* schedule, void* stream);

/* dS[entry] = sum of the partials of row s_reverse[entry], cast to act_dtype
 * (fused_moe.py:437-443 returns dS as [T,K] in the weights' dtype).          */
int mts_moe_bwd_ds(const float* ds_partial, const int32_t* s_reverse, int64_t TK, int I,
                   int act_dtype, void* d_weights, void* stream);

/* Replaces _moe_bwd_dX_expanded_kernel (fused_moe_kernels.py:674-756):
 * dx_expanded[r] = W1[e]^T [dg;du][r];  w1 is W1 itself [E,2I,H] (w1_as_stored = 1) or
 * its transposed copy [E,H,2I] (w1_as_stored = 0), see mts_moe_bwd_dy1.
 * The per-token sum is mts_moe_combine with weights == NULL.                 */
int mts_moe_bwd_dx(const void* d_pre_act, const void* w1, int w1_as_stored,
                   const int32_t* expert_start, int64_t TK, int E, int H, int I, int act_dtype,
                   void* dx_expanded, void* stream);

/* Replaces _moe_bwd_dW2_kernel (fused_moe_kernels.py:602-672):
 * dW2[e] = sum_{r in e} dO[x_gather[r]] (x) weighted_act[r]   -> [E,H,I] grad_dtype.
 * Experts without routes receive zeros.
 *
 * workspace (both weight-gradient entry points): NULL, or at least
 * mts_moe_bwd_dw_workspace_bytes(which, E, H, I) bytes (which = 1 for dW1, 2 for dW2).
 * With a workspace, an expert that holds more than 1.15 times the balanced share of the
 * routes has its rows cut into chunks that run as separate blocks and are added in a
 * fixed order by a second kernel, so that skewed routing does not leave the GPU waiting
 * for the tiles of the fullest expert; results stay run-to-run identical.  Without one,
 * every tile reduces over all rows of its expert in one block (bf16 activations only;
 * the fp32 path ignores the workspace).                                        */
int64_t mts_moe_bwd_dw_workspace_bytes(int which, int E, int H, int I);
int mts_moe_bwd_dw2(const void* d_out, const void* weighted_act, const int32_t* x_gather,
                    const int32_t* expert_start, int64_t T, int K, int E, int H, int I,
                    int act_dtype, int grad_dtype, void* d_w2, void* workspace,
                    int64_t workspace_bytes, void* stream);

/* Replaces _moe_bwd_dW1_kernel (fused_moe_kernels.py:758-828):
 * dW1[e] = sum_{r in e} [dg;du][r] (x) x[x_gather[r]]        -> [E,2I,H] grad_dtype. */
int mts_moe_bwd_dw1(const void* d_pre_act, const void* x, const int32_t* x_gather,
                    const int32_t* expert_start, int64_t T, int K, int E, int H, int I,
                    int act_dtype, int grad_dtype, void* d_w1, void* workspace,
                    int64_t workspace_bytes, void* stream);

/* Replaces the three launches that follow _moe_bwd_down_proj_kernel in
 * _FusedMoEFunction.backward (fused_moe.py:351-443: _moe_bwd_dW2_kernel,
 * _moe_bwd_dX_expanded_kernel, _moe_bwd_dW1_kernel) and the dS reduction with ONE launch
 * plus the chunk sum: the same arithmetic, block for block, as mts_moe_bwd_dw1,
 * mts_moe_bwd_dw2, mts_moe_bwd_dx (w1 as stored, [E,2I,H]) and mts_moe_bwd_ds, so the
 * results are bit-identical to those calls.  The block index orders the work: the
 * weight-gradient tiles, which are the long ones, start first and the dX tiles fill the
 * CUs as they come free.  mts_moe_bwd_joint_supported() says whether the shapes allow it
 * (16-bit activations, 2I a multiple of 64); both weight gradients have grad_dtype.
 * workspace1 / workspace2: as for mts_moe_bwd_dw1 / mts_moe_bwd_dw2 (may be NULL).
 * d_w2 == NULL (then weighted_act and workspace2 may be NULL too): dW2 is left to a call of
 * mts_moe_bwd_dw2, which does not depend on mts_moe_bwd_dy1.
 *
 * schedule (may be NULL; no counterpart in the reference, whose launches leave the placement
 * of blocks to the hardware): all tiles of a weight-gradient unit (an expert, or a row chunk of
 * an over-full one) run on one XCD, and with uneven routing a round-robin deal of the units
 * leaves most of the chip waiting for the XCD that drew the longest ones.  The schedule is a
 * table, written on the GPU from expert_start alone, that deals the units out longest first to
 * the XCD with the fewest rows so far and splits the dX tiles so that every XCD ends up with the
 * same work.  It is used when both workspaces are given (it presumes their row chunks) and
 * changes which block computes a tile, not the tile: results are bit-identical with and without.
 * mts_moe_bwd_dy1 writes it as a by-product; mts_moe_bwd_schedule does in a launch of its own.
 * mts_moe_bwd_schedule_bytes(E): bytes of the table, 0 when E is beyond what it covers (32). */
int mts_moe_bwd_joint_supported(int act_dtype, int H, int I);
int64_t mts_moe_bwd_schedule_bytes(int E);
int mts_moe_bwd_schedule(const int32_t* expert_start, int64_t TK, int E, int32_t* schedule, void* stream);
int mts_moe_bwd_joint(const void* d_out, const void* weighted_act, const void* d_pre_act,
                      const void* x, const void* w1, const int32_t* x_gather,
                      const int32_t* expert_start, const int32_t* s_reverse,
                      const float* ds_partial, int64_t T, int K, int E, int H, int I,
                      int act_dtype, int grad_dtype, void* dx_expanded, void* d_w1, void* d_w2,
                      void* d_weights, void* workspace1, int64_t workspace1_bytes,
                      void* workspace2, int64_t workspace2_bytes, const int32_t* schedule, void* stream);

/* mts_moe_bwd_joint with the router's backward in the same launch: what mts_moe_head_bwd computes
 * (the autograd backward of minitrain/model/moe_router.py:64-90 given the routing-weight gradient
 * and the loss-term gradients), by the same per-block arithmetic and with bit-identical results,
 * as trailing blocks of the joint launch.  They form the routing-weight gradient from ds_partial
 * themselves, so they depend on nothing the launch writes, and run on the CUs that the last
 * round of dX tiles leaves idle; one small launch then sums the per-block partials of d_w_r.
 * w_r [E,H] f32, logits [T,E] f32, weights [T,K] f32, indices [T,K], counts [E] (needed with
 * g_load_balance), g_prob_mean [E] / g_z_loss / g_load_balance (each may be NULL: zero);
 * outputs dx_router [T,H] in act_dtype and d_w_r [E,H] f32; router_workspace as for
 * mts_moe_head_bwd (mts_moe_head_bwd_workspace_bytes).  dx (may be NULL): the layer's gradient
 * of x [T,H], i.e. mts_moe_combine(dx_expanded, NULL, dx_router, s_reverse, ...) as part of
 * the launch of partial sums (two routes per token) or as one more launch behind it.  mts_moe_bwd_joint_router_supported()
 * says whether the shapes allow it (those of mts_moe_bwd_joint, E <= 8, H a multiple of 4 whose
 * dW_r sums fit the block's LDS).                                                       */
int mts_moe_bwd_joint_router_supported(int act_dtype, int64_t T, int H, int I, int E);
int mts_moe_bwd_joint_router(const void* d_out, const void* weighted_act, const void* d_pre_act,
                             const void* x, const void* w1, const int32_t* x_gather,
                             const int32_t* expert_start, const int32_t* s_reverse,
                             const float* ds_partial, int64_t T, int K, int E, int H, int I,
                             int act_dtype, int grad_dtype, void* dx_expanded, void* d_w1, void* d_w2,
                             void* d_weights, void* workspace1, int64_t workspace1_bytes,
                             void* workspace2, int64_t workspace2_bytes, const float* w_r,
                             const float* logits, const float* weights, const int32_t* indices,
                             const int32_t* counts, const float* g_prob_mean, const float* g_z_loss,
                             const float* g_load_balance, int normalize, void* dx_router, void* dx,
                             float* d_w_r, void* router_workspace, int64_t router_workspace_bytes,
                             const int32_t* schedule, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MTS_MOE_H */
