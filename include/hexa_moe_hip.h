/* libhexa_moe_hip.so -- C ABI of the MI355X (gfx950) expert-specific operators.
 *
 * Plain pointers and sizes only; every pointer except the layout struct is a DEVICE pointer owned
 * by the caller; nothing here allocates, frees, synchronises with the host or reads device memory
 * back.  Every entry point enqueues its kernels on `stream` (a hipStream_t passed as void*; NULL is
 * the null stream) and returns immediately with 0 (HEXA_OK) or a negative HEXA_ERR_* code;
 * hexa_last_error() then holds a message (thread-local).  The library never exits the process.
 *
 * Each entry point names the reference interface it replaces (paths relative to the HEXA-MoE
 * repository, hexa_moe_cuda/hexa_moe/...).
 */
#ifndef HEXA_MOE_HIP_H
#define HEXA_MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HEXA_ABI_VERSION 9

/* element types */
#define HEXA_F32 0
#define HEXA_F16 1
#define HEXA_BF16 2

/* expert weight layouts accepted by hexa_esmm */
#define HEXA_W_IN_OUT 0 /* w[E][in][out]  (what the reference's ESMM_TENSOR_CORE takes)            */
#define HEXA_W_OUT_IN 1 /* w[E][out][in]  (nn.Linear style; what FUSED_GRAD takes for its `w`)      */

/* epilogue activations of hexa_esmm */
#define HEXA_ACT_NONE 0
#define HEXA_ACT_GELU 1 /* out_act = gelu_erf(out), written next to the pre-activation `out`        */
#define HEXA_ACT_GELU_BWD 2 /* out = (x.W) * gelu'(y1) with y1 READ from out_act (same shape as out)   */

/* return codes */
#define HEXA_OK 0
#define HEXA_ERR_ARG (-1)         /* null pointer, negative size, inconsistent flags                */
#define HEXA_ERR_UNSUPPORTED (-2) /* dtype combination or dimension granularity not implemented     */
#define HEXA_ERR_LAUNCH (-3)      /* the HIP runtime refused a launch                               */

/* Rows per row-tile of the gathered-row kernels; the routing pass emits one tile record per
 * HEXA_TILE_ROWS rows of every (slot, expert) segment. */
#define HEXA_TILE_ROWS 128
/* A second set of records with twice as many rows per tile, for the large-tile kernels. */
#define HEXA_TILE_ROWS_L 256
/* Tokens handled by one wavefront in the routing pass. */
#define HEXA_ROUTE_UNIT 512

/* ------------------------------------------------------------------------------------------------
 * Routing metadata ("route blob"): ONE caller-owned int32 device buffer per MoE depth that every
 * operator below consumes.  hexa_route_layout_get() gives the size and the position (in int32
 * units) of each part so the host can slice it:
 *   counts     [k][E]        tokens per expert per routing slot
 *   offsets    [k][E+1]      exclusive prefix of counts (unpadded; offsets[s][E] == T)
 *   token_ids  [k][T]        token ids grouped by expert, ascending inside a segment (stable)
 *   expert_ids [k][T]        expert of each list position (the reference's expert_idx_list)
 *   tile_count [k]           number of row tiles of the slot
 *   tile_info  [k][mt_ub][4] {expert, first list position, rows (<=HEXA_TILE_ROWS), 0}
 *   tile_count_l [k], tile_info_l [k][mt_ub_l][4]   the same with HEXA_TILE_ROWS_L rows per tile
 *   scratch    [k][units][E] per-wavefront histograms of the routing pass
 * The buffer may be shared by all MoE depths of a model (sized for the largest T*k): its contents
 * are rebuilt by hexa_route_build for each depth and reused by that depth's forward and backward
 * operators.
 * ---------------------------------------------------------------------------------------------- */
typedef struct hexa_route_layout {
    int64_t counts, offsets, token_ids, expert_ids, tile_count, tile_info, tile_count_l, tile_info_l, scratch;
    int64_t total_ints; /* size of the blob in int32 elements */
    int32_t mt_ub;      /* row-tile upper bound per slot: T/HEXA_TILE_ROWS + E                      */
    int32_t mt_ub_l;    /* the same for HEXA_TILE_ROWS_L                                            */
    int32_t units;      /* wavefront units per slot: ceil(T/HEXA_ROUTE_UNIT)                        */
    int32_t reserved;
} hexa_route_layout;

int hexa_route_layout_get(int num_tokens, int top_k, int num_experts, hexa_route_layout* out);

/* Routing segment pass: histogram + exclusive scan + stable scatter, all slots in one call, no
 * padding, no host round trip.  Element (t, s) of the routing choice is read at
 * routing[t*token_stride + s*slot_stride]; `routing_is_i64` selects int64 (torch.topk's output) or
 * int32 elements.  Ids outside [0, E) are skipped.
 * Replaces TOKEN_COUNT + TOKEN_ASSIGN: torch/hexa_moe_ops.cpp:9-43 -> launch_count / launch_assign,
 * kernels/shared_cuda_core.cu:126-182, 284-333, and the per-slot Python loop impls/layers.py:233-251. */
int hexa_route_build(const void* routing, int routing_is_i64, int64_t token_stride, int64_t slot_stride,
                     int num_tokens, int top_k, int num_experts, int32_t* route, void* stream);

/* The two reference ops one to one (a single routing slot, contiguous int32 routing[T]).
 * `pad` is the segment granularity: 16 reproduces the reference's expanded_tokens_per_expert
 * (shared_cuda_core.cu:165-171), 1 gives the exact prefix.  `scratch` holds
 * ceil(T/HEXA_ROUTE_UNIT)*E int32.  token/expert lists: only real positions are written; padding
 * positions keep what the caller filled in (-1 in the reference, impls/layers.py:238-239).
 * Replaces launch_count (include/hexa_moe.h:3-10) and launch_assign (include/hexa_moe.h:12-20). */
int hexa_token_count(int32_t* tokens_per_expert, int32_t* expanded_tokens_per_expert, const int32_t* routing,
                     int num_tokens, int num_experts, int pad, int32_t* scratch, void* stream);
int hexa_token_assign(int32_t* token_idx_list, int32_t* expert_idx_list,
                      const int32_t* expanded_tokens_per_expert, const int32_t* routing, int num_tokens,
                      int num_experts, int32_t* scratch, void* stream);

/* Build a route blob from reference-style lists (k slots of exactly T entries each, grouped by
 * expert, no padding): what a caller holding token_idx_list / expert_idx_list from the two ops above
 * (pad = 1) passes on to the operators.  Replaces the host-side rebuild of expert_start_list in
 * launch_fused_grad_* (kernels/fused_ops_full.cu:486-512). */
int hexa_route_from_lists(const int32_t* token_idx_list, const int32_t* expert_idx_list, int num_tokens,
                          int top_k, int num_experts, int32_t* route, void* stream);

/* The same from the reference's own list format: the k slots' lists concatenated, every expert's
 * segment padded to a multiple of 16 with -1 (kernels/shared_cuda_core.cu:165-171 as called from
 * impls/layers.py:233-249), slot s occupying [slot_ends[s], slot_ends[s+1]) of the lists; slot_ends
 * is the caller's device array of k+1 cumulative lengths (cum_ids, impls/layers.py:245-248) and
 * list_len the lists' total length.  Fillers are dropped in place of being skipped by every operator
 * (kernels/esmm_full.cu:96-101); entries keep their order. */
int hexa_route_from_padded_lists(const int32_t* token_idx_list, const int32_t* expert_idx_list,
                                 const int32_t* slot_ends, int64_t list_len, int num_tokens, int top_k,
                                 int num_experts, int32_t* route, void* stream);

/* ESMM: out[(s),t,:] (+)= x[(s),t,:] . W[e_s(t)] + bias[e_s(t)] over all routed (slot, token) pairs.
 *   m2s == 0: x [T,in] shared by the slots, out [k,T,out]      (fc1 of the MoE FFN)
 *   m2s != 0: x [k,T,in] per slot,          out [T,out] = sum over slots (fc2; deterministic order)
 * w_layout selects w[E][in][out] or w[E][out][in]; bias [E][out] may be NULL.  x_dt is F32 (then w,
 * bias and out must be F32: true-fp32 MFMA path) or F16/BF16 (w may be the same 16-bit type or F32,
 * fp32 accumulation; out may be that 16-bit type or F32).  accumulate != 0 adds into `out`.
 * act == HEXA_ACT_GELU additionally writes gelu(out) to out_act (same shape/dtype as out; m2s == 0).
 * act == HEXA_ACT_GELU_BWD multiplies the result by gelu'(y1), y1 read from out_act (same shape/dtype
 * as out; m2s == 0, no accumulate): the backward ESMM dy1 = (dy.W2^T) * act'(y1) in one pass.
 * Dimension granularity: in and out multiples of 8 (16-bit) / 4 (fp32).
 * slot_ws (may be NULL) is scratch for m2s != 0 with top_k > 1: (top_k-1)*T*out elements of out_dt.
 * With it, all slots run in ONE launch (slot 0 writes `out`, the others write slot_ws) followed by a
 * small reduction out += sum(slot_ws) in slot order; without it the slots run one launch after the
 * other, each adding into `out`.  Both orders are fixed, so results are reproducible either way.
 * Replaces ESMM_TENSOR_CORE (torch/hexa_moe_ops.cpp:45-117) -> launch_esmm_accum_shared_tensor_{full,
 * mix,half} (include/hexa_moe.h:22-72, kernels/esmm_full.cu:249-300), and with w_layout OUT_IN the
 * ESMM task of FUSED_GRAD (kernels/fused_ops_full.cu:117-247). */
int hexa_esmm(void* out, const void* x, const void* w, const void* bias, const int32_t* route, int m2s,
              int w_layout, int accumulate, int num_tokens, int top_k, int in_dim, int out_dim,
              int num_experts, int x_dt, int w_dt, int bias_dt, int out_dt, int act, void* out_act,
              void* slot_ws, void* stream);

/* ESTMM: dw[e][o][i] (+)= sum over slots s and tokens t routed to e of dy[(s),t,o] * x[(s),t,i].
 * dy_per_slot / x_per_slot say whether the operand is [k,T,*] (1) or [T,*] shared by the slots (0).
 * dt is the element type of dy and x (F32, F16 or BF16); dw_dt is F32 or dt.  Experts without tokens
 * get exact zeros (or are left untouched when accumulating).
 * plan / max_slots / scratch (optional; used by the 16-bit kernels).  With a plan from hexa_estmm_plan for the same
 * routing, max_slots and result size, the persistent kernel runs (up to 256 experts and 8 slots): one workgroup per
 * CU takes (expert, 128 x 128 block) items from a queue, longest first, so the load balances without cutting
 * experts; only an expert whose list is longer than a workgroup's share of the whole launch is cut into up to 8
 * parts, whose fp32 partial results go through `scratch` (max_slots * out_dim * in_dim floats; max_slots < 2 or
 * scratch == NULL: nothing is cut) and are added in a fixed order, so results stay bit-reproducible.  The plan
 * also holds the queue's counters, which the call updates and leaves at zero: calls that share a plan must not
 * overlap (calls on one stream do not).  Without a plan one workgroup walks an expert's whole token list per
 * block and the kernel is as slow as the busiest expert.
 * Replaces the ESTMM task of FUSED_GRAD (kernels/fused_ops_full.cu:248-371). */
int hexa_estmm(void* dw, const void* dy, const void* x, const int32_t* route, int dy_per_slot, int x_per_slot,
               int accumulate, int num_tokens, int top_k, int out_dim, int in_dim, int num_experts, int dt,
               int dw_dt, int32_t* plan, int max_slots, float* scratch, void* stream);

/* Work plan of hexa_estmm for one routing: HEXA_ESTMM_PLAN_INTS(num_experts) ints (experts by decreasing load,
 * their parts, first work unit and first scratch slot, number of units, then the work queue's counters, zeroed).
 * out_dim / in_dim: the size of the result the plan is for (0, 0: unknown -- experts above 1.5x the mean load are
 * cut, the rule of the one-item-per-workgroup kernel).  Depends on the routing, max_slots and that size only, so
 * one plan serves every hexa_estmm call of a layer's backward whose results have the same number of 128 x 128
 * blocks.  No counterpart in the reference, whose ESTMM task walks each expert's list in one thread block
 * (kernels/fused_ops_full.cu:248-371). */
#define HEXA_ESTMM_PLAN_INTS(num_experts) (4 * (num_experts) + 32)
int hexa_estmm_plan(int32_t* plan, const int32_t* route, int num_tokens, int top_k, int num_experts, int max_slots,
                    int out_dim, int in_dim, void* stream);

/* ESS: db[e][o] (+)= sum over slots and tokens routed to e of dy[(s),t,o].
 * ws (optional, ws_floats floats of scratch; 8*num_experts*out_dim is enough): long token lists are then
 * summed in up to 8 parts by separate workgroups and folded in a fixed order, which keeps the kernel
 * from being as slow as the busiest expert's list; results stay bit-reproducible.
 * Replaces the ESS task of FUSED_GRAD (kernels/fused_ops_full.cu:372-431). */
int hexa_ess(void* db, const void* dy, const int32_t* route, int dy_per_slot, int accumulate, int num_tokens,
             int top_k, int out_dim, int num_experts, int dt, int db_dt, float* ws, int64_t ws_floats, void* stream);

/* hexa_ess for callers that cannot allocate or hand over scratch (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same kernels and the same split walk as hexa_ess with
 * 8*num_experts*out_dim floats of scratch, so the results are bit-identical to that call, but the partial sums
 * live in an array built into the library (HEXA_ESS_NOALLOC_MAX_FLOATS floats per device, held until the
 * process ends).  8*num_experts*out_dim beyond that limit is rejected with HEXA_ERR_UNSUPPORTED.  The call
 * allocates and frees nothing.  All calls on one device share the array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are ordered and safe.  The device of `stream` must be the
 * current device.  No counterpart in the reference (its ESS task allocates nothing because it walks each
 * list in one thread block, kernels/fused_ops_full.cu:372-431). */
#define HEXA_ESS_NOALLOC_MAX_FLOATS (2 * 1024 * 1024)
int hexa_ess_noalloc(void* db, const void* dy, const int32_t* route, int dy_per_slot, int accumulate,
                     int num_tokens, int top_k, int out_dim, int num_experts, int dt, int db_dt, void* stream);

/* The reference's fused backward of one expert linear:
 *   j_x[(s),t,:in] (+)= j_y[(s),t,:out] . w[e]      w [E][out][in]
 *   j_w[e]         (+)= sum j_y^T x                 j_w [E][out][in]
 *   j_b[e]         (+)= sum j_y                     j_b [E][out], NULL = FUSED_GRAD_NO_BIAS
 *   m2s == 0: j_y [T,out] shared, x and j_x [k,T,in]     (fc2 call, impls/layers.py:409-416)
 *   m2s != 0: j_y [k,T,out], x [T,in] shared, j_x [T,in] (fc1 call, impls/layers.py:435-451)
 * act_dt: element type of j_y and x; w_dt: of w; jx_dt / jw_dt / jb_dt: of the results.
 * slot_ws: scratch of hexa_esmm for the m2s != 0 case ((top_k-1)*T*in elements of jx_dt) or NULL.
 * plan / max_slots / estmm_scratch: as for hexa_estmm (a plan from hexa_estmm_plan for the same routing; NULL / 0 /
 * NULL walks every expert's list in one workgroup).  ess_ws / ess_ws_floats: as for hexa_ess (NULL / 0: one pass).
 * With them a caller of the fused op gets the balanced ESTMM and the split ESS walk; results do not depend on it
 * beyond the order of the partial sums, which is fixed either way.
 * Replaces FUSED_GRAD / FUSED_GRAD_NO_BIAS (torch/hexa_moe_ops.cpp:119-275) ->
 * launch_fused_grad_{bias,no_bias}_{full,mix,half} (include/hexa_moe.h:74-181). */
int hexa_fused_grad(void* j_b, void* j_x, void* j_w, const void* j_y, const void* w, const void* x,
                    const int32_t* route, int m2s, int accumulate, int num_tokens, int top_k, int in_dim,
                    int out_dim, int num_experts, int act_dt, int w_dt, int jx_dt, int jw_dt, int jb_dt,
                    void* slot_ws, int32_t* plan, int max_slots, float* estmm_scratch, float* ess_ws,
                    int64_t ess_ws_floats, void* stream);

/* Steps 6-8 of the backward in one call: out[s][t][:] = (x[t][:] . w[e_s(t)]) * gelu'(y1[s][t][:]) (out, y1
 * [k,T,out_dim] in x's type; no bias) and db[e][:] (+)= the sum of expert e's rows of `out` (ESS of the result).
 * On the 16-bit fast path the column sums are taken in the producing kernel's store loop, per row tile, and
 * folded in a fixed order, so `out` is not read again; otherwise hexa_esmm and hexa_ess run one after the other.
 * ws: hexa_esmm_ess_ws_floats() floats (NULL: always the two-operator form).
 * Replaces the ESMM task of FUSED_GRAD + activation jacobian + the ESS task of the next FUSED_GRAD
 * (impls/layers.py:404-436, kernels/fused_ops_full.cu:372-431) for GELU. */
int hexa_esmm_ess_ws_floats(int num_tokens, int top_k, int out_dim, int num_experts, int64_t* out);
int hexa_esmm_gelu_bwd_ess(void* out, void* db, const void* x, const void* w, const void* y1, const int32_t* route,
                           int w_layout, int db_accumulate, int num_tokens, int top_k, int in_dim, int out_dim,
                           int num_experts, int x_dt, int w_dt, int db_dt, float* ws, int64_t ws_floats, void* stream);

/* Elementwise backward of the fused GELU: dy1 = dy2 * gelu'(y1), n elements of type dt.  The
 * reference evaluates act' with torch.autograd.functional.jacobian (impls/layers.py:281-283,427). */
int hexa_gelu_bwd(void* dy1, const void* dy2, const void* y1, int64_t n, int dt, void* stream);

/* ---- routing front end (fused; the PyTorch path of the host code stays available) ----------------
 * Gate projection logits[t][e] = sum_d x[t][d]*wg[e][d] with fp32 accumulation; x is F32/F16/BF16,
 * wg fp32 [E][d], d a multiple of 8.  Replaces LinearTopKGate.forward with fp32_gate (gates/top.py:17-19:
 * a cast of x to fp32 plus a skinny fp32 GEMM). */
int hexa_gate_logits(float* logits, const void* x, const float* wg, int num_tokens, int model_dim,
                     int num_experts, int x_dt, void* stream);

/* Backward of the gate projection: dx[t][c] = sum_e dlogits[t][e]*wg[e][c] (type of x; NULL to skip) and
 * dwg[e][c] = sum_t dlogits[t][e]*x[t][c] (fp32; NULL to skip), both with fp32 products and sums.  dwg is
 * reduced over per-workgroup partial sums in a fixed order (deterministic); `ws` holds them and must have
 * hexa_gate_ws_floats() floats.  Replaces what autograd derives from gates/top.py:17-19 (two skinny fp32
 * GEMMs and the casts around them). */
int hexa_gate_ws_floats(int num_tokens, int model_dim, int num_experts, int64_t* out);
int hexa_gate_backward(void* dx, float* dwg, const float* dlogits, const void* x, const float* wg, int num_tokens,
                       int model_dim, int num_experts, int x_dt, float* ws, void* stream);

/* softmax(logits + noise_scale*noise) -> scores [T][E]; top-k expert ids idx [T][k] (int32, descending
 * score, ties to the lower id); me[e] = sum_t scores, ce[e] = (E/T)*#{t: top-1 = e}; l_aux =
 * sum_e me*ce / T (the GShard loss).  noise may be NULL.  ws: hexa_router_ws_floats() floats.
 * Replaces routing() + simplified_extract_critical + gshard_loss
 * (impls/cascaded_moe.py:515-531, impls/layers.py:476-484, impls/losses.py:12-19). */
int hexa_router_ws_floats(int num_tokens, int num_experts, int64_t* out);
int hexa_router_forward(float* scores, int32_t* idx, float* me, float* ce, float* l_aux, const float* logits,
                        const float* noise, float noise_scale, int num_tokens, int num_experts, int top_k,
                        float* ws, void* stream);
/* dlogits = d l_aux / d logits * (*grad_l_aux), through the softmax (ce is treated as a constant, as
 * in the reference where the one-hot mask carries no gradient). */
int hexa_router_backward(float* dlogits, const float* scores, const float* ce, const float* grad_l_aux,
                         int num_tokens, int num_experts, void* stream);

/* The same front end with the load-importance loss of impls/losses.py:21-42 (what the Swin-MoE configs
 * train with: IS_GSHARD_LOSS False).  idx = top-k of softmax(logits + noise_scale*noise); thr[t] = the
 * k-th choice's noisy logit; scores = softmax(logits) WITHOUT noise; importance[e] = sum_t scores;
 * load[e] = sum_t Phi((scores[t][e] - thr[t]) / sigma); l_aux = (cv2(importance) + cv2(load)) / 2 with
 * cv2(v) = unbiased var / (mean^2 + 1e-10).  sigma is the reference's gate_noise / E (it divides by
 * it whether or not noise was added).  g_importance / g_load [E] receive d l_aux / d importance, load
 * for the backward call, which returns dlogits = d l_aux / d logits * (*grad_l_aux) through the
 * softmax and through the threshold.  ws: hexa_router_ws_floats() floats.  2 <= E <= 1024.  The
 * reductions over tokens and the variance are carried in double (v[e] - mean cancels).
 * Replaces routing() + simplified_extract_critical + load_importance_loss
 * (impls/cascaded_moe.py:515-531, impls/layers.py:476-484, impls/losses.py:21-42). */
int hexa_router_forward_load_importance(float* scores, int32_t* idx, float* thr, float* importance, float* load,
                                        float* g_importance, float* g_load, float* l_aux, const float* logits,
                                        const float* noise, float noise_scale, float sigma, int num_tokens,
                                        int num_experts, int top_k, float* ws, void* stream);
int hexa_router_backward_load_importance(float* dlogits, const float* scores, const float* thr, const int32_t* idx,
                                         const float* g_importance, const float* g_load, const float* grad_l_aux,
                                         float sigma, int num_tokens, int num_experts, int top_k, void* stream);

/* ---- one MoE depth per call ---------------------------------------------------------------------------
 * hexa_moe_depth_forward / hexa_moe_depth_backward enqueue every kernel of one MoE depth -- the routing front
 * end, the routing segment pass and the ten steps of the formula table with the exact-GELU activation -- from
 * ONE call each, so a training step costs the host two library calls instead of two dozen.  They run the same
 * kernels as the single-operator entry points above, in the same order, and give the same results.
 * Replaces the bodies of MoE_Cascaded.forward's MoE branch (impls/cascaded_moe.py:508-568),
 * FusedMoE_Shared_CudaCore.forward (impls/layers.py:99-277) and .backward (impls/layers.py:280-474).
 *
 * All sizes and element types travel in a descriptor.  act_dt is the type of x, y1, y2, y, dy, dy1 and dx; w_dt of
 * fc1_w [E][hidden][d_in] and fc2_w [E][hidden][d_out] (act_dt or F32); b*_dt of the biases; g*_dt of the
 * gradients (F32 or act_dt).  loss: 0 = GShard, 1 = load-importance (then sigma = gate_noise / E > 0). */
typedef struct hexa_moe_depth_desc {
    int32_t num_tokens, top_k, num_experts, d_in, hidden, d_out;
    int32_t act_dt, w_dt, b1_dt, b2_dt, gw1_dt, gw2_dt, gb1_dt, gb2_dt;
    int32_t loss;
    float noise_scale; /* factor of `noise` in the logits (gate_noise / E while training, else 0) */
    float sigma;       /* load-importance only */
    int32_t reserved;
} hexa_moe_depth_desc;

/* Bytes of caller scratch the two calls need (either pointer may be NULL). */
int hexa_moe_depth_ws_bytes(const hexa_moe_depth_desc* d, int64_t* forward_bytes, int64_t* backward_bytes);

/* Forward.  With wg (fp32 [E][d_in]) the call starts at the gate: logits = x.wg^T (fp32), scores / idx / l_aux as
 * hexa_router_forward or hexa_router_forward_load_importance (noise [T][E] fp32 or NULL); logits, scores [T][E],
 * idx [T][k] int32, thr [T] (load-importance only, else NULL) and stats (GShard: me[E], ce[E], l_aux = 2E+1 floats;
 * load-importance: importance, load, their two gradients, l_aux = 4E+1 floats) are outputs the backward needs.
 * With wg == NULL the routing decision is the caller's: idx is read ([T][k] int32) and logits / scores / thr /
 * stats / noise are ignored.
 * Then: route = hexa_route_build(idx); y1 = x.W1^T + b1 and y2 = gelu(y1) ([k][T][hidden], saved for the backward);
 * y [T][d_out] = sum over slots of y2.W2 + b2.  Biases may be NULL.
 * plan (may be NULL): HEXA_ESTMM_PLAN_INTS(num_experts) ints that receive the work plan of the backward's ESTMM
 * calls (as hexa_estmm_plan; it depends on the routing only); hand the same buffer to hexa_moe_depth_backward and
 * that call skips making it.  (With the GShard loss and up to 240 experts the router, the loss, the routing pass and the plan
 * take two launches in all: the router counts its own tokens for the routing pass, whose one launch scatters the
 * tokens, finishes the loss and makes the plan.)
 * events (may be NULL): 2*n caller-owned hipEvent_t handles; pair i is recorded on `stream` around major kernel i
 * (0: fc1 + GELU, 1: fc2 and its slot sum), for callers that time kernels inside a step; NULL handles in the
 * array are skipped. */
int hexa_moe_depth_forward(const hexa_moe_depth_desc* d, const void* x, const float* wg, const float* noise,
                           const void* fc1_w, const void* fc1_b, const void* fc2_w, const void* fc2_b, float* logits,
                           float* scores, int32_t* idx, float* thr, float* stats, int32_t* route, int32_t* plan, void* y1,
                           void* y2, void* y, void* ws, int64_t ws_bytes, void* const* events, int num_events,
                           void* stream);

/* Backward of the same depth from dy [T][d_out] and (with wg) the device scalar grad_l_aux (NULL: the auxiliary
 * loss carries no gradient).  Results (each may be NULL to skip it): dx [T][d_in] = the expert path's input
 * gradient plus, with wg, the gate path's; dwg [E][d_in] fp32; dw1 [E][hidden][d_in], db1 [E][hidden],
 * dw2 [E][hidden][d_out], db2 [E][d_out].  dy1 is caller memory for the hidden gradient ([k][T][hidden] of act_dt);
 * its contents after the call are dy1 = (dy.W2^T) * gelu'(y1).  plan: the buffer the forward filled (its queue
 * counters are used and left at zero), or NULL.
 * events: pairs around (0) the dy1 kernel with its bias-gradient sums, (1) the dx kernel and its slot sum,
 * (2) ESTMM dW2, (3) ESTMM dW1. */
int hexa_moe_depth_backward(const hexa_moe_depth_desc* d, const void* dy, const float* grad_l_aux, const void* x,
                            const float* wg, const void* fc1_w, const void* fc2_w, const float* scores,
                            const int32_t* idx, const float* thr, const float* stats, const int32_t* route,
                            int32_t* plan, const void* y1, const void* y2, void* dx, float* dwg, void* dw1,
                            void* db1, void* dw2, void* db2, void* dy1, void* ws, int64_t ws_bytes, void* const* events,
                            int num_events, void* stream);

const char* hexa_last_error(void);
int hexa_abi_version(void);

/* Tuning / testing knobs of the kernels ("tile", "pipe", "general_kernels", "esmm_map", "esmm_group",
 * "estmm_group", "esmm_stream", "route_kernels", "batch", "ffn_fused", "gate_router"; 0 = automatic).  Each starts from an environment variable
 * (HEXA_MOE_TILE, HEXA_MOE_PIPE, HEXA_MOE_GENERAL_KERNELS, HEXA_ESMM_MAP, HEXA_ESMM_GROUP, HEXA_ESTMM_GROUP,
 * HEXA_ESMM_STREAM, HEXA_ROUTE_KERNELS).  Every setting computes the same results; the tests use it to run every kernel
 * variant.  No counterpart in the reference. */
int hexa_set_option(const char* name, int value);

#ifdef __cplusplus
}
#endif
#endif /* HEXA_MOE_HIP_H */
