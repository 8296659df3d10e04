/*
 * galvatron_moe.h -- C ABI of libgalvatron_moe.so, the MI355X (gfx950) implementation of the
 * Hetu-Galvatron MoE expert-layer hot path: top-k routing, token permute / unpermute and the
 * grouped expert GEMM with SwiGLU, forward and backward.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless the comment says "host".  The library never
 *     allocates, frees or retains tensor memory: outputs and workspaces are passed in.
 *   - Every entry point enqueues its kernels on `stream` (a hipStream_t passed as void*) and
 *     returns without synchronising.  Entry points are re-entrant and keep no state.
 *   - Return value: 0 on success, a negative gmoe_status otherwise (gmoe_status_string()).
 *     No kernel is launched when an argument check fails.
 *   - Matrices are dense row-major.  `dtype` is a gmoe_dtype.
 *   - Paths in the comments are relative to the reference tree (galvatron/core/runtime/...).
 */
#ifndef GALVATRON_MOE_H
#define GALVATRON_MOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GMOE_ABI_VERSION 10

typedef enum {
  GMOE_F32 = 0,
  GMOE_BF16 = 1,
  GMOE_F16 = 2,
  GMOE_F8E4M3 = 3 /* OCP e4m3fn, expert weights only */
} gmoe_dtype;

typedef enum {
  GMOE_OK = 0,
  GMOE_ERR_INVALID = -1,     /* bad pointer / shape / flag */
  GMOE_ERR_UNSUPPORTED = -2, /* valid request the library does not implement */
  GMOE_ERR_LAUNCH = -3,      /* HIP reported an error when launching */
  GMOE_ERR_TOO_LARGE = -4    /* sizes beyond the fixed maximum of an entry point without workspace */
} gmoe_status;

/* GMOE_SCORE_IDENTITY: the input already holds the scores (gmoe_seq_aux_loss and its gradient only) */
typedef enum { GMOE_SCORE_SOFTMAX = 0, GMOE_SCORE_SIGMOID = 1, GMOE_SCORE_IDENTITY = 2 } gmoe_score_fn;
typedef enum { GMOE_ACT_SILU = 0, GMOE_ACT_GELU = 1 } gmoe_act;

int gmoe_abi_version(void);
const char* gmoe_status_string(int status);

/* ---------------------------------------------------------------------------------------------
 * Router.  Replaces `topk_softmax_with_capacity` without capacity (moe/moe_utils.py:430-518) and
 * the statistics of `switch_load_balancing_loss_func` / `z_loss_func` (moe/moe_utils.py:14-59,
 * 115-127) that `TopKRouter.routing` (moe/router.py:371-421) needs.
 *
 *   logits  [T,E] dtype            in
 *   probs   [T,E] dtype            out  gate of the selected experts, 0 elsewhere
 *   routing_map [T,E] uint8        out  1 where selected (torch.bool storage)
 *   topk_idx [T,k] int32           out, optional (NULL): selected experts, best first
 *   tokens_per_expert [E] int64    out  column sums of routing_map
 *   stats [E+1] fp32               out, optional (NULL): stats[e] = sum_t score(t,e) where score is
 *                                  the fp32 softmax over all E logits (softmax score function) or
 *                                  the normalised sigmoid (router.py:173-191); stats[E] =
 *                                  sum_t logsumexp(logits[t,:])^2
 *   stats_ws                       workspace of gmoe_route_workspace_bytes(T,E) bytes; required
 *                                  when stats != NULL
 * Top-k ties are broken towards the lowest expert index; NaN ranks above every number.
 * expert_bias [E] fp32 (optional) is added to the sigmoid scores for selection only.
 * selection_scores [T,E] fp32 (optional): top-k ranks this matrix instead of the scores, the gates
 * still come from the scores; with pre_softmax (k > 1) or the sigmoid score function (k == 1) this
 * is TopKRouter.sinkhorn_load_balancing (moe/router.py:140-171: indices from the sinkhorn-normalised
 * costs, gate = activation(logits) on the selected experts).
 * num_groups/group_topk > 0 enable group-limited routing (moe/moe_utils.py:372-427).
 * scaling <= 0 means "no scaling factor".
 */
int64_t gmoe_route_workspace_bytes(int64_t T, int E);
int gmoe_route_topk(const void* logits, int dtype, int64_t T, int E, int k, int score_fn,
                    int pre_softmax, float scaling, const float* expert_bias,
                    const float* selection_scores, int num_groups, int group_topk, void* probs,
                    uint8_t* routing_map, int32_t* topk_idx, int64_t* tokens_per_expert, float* stats,
                    void* stats_ws, void* stream);

/* Backward of the router w.r.t. the logits (autograd of moe/moe_utils.py:482-514 plus the
 * gradients MoEAuxLossAutoScaler injects, moe/moe_utils.py:166-203):
 *   dlogits[t,e] = d<probs, dprobs>/dlogits + aux_scale * d(sum_e stats[e]*f[e])/dlogits
 *                  + z_scale * d(sum_t lse_t^2)/dlogits
 * with f = tokens_per_expert (may be NULL when aux_scale == 0).  dprobs is [T,E] in `dtype`
 * (only the selected entries are read), dlogits is [T,E] in `dtype`.  loss_scale (optional, one
 * fp32 on the device) multiplies aux_scale and z_scale: the value of
 * MoEAuxLossAutoScaler.main_loss_backward_scale, read without a host synchronisation. */
int gmoe_route_topk_bwd(const void* logits, int dtype, int64_t T, int E, int k, int score_fn,
                        int pre_softmax, float scaling, const uint8_t* routing_map,
                        const void* dprobs, const int64_t* tokens_per_expert, float aux_scale,
                        float z_scale, const float* loss_scale, void* dlogits, void* stream);

/* Sequence-level load-balancing loss (`sequence_load_balancing_loss_func`, moe/moe_utils.py:62-112,
 * called from TopKRouter.seq_aux_loss_load_balancing, moe/router.py:233-276).  Token (s, b) is row
 * s * batch_size + b of logits / routing_map [seq_length * batch_size, E].
 *   seq_counts [B,E] fp32  out  tokens of sequence b routed to expert e (from routing_map)
 *   seq_scores [B,E] fp32  out  sum_s score(s,b,e), score = fp32 softmax over all experts, or the
 *                               sigmoid divided by its row sum when k > 1 (moe/router.py:173-191)
 *   loss [1] fp32          out  coeff * mean_b sum_e (seq_counts * E / (S k)) * (seq_scores / S)
 * Sums run in a fixed order. */
int gmoe_seq_aux_loss(const void* logits, int dtype, const uint8_t* routing_map, int64_t seq_length,
                      int batch_size, int E, int k, int score_fn, float coeff, float* seq_counts,
                      float* seq_scores, float* loss, void* stream);

/* Its gradient: dlogits[t,:] = scale * grad_loss[0] * J_t^T seq_counts[t % batch_size, :], J_t the
 * Jacobian of token t's scores; scale = coeff * E / (B S^2 k) for the loss above.  grad_loss
 * (optional, one fp32 on the device) is the incoming gradient of the loss, e.g. what
 * MoEAuxLossAutoScaler injects (moe/moe_utils.py:166-203).  dlogits [T,E] in `dtype`. */
int gmoe_seq_aux_loss_bwd(const void* logits, int dtype, int64_t seq_length, int batch_size, int E,
                          int k, int score_fn, const float* seq_counts, float scale,
                          const float* grad_loss, void* dlogits, void* stream);

/* Column statistics of a [T,E] matrix of scores or logits, for the reference's free loss functions
 * `switch_load_balancing_loss_func` (moe/moe_utils.py:14-59: sum_t probs[t,e]) and `z_loss_func`
 * (moe/moe_utils.py:115-127: sum_t logsumexp(logits[t,:])^2):
 *   stats[e] = sum_t score(x)[t,e]   score_fn = identity: x itself; softmax / sigmoid as in
 *                                    gmoe_seq_aux_loss
 *   stats[E] = sum_t logsumexp(x[t,:])^2   (0 for score_fn = identity)
 * fp32 sums in a fixed order.  stats_ws: gmoe_route_workspace_bytes(T, E) bytes.  The loss values
 * follow from gmoe_router_bookkeeping on these statistics. */
int gmoe_score_stats(const void* x, int dtype, int64_t T, int E, int k, int score_fn, float* stats,
                     void* stats_ws, void* stream);

/* Gradient of  aux_scale * sum_e weights[e] * stats[e] + z_scale * stats[E]  (the statistics of
 * gmoe_score_stats) with respect to x, times grad_loss[0] (optional, one fp32 on the device):
 * the backward of the two free loss functions above.  weights [E] fp32 (e.g. tokens_per_expert),
 * may be NULL when aux_scale == 0; dx [T,E] in `dtype`. */
int gmoe_score_stats_bwd(const void* x, int dtype, int64_t T, int E, int k, int score_fn,
                         const float* weights, float aux_scale, float z_scale,
                         const float* grad_loss, void* dx, void* stream);

/* Sinkhorn normalisation of the routing costs (`sinkhorn`, moe/moe_utils.py:130-144): with
 * cost = exp(float(logits)), iterate d0 = (1/T) / (cost d1 + 1e-8), d1 = (1/E) / (cost^T d0 + 1e-8)
 * from d0 = d1 = 1 while the error exceeds tol (the error starts at 1e9 and is mean|d1 - d1_old|
 * after an iteration; at most max_iters iterations), then norm_out [T,E] fp32 = d1 * cost * d0.  One workgroup; the loop runs on the device, so there is
 * no host synchronisation per iteration.  iters_out (optional, one int on the device) receives the
 * iteration count. */
int gmoe_sinkhorn(const void* logits, int dtype, int64_t T, int E, float tol, int max_iters,
                  float* norm_out, int* iters_out, void* stream);

/* Router bookkeeping from the statistics of gmoe_route_topk, in one launch, every output optional:
 *   aux_loss[0] = aux_factor * sum_e stats[e] * tokens_per_expert[e]
 *                 (`switch_load_balancing_loss_func`, moe/moe_utils.py:55-58, aux_factor =
 *                 E * coeff / (T^2 k));   z_loss[0] = z_factor * stats[E]  (moe/moe_utils.py:126)
 *   *aux_tracker_slot += aux_loss * aux_tracker_scale,  *z_tracker_slot += z_loss * z_tracker_scale
 *                 (`save_to_aux_losses_tracker`, moe/moe_utils.py:547-574: the element
 *                 values[layer_idx - 1] of the logging tracker)
 *   local_tokens_per_expert[e] += tokens_per_expert[e]   (moe/router.py:415-419, fp32 [E]) */
int gmoe_router_bookkeeping(const float* stats, const int64_t* tokens_per_expert, int E,
                            float aux_factor, float z_factor, float* aux_loss, float* z_loss,
                            float* aux_tracker_slot, float aux_tracker_scale, float* z_tracker_slot,
                            float z_tracker_scale, float* local_tokens_per_expert, void* stream);

/* `get_updated_expert_bias` (moe/moe_utils.py:645-662) without its all-reduce: for every row r of
 * tokens_per_expert / expert_bias [rows, E] fp32,
 *   updated_bias[r,e] = expert_bias[r,e] + sign(mean_e(tokens[r,:]) - tokens[r,e]) * update_rate. */
int gmoe_expert_bias_update(const float* tokens_per_expert, const float* expert_bias, int64_t rows,
                            int E, float update_rate, float* updated_bias, void* stream);

/* Expert capacity (`topk_softmax_with_capacity` with capacity_factor, moe/moe_utils.py:519-544):
 * per expert column keep the `capacity` tokens with the largest gate value (by_position = 0, the
 * "probs" drop policy, a top-`capacity` over the token axis of the dense probs) or the first
 * `capacity` routed tokens (by_position = 1, the "position" policy: top-`capacity` of the 0/1 map).
 * Among equal keys the lowest token index wins (torch.topk leaves that order unspecified).
 *   out_map[t,e]   = pad ? chosen : (chosen && routing_map[t,e])       (pad_to_capacity)
 *   out_probs[t,e] = out_map[t,e] ? probs[t,e] : 0
 * probs / out_probs [T,E] in probs_dtype, maps [T,E] uint8.  capacity >= 1 (clamped to T). */
int gmoe_capacity_select(const void* probs, int probs_dtype, const uint8_t* routing_map, int64_t T,
                         int E, int64_t capacity, int by_position, int pad, void* out_probs,
                         uint8_t* out_map, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Permutation plan.  Replaces the index computation of `permute` (moe/moe_utils.py:264-272:
 * transpose + arange + masked_select) and `triton_make_row_id_map` (moe/fused_kernels.py:514-605).
 *
 *   routing_map [T,E] uint8              in
 *   dst_map [T,E] int32                  out  destination row of (token,expert) in the
 *                                        expert-major permuted tensor, -1 if not routed or dropped
 *   sorted_indices [sorted_cap] int64    out, optional: sorted_indices[dst] = token
 *   row_id_map [E,T] int64               out, optional: dst_map transposed, the reference's layout
 *   tokens_per_expert [E] int64          out  rows kept per expert
 *   expert_offsets [E+1] int64           out  exclusive prefix of tokens_per_expert
 *   capacity                             <= 0: dropless.  > 0: keep only the first `capacity` tokens
 *                                        of every expert and give every expert a block of exactly
 *                                        `capacity` rows (drop_and_pad, moe/moe_utils.py:252-263)
 * Destination rows >= sorted_cap are treated as dropped (dst_map = -1).
 */
int64_t gmoe_permute_plan_workspace_bytes(int64_t T, int E);
int gmoe_permute_plan(const uint8_t* routing_map, int64_t T, int E, int64_t capacity,
                      int32_t* dst_map, int64_t* sorted_indices, int64_t sorted_cap,
                      int64_t* row_id_map, int64_t* tokens_per_expert, int64_t* expert_offsets,
                      void* workspace, void* stream);

/* gmoe_permute_plan for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same arguments without the workspace, same
 * results.  No counterpart in the reference.  The chunk counts live in a device array inside the
 * library (512 KiB per GPU, held until the process ends); the call allocates and frees nothing.
 * Limit: E * ceil(T / 256) <= gmoe_permute_plan_static_max_slots() (65536), else
 * GMOE_ERR_TOO_LARGE and nothing is launched.  All calls on one GPU share that array: calls that
 * overlap on one GPU (different streams or threads) race; calls on one stream are ordered. */
int64_t gmoe_permute_plan_static_max_slots(void);
int gmoe_permute_plan_static(const uint8_t* routing_map, int64_t T, int E, int64_t capacity,
                             int32_t* dst_map, int64_t* sorted_indices, int64_t sorted_cap,
                             int64_t* row_id_map, int64_t* tokens_per_expert,
                             int64_t* expert_offsets, void* stream);

/* Row scatter: permuted[dst_map[t,e]] = tokens[t] for every routed (t,e).  Replaces
 * `tokens.index_select(0, sorted_indices)` (moe/moe_utils.py:275) and `_permute_kernel`
 * (moe/fused_kernels.py:643-695).  Optionally permutes the gate values too:
 * permuted_probs[dst] = probs[t,e] (moe/token_dispatcher.py:233-235).
 *   tokens [T,H], permuted [n_out,H] in `dtype`; probs [T,E], permuted_probs [n_out] in probs_dtype. */
int gmoe_permute_rows(const void* tokens, int dtype, int64_t T, int64_t H, int E,
                      const int32_t* dst_map, int64_t n_out, void* permuted, const void* probs,
                      int probs_dtype, void* permuted_probs, void* stream);

/* Row gather-reduce: out[t] = sum_e permuted[dst_map[t,e]] * (merging_probs ? merging_probs[t,e] : 1),
 * accumulated in fp32 over ascending e.  Replaces `unpermute` (moe/moe_utils.py:318-353) and
 * `_unpermute_kernel` (moe/fused_kernels.py:199-264); also the backward of gmoe_permute_rows.
 * Optional: unpermuted_probs[t,e] = permuted_probs_in[dst] (0 where not routed).
 * Optional: addend and residual, [T,H] in `dtype`, added to the rounded sum in that order with a
 * rounding after each: out[t] = round(round(round(sum) + addend[t]) + residual[t]), the result of
 * `output += shared_expert_output` (moe/token_dispatcher.py:686-688) followed by
 * `... + mlp_residual` (models/moe_modules.py:124-127) in one pass. */
int gmoe_unpermute_rows(const void* permuted, int dtype, int64_t T, int64_t H, int E,
                        const int32_t* dst_map, int64_t n_out, const void* merging_probs,
                        int probs_dtype, void* out, const void* permuted_probs_in,
                        void* unpermuted_probs, const void* addend, const void* residual,
                        void* stream);

/* Backward of gmoe_unpermute_rows with merging probs (`_unpermute_bwd_with_merging_probs_kernel`,
 * moe/fused_kernels.py:319-396): grad_permuted[dst] = grad_out[t] * p[t,e];
 * grad_probs[t,e] = <fwd_input[dst], grad_out[t]> (fp32), 0 where not routed. */
int gmoe_unpermute_rows_bwd(const void* grad_out, const void* fwd_input, int dtype, int64_t T,
                            int64_t H, int E, const int32_t* dst_map, int64_t n_out,
                            const void* merging_probs, int probs_dtype, void* grad_permuted,
                            void* grad_probs, void* stream);

/* Generic scatter-add for callers that only hold `sorted_indices` (moe/moe_utils.py:347-353):
 * acc[sorted_indices[r]] += permuted[r] (* permuted_probs[r]) with fp32 atomics into the zeroed
 * fp32 buffer acc [T,H]; then gmoe_cast_rows converts acc to the output dtype. */
int gmoe_scatter_add_rows(const void* permuted, int dtype, int64_t n_rows, int64_t H,
                          const int64_t* sorted_indices, const void* permuted_probs,
                          int probs_dtype, int64_t T, float* acc, void* stream);
int gmoe_cast_rows(const float* src, int64_t n_elems, int dst_dtype, void* dst, void* stream);

/* Chunk sort: the rows of `inp` are split into `num_splits` consecutive chunks of split_sizes[i]
 * rows; out is the concatenation of chunks sorted_idxs[0], sorted_idxs[1], ...  Replaces
 * `sort_chunks_by_idxs` (moe/moe_utils.py:356-369) and `_sort_chunks_by_idxs_kernel`
 * (moe/fused_kernels.py:785-871).  row_map [n_rows] int64 (out): row_map[dst] = src, which makes the
 * backward a call with `use_row_map` = 1 and the roles swapped (`_sort_chunks_by_map`, :913-959).
 * split_sizes / sorted_idxs are device int64 [num_splits]. */
int gmoe_sort_chunks(const void* inp, int dtype, int64_t n_rows, int64_t H,
                     const int64_t* split_sizes, const int64_t* sorted_idxs, int num_splits,
                     void* out, int64_t* row_map, void* stream);
int gmoe_scatter_rows_by_map(const void* inp, int dtype, int64_t n_rows, int64_t H,
                             const int64_t* row_map, void* out, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Expert activation.  y [N,2F] = [gate | up]; out [N,F] = act(y[:, :F]) * y[:, F:].  Replaces the
 * `glu` closure (moe/mlp.py:52-57) and swiglu / swiglu_back (transformer/fused_kernels.py:142-162).
 */
int gmoe_glu_fwd(const void* y, int dtype, int64_t N, int64_t F, int act, void* out, void* stream);
int gmoe_glu_bwd(const void* grad_out, const void* y, int dtype, int64_t N, int64_t F, int act,
                 void* grad_y, void* stream);
/* The same pair with the activation input kept as fp8 for the backward
 * (SwiGLUFunction with fp8_input_store, transformer/fused_kernels.py:190-204, selected by
 * activation_func_fp8_input_store at moe/mlp.py:329): the forward also writes y_fp8 [N,2F] =
 * y.to(float8_e4m3fn) (round to nearest even; beyond the format's range and NaN -> the NaN code),
 * the backward reads y_fp8, widens it to `dtype` (exact) and computes as gmoe_glu_bwd on that. */
int gmoe_glu_fwd_fp8store(const void* y, int dtype, int64_t N, int64_t F, int act, void* out,
                          void* y_fp8, void* stream);
int gmoe_glu_bwd_fp8in(const void* grad_out, const void* y_fp8, int dtype, int64_t N, int64_t F,
                       int act, void* grad_y, void* stream);

/* Bias of experts built with `add_bias_linear` (SequentialMLP only; GroupedMLP refuses it,
 * moe/mlp.py:43-45).  out [N,M] = x [N,M] + bias[expert of the row] with one rounding: the fc1 bias
 * in front of the activation (transformer/mlp.py:104-135, `intermediate_parallel + bias_parallel`
 * and bias_swiglu_impl), and with x = NULL the fc2 bias handed on as rows
 * (`output_bias.expand_as(output)`, moe/mlp.py:200-207).  bias [E,M]; expert_offsets [E+1] int64
 * (device), NULL with E = 1 for one group of all N rows; rows past the last offset keep x (zero
 * without x); out may be x.  The backward sums the incoming gradient over each expert's rows in
 * fp32 in a fixed order: grad_bias [E,M] (zero for an expert without rows); the gradient of x is
 * the incoming gradient itself. */
int gmoe_bias_rows(const void* x, const void* bias, int dtype, int64_t N, int64_t M,
                   const int64_t* expert_offsets, int E, void* out, void* stream);
int gmoe_bias_rows_bwd(const void* grad, int dtype, int64_t N, int64_t M,
                       const int64_t* expert_offsets, int E, void* grad_bias, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Grouped GEMM.  Replaces `grouped_gemm.ops.gmm(a, b, batch_sizes, trans_b)` (third-party
 * fanshiqing/grouped_gemm v1.1.4; call sites moe/mlp.py:106-112) and its backward.
 * expert_offsets [E+1] int64 (device) is the exclusive prefix of batch_sizes; the rows
 * [expert_offsets[e], expert_offsets[e+1]) of the row-partitioned operands belong to expert e.
 *
 *   trans_a == 0:  a [N,K], b [E,K,M] (trans_b == 0) or [E,M,K] (trans_b == 1), c [N,M]
 *                  c[rows_e] = a[rows_e] @ op(b[e])
 *   trans_a == 1:  a [N,K], b [N,M], c [E,K,M];  c[e] = a[rows_e]^T @ b[rows_e]
 *                  (zeros for an empty expert); trans_b must be 0
 * a, b in `dtype` (GMOE_BF16, GMOE_F16 or GMOE_F32), fp32 accumulation, c in `out_dtype`.
 * K and M must be multiples of 8 (16-byte rows).  One persistent kernel walks a device-side tile
 * list built from expert_offsets; no host synchronisation.
 * workspace (optional, 16-byte aligned, workspace_bytes long): scratch for fp32 partial tiles.  With
 * gmoe_gmm_workspace_bytes(...) bytes, the launch for the experts' short last row tiles (trans_b
 * with large groups) splits its reduction over otherwise idle CUs; without, it runs unsplit.  The
 * result does not depend on the contents of the workspace, only (in the last bits: another order of
 * the same fp32 additions) on whether one is given.
 */
int64_t gmoe_gmm_workspace_bytes(int E, int64_t N, int64_t K, int64_t M, int trans_a, int trans_b,
                                 int dtype);
int gmoe_gmm(const void* a, const void* b, void* c, const int64_t* expert_offsets, int E,
             int64_t N, int64_t K, int64_t M, int trans_a, int trans_b, int dtype, int out_dtype,
             void* workspace, int64_t workspace_bytes, void* stream);

/* Forward of the gated expert MLP's first half in one launch: fc1 = gmm(a, w1) with w1 [E,K,2F]
 * ([gate | up] columns, moe/mlp.py:80-95) and act_out [N,F] = act(fc1[:, :F]) * fc1[:, F:]
 * (moe/mlp.py:106-110: gmm followed by the activation closure).  fc1 [N,2F] is written too (the
 * backward needs it).  act_out is computed from fc1 as rounded to `dtype`, so it is bit-identical
 * to gmoe_gmm followed by gmoe_glu_fwd. */
int gmoe_gmm_glu(const void* a, const void* w1, void* fc1, void* act_out,
                 const int64_t* expert_offsets, int E, int64_t N, int64_t K, int64_t F, int act,
                 int dtype, void* stream);

/* Backward of the second half in one launch: d(act) = gmm(grad_out [N,K], w2 [E,F,K], trans_b) is
 * turned into grad_fc1 [N,2F] = [d * act'(gate) * up | d * act(gate)] in the GEMM's epilogue, with
 * fc1 [N,2F] read back (autograd of moe/mlp.py:110-112; formulae of
 * transformer/fused_kernels.py:157-162).  d(act) itself is not stored. */
int gmoe_gmm_glu_bwd(const void* grad_out, const void* w2, const void* fc1, void* grad_fc1,
                     const int64_t* expert_offsets, int E, int64_t N, int64_t K, int64_t F, int act,
                     int dtype, void* stream);

/* Grouped GEMM with block-scaled fp8 weights: b_q [E,K,M] (or [E,M,K] if trans_b) e4m3fn,
 * b_scale [E, ceil(K/128), ceil(M/128)] (or [E, ceil(M/128), ceil(K/128)]) bf16, one scale per
 * 128x128 tile of b_q[e].  a [N,K] bf16, c [N,M] bf16.  The fp8 values go to the matrix cores
 * widened to bf16 (exact); each 128-element block of the reduction is accumulated in fp32 and
 * its sum multiplied by the block's scale in fp32, so nothing but the output is rounded.  K and M
 * must be multiples of 16.  No counterpart in the reference (its fp8
 * expert path is commented out, moe/mlp.py:164-184). */
int gmoe_gmm_fp8w(const void* a, const void* b_q, const void* b_scale, void* c,
                  const int64_t* expert_offsets, int E, int64_t N, int64_t K, int64_t M,
                  int trans_b, void* stream);

/* fp8 on both sides, on the block-scaled fp8 MFMA of gfx950 (v_mfma_scale_f32_32x32x64_f8f6f4): no
 * counterpart in the reference (its fp8 expert path is commented out, moe/mlp.py:164-184); the
 * formats are this library's.
 *
 * gmoe_quantize_fp8_rows: x [N,K] (`dtype`) -> q [N,K] e4m3fn and scales [ceil(K/128)][N] int32,
 * one power-of-two scale 2^e per row and 128 reduction elements with the smallest e for which
 * amax * 2^-e <= 448 (e = -127 for an all-zero block), q = rne(x * 2^-e); the dword holds the E8M0
 * byte e + 127 in all four bytes.  K a multiple of 8.
 *
 * gmoe_gmm_fp8a: c[rows_e] (bf16) = deq(a_q)[rows_e] @ deq(b_q[e]) (or its transpose with
 * trans_b), the weights and their scales as for gmoe_gmm_fp8w.  Products are exact; the MFMA adds
 * 64 of them with its own internal precision (measured: within 2^-14.9 of the sum of their
 * magnitudes), everything after that is fp32: the weight scales applied to fp32 partial sums, the
 * row scales inside the MFMA (an exponent adjustment), the output rounded once.  The kernel is
 * built for few rows per expert (up to 192 rows of an expert share one pass over its weights; more
 * rows are cut into equal chunks, each of which streams the weights again).  K a multiple of 64 and
 * at most 32768, M a multiple of 16; GMOE_ERR_UNSUPPORTED otherwise. */
int gmoe_quantize_fp8_rows(const void* x, int dtype, int64_t N, int64_t K, void* q, int32_t* scales,
                           void* stream);
int gmoe_gmm_fp8a(const void* a_q, const int32_t* a_scale, const void* b_q, const void* b_scale,
                  void* c, const int64_t* expert_offsets, int E, int64_t N, int64_t K, int64_t M,
                  int trans_b, void* stream);
/* The gated activation (gmoe_glu_fwd) and its backward (gmoe_glu_bwd) with gmoe_quantize_fp8_rows
 * applied to their result in the same pass: the rows that enter the next fp8 product leave as codes
 * and scales only, bit-identical to the two launches (the result is rounded to `dtype` before it is
 * quantised, as the activation kernels store it).  Forward: y [N,2F] -> q [N,F], scales [ceil(F/128)][N],
 * F a multiple of 8.  Backward: grad_out [N,F], y [N,2F] -> q [N,2F], scales [2F/128][N], F a multiple
 * of 128; GMOE_ERR_UNSUPPORTED otherwise.  No counterpart in the reference. */
int gmoe_glu_fwd_quantize_fp8_rows(const void* y, int dtype, int64_t N, int64_t F, int act, void* q,
                                   int32_t* scales, void* stream);
int gmoe_glu_bwd_quantize_fp8_rows(const void* grad_out, const void* y, int dtype, int64_t N, int64_t F,
                                   int act, void* q, int32_t* scales, void* stream);

/* The quantiser of that format: w [batch, K, M] (dtype) -> q [batch, K, M] e4m3fn and
 * scale [batch, ceil(K/128), ceil(M/128)] bf16 with scale = bf16(amax(tile) / 448) (1 for an
 * all-zero tile) and q = round-to-nearest-even(w / scale) saturated to +-448.  M must be a multiple
 * of 8.  No counterpart in the reference. */
int gmoe_quantize_fp8_block(const void* w, int dtype, int64_t batch, int64_t K, int64_t M, void* q,
                            void* scale, void* stream);

/* The router's gate projection (Router.gating, moe/router.py:49-68:
 * logits = F.linear(input.to(router_dtype), weight.to(router_dtype))):
 *   logits[t,e] = sum_h x[t,h] * weight[e,h]        fp32 accumulation, one rounding to logits_dtype
 * x [T,H] and weight [E,H] in `dtype`; logits [T,E] in logits_dtype = dtype, or GMOE_F32 (what
 * moe_router_dtype='fp32' asks for: products of 16-bit values are exact in fp32, so the cast of the
 * operands is not materialised).  H a multiple of 8 (4 for fp32).  E <= 64 runs a dedicated
 * one-pass kernel; larger E (a multiple of 8) runs as one group on the grouped-GEMM kernels, where
 * [T,E] is only a few output tiles: with a workspace of gmoe_gate_fwd_workspace_bytes(...) bytes (0
 * for E <= 64, -1 for an unsupported shape; the workspace may be NULL) the reduction over H is spread
 * over the idle CUs in a fixed order. */
int64_t gmoe_gate_fwd_workspace_bytes(int64_t T, int64_t H, int E, int dtype);
int gmoe_gate_fwd(const void* x, const void* weight, int64_t T, int64_t H, int E, int dtype,
                  void* logits, int logits_dtype, void* workspace, int64_t workspace_bytes, void* stream);

/* Its gradients (autograd of F.linear):
 *   dx[t,h]      = sum_e dlogits[t,e] * weight[e,h]            [T,H] in `dtype`
 *   dweight[e,h] = sum_t dlogits[t,e] * x[t,h]                 [E,H] in `dtype` (zeros when T == 0)
 * dlogits [T,E] in logits_dtype.  E <= 16: dedicated one-pass kernels; larger E (a multiple of 8):
 * dense products on the grouped-GEMM kernels, an fp32 dlogits against 16-bit operands entering as the
 * sum of two 16-bit terms (exact products, fp32 sums); the weight gradient's reduction over T is cut
 * into row ranges whose fp32 partial sums are added in a fixed order.
 * gmoe_gate_bwd_input workspace: gmoe_gate_bwd_input_workspace_bytes(...) bytes (0 for E <= 16 or when
 * logits_dtype == dtype; -1 for an unsupported shape).
 * gmoe_gate_bwd_weight workspace: fp32 [workspace_rows, E*H] with workspace_rows >=
 * gmoe_gate_bwd_workspace_rows(T, H, E, dtype) (-1 for an unsupported shape); partial sums are added
 * in a fixed order. */
int64_t gmoe_gate_bwd_input_workspace_bytes(int64_t T, int64_t H, int E, int dtype, int logits_dtype);
int gmoe_gate_bwd_input(const void* dlogits, int logits_dtype, const void* weight, int64_t T, int64_t H,
                        int E, int dtype, void* dx, void* workspace, int64_t workspace_bytes,
                        void* stream);
int64_t gmoe_gate_bwd_workspace_rows(int64_t T, int64_t H, int E, int dtype);
int gmoe_gate_bwd_weight(const void* dlogits, int logits_dtype, const void* x, int64_t T, int64_t H,
                         int E, int dtype, void* dweight, float* workspace, int64_t workspace_rows,
                         void* stream);

/* RMS normalisation of rows: y = (x * rstd) * weight, rstd[t] = 1 / sqrt(mean_h(x[t,h]^2) + eps),
 * fp32 math, one rounding to `dtype`.  Replaces the RMSNorm module GalvatronNorm constructs
 * (transformer/norm.py:20-26: flash_attn.ops.rms_norm.RMSNorm, third-party flash-attn >= 2.0.8,
 * restated from its published formula) at its use as pre_router_norm
 * (models/moe_modules.py:24-30).  x, y [T,H] and weight [H] in `dtype`, rstd [T] fp32 (kept for
 * the backward).  H a multiple of 8 (4 for fp32), at most 16384 (8192 for fp32). */
int gmoe_rmsnorm_fwd(const void* x, const void* weight, int64_t T, int64_t H, float eps, int dtype,
                     void* y, float* rstd, void* stream);

/* Backward of gmoe_rmsnorm_fwd (autograd of the same module):
 *   dx[t,:] = rstd[t] * (dy*w - xhat * mean_h(dy*w*xhat)),  xhat = x * rstd[t]
 *   dweight[h] = sum_t dy[t,h] * xhat[t,h]      (written, not accumulated; zeros when T == 0)
 * dresidual (optional, [T,H] in `dtype`): the gradient that reached x along the residual branch
 * (models/moe_modules.py:27: mlp_residual = hidden_states); the kernel then writes
 * round(round(dx) + dresidual), the bits of autograd's separate add.
 * workspace: fp32 [workspace_rows, H] with workspace_rows >= gmoe_rmsnorm_bwd_workspace_rows(T, H,
 * dtype) (-1 for an unsupported shape); the partial sums are added in a fixed order. */
int64_t gmoe_rmsnorm_bwd_workspace_rows(int64_t T, int64_t H, int dtype);
int gmoe_rmsnorm_bwd(const void* dy, const void* x, const void* weight, const float* rstd,
                     const void* dresidual, int64_t T, int64_t H, int dtype, void* dx, void* dweight,
                     float* workspace, int64_t workspace_rows, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GALVATRON_MOE_H */
