/*
 * optimus_mi355x.h — C ABI of liboptimus_mi355x.so
 *
 * MI355X (gfx950) implementation of the single-GPU training hot path of
 * IntelLabs/Optimus-LM: the fast MoE block's operators and the flat-buffer
 * mixed-precision AdamW step.  These entry points are what a binding of the
 * reference's native-op module (pybind module `pcl_xpu_customops`,
 * pytorch_xpu_extensions/pcl.xpu.customops/csrc/ops/sparse_moe_block.sycl:538-548)
 * and of its Python-level hot loops (optimus/models/common/moe.py,
 * optimus/optimizers.py) would bind.
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer to contiguous row-major memory unless the
 *     parameter is documented as "host";
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); every call
 *     only enqueues work on it: no allocation, no host synchronisation;
 *   - the caller allocates every output and zero-fills the buffers documented as
 *     "pre-zeroed" (same ownership rule as the reference ops, moe.py:492-497, :336);
 *   - return value: OM_OK or a negative OM_ERR_* code; nothing throws.
 */
#ifndef OPTIMUS_MI355X_H
#define OPTIMUS_MI355X_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    OM_OK = 0,
    OM_ERR_NULL = -1,      /* a required pointer is NULL                        */
    OM_ERR_DTYPE = -2,     /* dtype code not supported by this entry point      */
    OM_ERR_SHAPE = -3,     /* sizes violate a documented constraint             */
    OM_ERR_ALIGN = -4,     /* pointer / row pitch not aligned as documented     */
    OM_ERR_LAUNCH = -5,    /* the HIP runtime rejected a launch                 */
    OM_ERR_WORKSPACE = -6  /* workspace too small                               */
};

/* element types */
enum { OM_F32 = 0, OM_BF16 = 1 };
/* index types of `selected_experts` (the reference dispatches kLong, else int32) */
enum { OM_I32 = 0, OM_I64 = 1 };

/* Library version and the GPU architecture the kernels were compiled for ("gfx950"). */
int om_version(void);
const char *om_arch(void);
const char *om_strerror(int code);

/* ------------------------------------------------------------------------------------
 * Flat-buffer mixed-precision AdamW step
 * replaces: the chunked 13-op elementwise sequence of MixedPrecisionAdamW.step,
 *           optimus/optimizers.py:162-205 (formula restated at optimizers.py:1745-1760).
 * One pass over n elements:  g=float(grad); m=m*b1+(1-b1)*g; v=v*b2+(1-b2)*g*g;
 *   w += -lr*(m/(1-b1^t))/(sqrt(v/(1-b2^t))+eps); if wd>0: w += (-lr*wd)*w; param=cast(w).
 * param_dtype OM_BF16: param, grad are bf16; master/exp_avg/exp_avg_sq fp32.
 * param_dtype OM_F32 : grad fp32 and `master` IS the parameter buffer; `param` is ignored
 *                      (the reference aliases them, optimizers.py:100-102).
 * `step` is t = step_id + 1 (1-based).  All five buffers must be 16-byte aligned.
 * n may exceed 2^31; beyond 2^33 elements the call makes several launches over consecutive
 * sub-ranges (element-wise work: the same bits).                                           */
int om_adamw_step(void *param, const void *grad, float *master, float *exp_avg,
                  float *exp_avg_sq, int64_t n, double lr, double beta1, double beta2,
                  double eps, double weight_decay, int64_t step, int param_dtype,
                  void *stream);

/* om_adamw_traffic_probe: the loads and stores of om_adamw_step in bf16 mode (14 B read and 14 B
 * written per element, same kernel shape and cache hints) with the arithmetic left out: master,
 * exp_avg and exp_avg_sq are written back as read and param = bf16(master), which is what the
 * optimizer keeps there anyway.  It has no counterpart in the reference; it exists so that a
 * benchmark can state what this access pattern reaches on the GPU at hand next to the update
 * itself.  n a multiple of 4 (a shorter tail is left untouched).                              */
int om_adamw_traffic_probe(void *param, const void *grad, float *master, float *exp_avg,
                           float *exp_avg_sq, int64_t n, void *stream);

/* ------------------------------------------------------------------------------------
 * Gradient norm and clip coefficient over the flat gradient buffer
 * replaces: the "4opt-step_grad-clip" block of MixedPrecisionAdamW.step,
 *           optimus/optimizers.py:136-160 — torch.nn.utils.get_total_norm (always) and
 *           clip_grad_norm_ / clip_grads_with_norm_ (max_norm 1.0, after warm-up) over the
 *           parameters' gradient views (optimizers.py:109-111 makes them slices of flat_grad).
 * The flat buffer is cut into chunks [chunk_offsets[c], chunk_offsets[c+1]) that never straddle
 * two parameters; parameter s owns chunks [seg_first_chunk[s], seg_first_chunk[s+1]).  Both
 * tables are int64 device arrays built once by the caller (any chunk length; 65536 elements is
 * a good one).
 * om_grad_sumsq: partials[c] = fp32 sum of squares of chunk c (one read of the gradients).
 * om_grad_norm_clip_coef: seg_norms[s] = sqrt(sum of its partials) rounded to the gradient
 *   dtype (what vector_norm returns for a bf16 tensor); *total_norm = norm of seg_norms, rounded
 *   likewise; if clip_coef is not null, *clip_coef = min(1, max_norm * (1/(total_norm + 1e-6)))
 *   with each intermediate rounded to the gradient dtype (torch evaluates the expression on a
 *   0-dim tensor of that dtype).  All outputs are fp32 device scalars/arrays holding those
 *   rounded values.                                                                       */
int om_grad_sumsq(const void *grad, int grad_dtype, const int64_t *chunk_offsets,
                  int64_t n_chunks, float *partials, void *stream);
int om_grad_norm_clip_coef(const float *partials, const int64_t *seg_first_chunk,
                           int64_t n_segs, int grad_dtype, double max_norm, float *seg_norms,
                           float *total_norm, float *clip_coef, void *stream);

/* om_grad_scale: grad = cast(float(grad) * *coef) in place over n elements, coef a device fp32
 * scalar (the clip_coef above): the in-place multiply of clip_grads_with_norm_
 * (optimizers.py:145/150/154) for gradient tensors that no update kernel reads (parameters of the
 * model that the optimizer does not hold, or skip_optimizer_step).  grad 16-byte aligned.       */
int om_grad_scale(void *grad, int64_t n, int grad_dtype, const float *coef, void *stream);

/* om_shard_clip_multiplier: the clip decision of the sharded optimizer's step
 * (ShardedMixedPrecisionAdamW.step, optimizers.py:398-432) on the device, so that the step never
 * reads the norm back.  mode 0 (no process group, :404-405): *value is this shard's gradient norm,
 * already rounded to the gradient dtype (om_grad_norm_clip_coef's total_norm over one segment), and
 * the coefficient max_norm / (norm + 1e-6) is evaluated with every op rounded to that dtype.
 * mode 1 (:399-403): *value is the all-reduced sum of the ranks' squared fp32 shard norms; the norm
 * and the coefficient are fp32.  *grad_norm receives the norm; *multiplier what
 * `if clip_coef < 1.0: flat_grad_shard.mul_(clip_coef)` multiplies by: the coefficient rounded to
 * the gradient dtype (the cast torch applies to a 0-dim device operand) when it is below 1, else 1.
 * Feed *multiplier to om_adamw_step_clipped / om_grad_scale.  All three are device fp32 scalars. */
int om_shard_clip_multiplier(const float *value, int mode, int grad_dtype, double max_norm,
                             float *grad_norm, float *multiplier, void *stream);

/* om_adamw_step with the clip folded in: g = cast(grad * *grad_scale) is what the update uses,
 * i.e. the in-place multiply of clip_grads_with_norm_ (optimizers.py:145/150/154) without its
 * read-modify-write pass over the gradients.  *grad_scale is a device fp32 scalar (the clip_coef
 * above).  store_scaled_grad != 0 also writes g back into `grad`, which leaves the gradient
 * buffer as the reference leaves it (+2 B/element of traffic in bf16 mode); 0 leaves `grad`
 * untouched.                                                                              */
int om_adamw_step_clipped(void *param, void *grad, float *master, float *exp_avg,
                          float *exp_avg_sq, int64_t n, double lr, double beta1, double beta2,
                          double eps, double weight_decay, int64_t step, int param_dtype,
                          const float *grad_scale, int store_scaled_grad, void *stream);

/* ------------------------------------------------------------------------------------
 * Routers
 * om_route_softmax_topk replaces optimus/models/common/moe.py:467-471
 *   (= optimus/models/olmoe/modeling_olmoe.py:295-299): fp32 softmax over N experts,
 *   top-K by (probability desc, expert index asc), optional renormalisation, cast.
 *   logits [T,N] (OM_F32 or OM_BF16); weights_out [T,K] (weights_dtype);
 *   experts_out [T,K] int64, in descending-probability order.  N <= 512, K <= min(N,64).
 * om_route_softmax_topk_bwd is the backward of the same expression (autograd in the
 *   reference): dlogits [T,N] in logits dtype from dweights [T,K].                      */
int om_route_softmax_topk(const void *logits, int logits_dtype, int64_t T, int N, int K,
                          int norm_topk_prob, void *weights_out, int weights_dtype,
                          int64_t *experts_out, void *stream);
int om_route_softmax_topk_bwd(const void *logits, int logits_dtype, const int64_t *experts,
                              const void *dweights, int weights_dtype, int64_t T, int N, int K,
                              int norm_topk_prob, void *dlogits, void *stream);

/* om_router_gate_softmax_topk is the whole OLMoE router in one launch: the gate projection
 *   router_logits = gate(hidden_states) (nn.Linear without bias), optimus/models/common/moe.py:456
 *   (= optimus/models/olmoe/modeling_olmoe.py:284), followed by :467-471 as above.
 *   x [T,H] and gate_weight [N,H] are bf16; the logits are accumulated and kept in fp32 (the value
 *   of x.float() @ gate_weight.float().T up to the order of the sum; a bf16 router rounds them to
 *   bf16 before the softmax) and written to logits_out [T,N] fp32 when it is not null (the
 *   backward and output_router_logits need them).  N <= 256, K <= min(N,64), H a multiple of 512
 *   (256 for N > 64, 64 for N > 128); other shapes return OM_ERR_SHAPE and the caller uses the
 *   two-step form (om_router_gate_logits[_split] + om_route_softmax_topk).
 * om_router_gate_logits is the projection alone, for routers that score the fp32 logits
 *   differently (optimus/models/deepseek_v3/modeling_deepseek_v3.py:160 casts both operands to
 *   float32 and calls F.linear).                                                          */
int om_router_gate_softmax_topk(const void *x, const void *gate_weight, int64_t T, int H, int N,
                                int K, int norm_topk_prob, float *logits_out, void *weights_out,
                                int weights_dtype, int64_t *experts_out, void *stream);
int om_router_gate_logits(const void *x, const void *gate_weight, int64_t T, int H, int N,
                          float *logits_out, void *stream);

/* om_router_gate_logits_split: the same projection as om_router_gate_logits for gates with many
 * experts (the DeepSeek-V3 router, 256 x 7168): 128 tokens and a slice of H per block, the weight
 * tile shared through LDS, the slices added in a fixed order.  N <= 256, H a multiple of 8 (a last
 * step with fewer than 64 columns multiplies zero-filled token fragments).
 * workspace: om_router_gate_logits_split_workspace_bytes(T,H,N) bytes, 16-byte aligned
 * (negative = error code).  Same value as om_router_gate_logits up to the order of the sum.   */
int64_t om_router_gate_logits_split_workspace_bytes(int64_t T, int H, int N);
int om_router_gate_logits_split(const void *x, const void *gate_weight, int64_t T, int H, int N,
                                float *logits_out, void *workspace, int64_t workspace_bytes,
                                void *stream);

/* om_router_gate_wgrad: gradient of the gate's weight,
 *   dweight[n,h] = sum_t dlogits[t,n] * x[t,h]
 * i.e. what autograd computes for the nn.Linear behind `router_logits = self.gate(hidden_states)`
 * (optimus/models/common/moe.py:456, optimus/models/olmoe/modeling_olmoe.py:284) from the
 * gradient of the logits.  x [T,H] bf16; dlogits [T,N] fp32, rounded to bf16 as it is loaded;
 * products accumulate in fp32 over token ranges and the partial sums are added in a fixed order
 * (deterministic).  dweight [N,H] in dweight_dtype (OM_BF16 / OM_F32).  N <= 256, H a multiple
 * of 8; other shapes return OM_ERR_SHAPE.
 * workspace: om_router_gate_wgrad_workspace_bytes(T,H,N) bytes of device memory, 16-byte
 * aligned (negative = error code).                                                        */
int64_t om_router_gate_wgrad_workspace_bytes(int64_t T, int H, int N);
int om_router_gate_wgrad(const void *x, const float *dlogits, int64_t T, int H, int N,
                         void *dweight, int dweight_dtype, void *workspace,
                         int64_t workspace_bytes, void *stream);

/* The gate projection of a float32 module and its backward, replacing the nn.Linear behind
 * `router_logits = self.gate(hidden_states)` (optimus/models/common/moe.py:456) where the block is
 * kept in float32 (the reference's small CPU-runnable configuration): plain float32 products,
 * sums in a fixed order (the weight gradient's sum over the tokens is kept in double and rounded
 * once).  Any T, H, N <= 65535.  Parity path, not tuned.
 *   om_router_gate_logits_f32 : logits[t,n]  = sum_h x[t,h] * gate_weight[n,h]
 *   om_router_gate_dgrad_f32  : dx[t,h]      = sum_n dlogits[t,n] * gate_weight[n,h]
 *   om_router_gate_wgrad_f32  : dweight[n,h] = sum_t dlogits[t,n] * x[t,h]                       */
int om_router_gate_logits_f32(const float *x, const float *gate_weight, int64_t T, int H, int N,
                              float *logits_out, void *stream);
int om_router_gate_dgrad_f32(const float *dlogits, const float *gate_weight, int64_t T, int H, int N,
                             float *dx, void *stream);
int om_router_gate_wgrad_f32(const float *x, const float *dlogits, int64_t T, int H, int N,
                             float *dweight, void *stream);

/* om_router_gate_dgrad: gradient of the gate's input,
 *   dx[t,h] = (base[t,h] +) sum_n bf16(dlogits[t,n]) * gate_weight[n,h]
 * what autograd computes for the same nn.Linear (mm(dlogits, weight)), optionally with the
 * accumulation into the tensor's other gradient folded in: `base` [T,H] bf16 (may be null, may be
 * dx itself) is the gradient that reached hidden_states through the experts, and
 * dx = bf16(float(base) + float(bf16(sum))) keeps both roundings of "matmul, then add".
 * dlogits [T,N] fp32 (rounded to bf16 as it is loaded), gate_weight [N,H] bf16, dx [T,H] bf16.
 * N <= 256, H a multiple of 8; other shapes return OM_ERR_SHAPE.                             */
int om_router_gate_dgrad(const float *dlogits, const void *gate_weight, const void *base, void *dx,
                         int64_t T, int H, int N, void *stream);

/* Load-balancing statistics of one layer's router logits
 * replaces: the per-token part of load_balancing_loss_func,
 *   optimus/models/olmoe/modeling_olmoe.py:44-57 (softmax, top-K, one-hot mean, probability
 *   mean), and of single_input_/layer_level_load_balancing_loss_func,
 *   optimus/models/common/ral_functions.py:6-35.
 * prob_sum[e] = sum over tokens of softmax(logits[t,:])[e] (fp32);
 * count[e]    = number of tokens whose top-K (probability desc, expert index asc) holds e, as float.
 * The loss is num_experts * sum_e (count[e]/T) * (prob_sum[e]/T); the means and the product are
 * left to the caller, who may combine several layers.  workspace: om_router_balance_workspace_bytes.
 * om_router_balance_bwd: dlogits[t,i] = p_i * (g_i - sum_j p_j g_j) with g = prob_grad [N] fp32,
 *   the gradient of the loss with respect to prob_sum (the counts carry no gradient).      */
int64_t om_router_balance_workspace_bytes(int64_t T, int N);
/* The *_masked forms take the attention mask of the same function
 * (optimus/models/olmoe/modeling_olmoe.py:58-83) as one weight per token, token_weight [T] fp32
 * (the mask entry of the token's batch row and position; null = every token counts once):
 *   prob_sum[e] = sum_t token_weight[t] * softmax(logits[t,:])[e]
 *   count[e]    = sum_t token_weight[t] * [e in top-K of token t]
 * and dlogits[t,i] = token_weight[t] * p_i * (g_i - sum_j p_j g_j) backward.  The caller divides by
 * the sum of the weights (all layers share one mask).                                          */
int om_router_balance_stats_masked(const void *logits, int logits_dtype, const float *token_weight,
                                   int64_t T, int N, int K, float *prob_sum, float *count,
                                   void *workspace, int64_t workspace_bytes, void *stream);
int om_router_balance_bwd_masked(const void *logits, int logits_dtype, const float *prob_grad,
                                 const float *token_weight, int64_t T, int N, void *dlogits,
                                 void *stream);
int om_router_balance_stats(const void *logits, int logits_dtype, int64_t T, int N, int K,
                            float *prob_sum, float *count, void *workspace,
                            int64_t workspace_bytes, void *stream);
int om_router_balance_bwd(const void *logits, int logits_dtype, const float *prob_grad, int64_t T,
                          int N, void *dlogits, void *stream);

/* om_route_sigmoid_group_topk replaces DeepseekV3ParallelTopkRouter.get_topk_indices and
 *   the weight computation of its forward,
 *   optimus/models/deepseek_v3/modeling_deepseek_v3.py:164-180 and :185-191:
 *   scores = sigmoid(logits); choice = scores + bias; group score = sum of the top-2 choice
 *   values of each of n_group contiguous groups; the topk_group best groups keep their
 *   choice values, all others become 0.0; experts = top-K of that; weights = scores at the
 *   experts, divided by (sum + 1e-20) when norm_topk_prob, times routed_scaling_factor.
 *   logits [T,N] fp32, bias [N] fp32 -> experts_out [T,K] int64 (descending choice value,
 *   lower index first among equals), weights_out [T,K] fp32.  N <= 512, N % n_group == 0.
 * om_route_sigmoid_topk_bwd: dlogits [T,N] fp32 (dense, zero off the selected experts).   */
int om_route_sigmoid_group_topk(const float *logits, const float *bias, int64_t T, int N,
                                int n_group, int topk_group, int K, int norm_topk_prob,
                                double routed_scaling_factor, int64_t *experts_out,
                                float *weights_out, void *stream);
int om_route_sigmoid_topk_bwd(const float *logits, const int64_t *experts, const float *dweights,
                              int64_t T, int N, int K, int norm_topk_prob,
                              double routed_scaling_factor, float *dlogits, void *stream);

/* ------------------------------------------------------------------------------------
 * Token permutation (index construction)
 * om_moe_sort fuses the reference's K1 + K2 + K3:
 *   compute_partial_token_counts      sparse_moe_block.sycl:108-173
 *   the two cumsums and the host read moe.py:513-520
 *   compute_input_and_output_indices  sparse_moe_block.sycl:175-280
 * into a stable counting sort of the (token, k) pairs whose expert lies in
 * [expert_start_idx, expert_end_idx).  Results are identical to the reference's:
 *   cum_token_counts [NR+1], cum_expert_counts_ep [T+1], and — for the TR =
 *   cum_token_counts[NR] routed rows — input_indices, output_indices,
 *   selected_experts_indices (each with room for T*K entries; entries >= TR are set to -1 in
 *   output_indices and to 0 in the other two, so a caller that sizes the work that follows by
 *   T*K instead of reading TR back can recognise them: om_moe_row_weights and
 *   om_moe_row_weights_grad skip them, the expert GEMMs and the per-token sums only ever read
 *   entries below TR).
 * All outputs stay on the device; nothing is read back.
 * workspace: om_moe_sort_workspace_bytes(T, K, NR) bytes, 4-byte aligned, no pre-zeroing. */
int64_t om_moe_sort_workspace_bytes(int64_t T, int K, int NR);
int om_moe_sort(const void *selected_experts, int index_dtype, int64_t T, int K,
                int expert_start_idx, int expert_end_idx, int32_t *cum_token_counts,
                int32_t *cum_expert_counts_ep, int32_t *input_indices, int32_t *output_indices,
                int32_t *selected_experts_indices, void *workspace, int64_t workspace_bytes,
                void *stream);

/* om_moe_sort_static: om_moe_sort without a workspace argument and without any allocation.  It has
 * no counterpart in the reference; it is for callers that cannot allocate device memory or carry a
 * workspace around: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  The block table that om_moe_sort keeps in the caller's workspace lives in a fixed
 * array of om_moe_sort_static_capacity_bytes() (4 MiB) inside the library, one copy per GPU, held
 * until the process ends.  Inputs whose om_moe_sort_workspace_bytes(T, K, NR) exceeds that capacity
 * return OM_ERR_WORKSPACE (4 MiB serves e.g. 8M pairs over 256 local experts).  Same results as
 * om_moe_sort, bit for bit.  The array is shared by every call on a GPU: calls that overlap on one
 * GPU (two streams, two threads) race; calls on one stream are ordered and safe.  Nothing in the
 * array needs to start at zero.  The array's address is looked up on the first call on a device,
 * for the device that is current in the calling thread: make that first call outside any graph
 * capture, with the device of the pointers and of the stream current (as for every entry point
 * here).                                                                                     */
int64_t om_moe_sort_static_capacity_bytes(void);
int om_moe_sort_static(const void *selected_experts, int index_dtype, int64_t T, int K,
                       int expert_start_idx, int expert_end_idx, int32_t *cum_token_counts,
                       int32_t *cum_expert_counts_ep, int32_t *input_indices, int32_t *output_indices,
                       int32_t *selected_experts_indices, void *stream);

/* The reference's two index kernels with their own table layout, for callers of the
 * pybind module that still run K2 (torch.cumsum) themselves.
 * replaces: compute_partial_token_counts      sparse_moe_block.sycl:138-173
 *           compute_input_and_output_indices  sparse_moe_block.sycl:217-280
 * partial_token_counts [NR,TH] and input_increment_buffer [NR,TH] are pre-zeroed by the
 * caller and updated in place; TB = T / TH tokens per table column (T % TH == 0, any TB; the
 * reference fixes TB = 8).  One wavefront per column; NR <= 1024.                           */
int om_compute_partial_token_counts(const void *selected_experts, int index_dtype,
                                    int32_t *partial_token_counts, int32_t *expert_counts_ep,
                                    int expert_start_idx, int expert_end_idx, int64_t T, int K,
                                    int64_t TH, void *stream);
int om_compute_input_and_output_indices(const void *selected_experts, int index_dtype,
                                        const int32_t *partial_cum_token_counts,
                                        int32_t *input_increment_buffer,
                                        const int32_t *cum_expert_counts_ep,
                                        int32_t *selected_experts_indices, int32_t *input_indices,
                                        int32_t *output_indices, int expert_start_idx,
                                        int expert_end_idx, int64_t T, int K, int64_t TH,
                                        void *stream);

/* ------------------------------------------------------------------------------------
 * Row movers (dtype OM_F32 or OM_BF16 for the activations; fp32 accumulation, one rounding)
 * om_index_add                    replaces index_add_op      sparse_moe_block.sycl:24-54
 *     output[indices[c],:] += input[c,:]   (atomic per element: duplicates are summed)
 * om_index_gather                 replaces index_gather      sparse_moe_block.sycl:75-106
 *     output[o,:] = input[indices[o],:]
 * om_shuffle_sub_matrix_reduce    replaces shuffle_sub_matrix_reduce   .sycl:505-532
 *     hidden_grad[t,:] = sum_{i in [cum_ep[t],cum_ep[t+1])} ggemm_input_grad[output_indices[i],:]
 * om_reduce_ggemm_output          replaces reduce_ggemm_output         .sycl:314-362
 *     final[t,:] = sum_i w[t, sel_idx[i]] * ggemm_output[output_indices[i],:]
 *     (weights_dtype may be OM_F32 while dtype is OM_BF16: the DeepSeek-V3 block keeps its
 *      routing weights in fp32, modeling_deepseek_v3.py:222-239)
 * om_reduce_ggemm_output_backward replaces reduce_ggemm_output_backward .sycl:425-475
 *     dy[pos,:] = w[t,k] * dout[t,:];  dw[t,k] = <y[pos,:], dout[t,:]>;  dw pre-zeroed.      */
int om_index_add(const void *input, void *output, const int32_t *indices, int64_t C, int64_t E,
                 int dtype, void *stream);
int om_index_gather(const void *input, const int32_t *indices, void *output, int64_t O,
                    int64_t E, int dtype, void *stream);
int om_shuffle_sub_matrix_reduce(const void *ggemm_input_grad, const int32_t *cum_expert_counts_ep,
                                 const int32_t *output_indices, void *hidden_states_grad,
                                 int64_t T, int64_t E, int dtype, void *stream);
int om_reduce_ggemm_output(const void *ggemm_output, const void *routing_weights,
                           const int32_t *cum_expert_counts_ep,
                           const int32_t *selected_experts_indices, const int32_t *output_indices,
                           void *final_hidden_states, int64_t T, int K, int64_t E, int dtype,
                           int weights_dtype, int skip_weights_scaling, void *stream);
/* om_reduce_ggemm_output_residual: the combine with the addition that follows it in the callers
 * folded in,
 *   final[t,:] = residual[t,:] + round(sum_i w * ggemm_output[...])     (sum rounded to `dtype` first,
 * so the two roundings of the reference's two steps are both there): the decoder layer's
 *   hidden_states = residual + hidden_states     (optimus/models/olmoe/modeling_olmoe.py:415)
 * and the DeepSeek-V3 block's routed + shared-expert sum (modeling_deepseek_v3.py:265).
 * residual [T,E] of `dtype`; may alias nothing else.                                          */
int om_reduce_ggemm_output_residual(const void *ggemm_output, const void *routing_weights,
                                    const int32_t *cum_expert_counts_ep,
                                    const int32_t *selected_experts_indices,
                                    const int32_t *output_indices, const void *residual,
                                    void *final_hidden_states, int64_t T, int K, int64_t E,
                                    int dtype, int weights_dtype, void *stream);
int om_reduce_ggemm_output_backward(const void *final_hidden_states_grad, const void *ggemm_output,
                                    const void *routing_weights,
                                    const int32_t *selected_experts_indices,
                                    const int32_t *input_indices, const int32_t *output_indices,
                                    void *ggemm_output_grad, void *routing_weights_grad,
                                    int64_t RT, int K, int64_t E, int dtype, int weights_dtype,
                                    void *stream);

/* ------------------------------------------------------------------------------------
 * RMSNorm either side of the MoE block, optionally fused with the residual add before it
 * replaces: OlmoeParallelRMSNorm.forward, optimus/models/olmoe/modeling_olmoe.py:98-104
 *   (= DeepseekV3ParallelRMSNorm.forward, optimus/models/deepseek_v3/modeling_deepseek_v3.py:35-40)
 *   and, with `residual`, the add of the decoder layer body in front of it (modeling_olmoe.py:402,
 *   :405-409): h = x + residual (rounded to the model dtype); r = rsqrt(mean(float(h)^2) + eps);
 *   out = weight * cast(float(h) * r).  residual, h_out and rstd_out may be NULL (h_out receives h,
 *   the next residual; rstd_out [rows] fp32 is what the backward needs).  x, residual, weight,
 *   out, h_out share `dtype`; E a multiple of 8 (bf16) / 4 (fp32); rows of any length.
 * om_rmsnorm_bwd: dx [rows,E] = r * (g*w - xn * mean(g*w*xn)), xn = float(h)*r, g = dy, and
 *   dweight [E] = sum_rows dy * cast(xn) (fp32 accumulation, deterministic order), from h (the
 *   tensor that was normalised) and rstd.  workspace: om_rmsnorm_bwd_workspace_bytes.        */
int om_rmsnorm_fwd(const void *x, const void *residual, const void *weight, double eps, void *out,
                   void *h_out, float *rstd_out, int64_t rows, int64_t E, int dtype, void *stream);
int64_t om_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t E);
int om_rmsnorm_bwd(const void *dy, const void *h, const void *weight, const float *rstd, void *dx,
                   void *dweight, void *workspace, int64_t workspace_bytes, int64_t rows, int64_t E,
                   int dtype, void *stream);

/* ------------------------------------------------------------------------------------
 * Grouped expert GEMMs (bf16 operands, fp32 MFMA accumulation, bf16 results)
 * The G experts own the row segments [cum_token_counts[g], cum_token_counts[g+1]) of the
 * activation matrices; cum_token_counts [G+1] is a DEVICE int32 array (no host copy, no
 * max_tokens_per_expert: the kernels size their work from `rows`, an upper bound on
 * cum_token_counts[G] known to the host, e.g. the allocated row count).
 * replaces GroupedGemmFunction, optimus/models/common/moe.py:163-215, whose tiling
 * specification is optimus/kernels/merged_mlp_triton_kernels.py:8-269:
 *   om_grouped_gemm_fwd    out[s:e,:]  = in[s:e,:]   @ W[g].T      (W [G,N,K] "out,in")
 *   om_grouped_gemm_dgrad  din[s:e,:]  = dout[s:e,:] @ W[g]
 *   om_grouped_gemm_wgrad  dW[g]       = dout[s:e,:].T @ in[s:e,:]  (zeros when s == e)
 * w_stride: elements between the matrices of consecutive experts in `weight` /
 * `weight_grad`; 0 means densely packed (N*K, the merged [G,N,K] layout).  A larger stride
 * serves per-expert nn.Linear weights that sit at a constant pitch inside one flat buffer
 * (a multiple of 8 elements, else OM_ERR_ALIGN).  N and K must be multiples of 8, the size of a
 * 16-byte vector (the 256x256 tile serves extents that are multiples of 256 with a contraction that
 * is a multiple of 128; the 128x128 tile everything else, with a partial last tile where an extent
 * is not a multiple of 128 and a zero-filled last contraction step where the contraction length is
 * not a multiple of 64).
 * Tensors
 * may exceed 2^31 elements (64-bit block-uniform bases, 32-bit offsets inside a tile); only a
 * source whose rows are fetched through an index (the *_gathered / *_weighted forms below) must
 * span fewer than 2^31 elements, e.g. 1M tokens of 2048.  fwd and dgrad (and the merged-MLP fusions below) keep
 * a per-expert tile table in LDS and take G <= 1024 (OM_ERR_SHAPE above that); wgrad has no
 * such limit.                                                                             */
int om_grouped_gemm_fwd(const void *input, const void *weight, void *output,
                        const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                        int64_t w_stride, void *stream);
int om_grouped_gemm_dgrad(const void *output_grad, const void *weight, void *input_grad,
                          const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                          int64_t w_stride, void *stream);
int om_grouped_gemm_wgrad(const void *output_grad, const void *input, void *weight_grad,
                          const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                          int64_t w_stride, void *stream);

/* The same three products for float32 modules (GroupedGemmFunction runs in the module's dtype,
 * moe.py:174-178, :201-210; the reference's small CPU-runnable configuration is float32): fp32
 * operands, fp32 MFMA accumulation, fp32 results.  N and K multiples of 8, w_stride a multiple
 * of 4.  Built for parity at fp32 accuracy, not tuned.                                       */
int om_grouped_gemm_fwd_f32(const float *input, const float *weight, float *output,
                            const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                            int64_t w_stride, void *stream);
int om_grouped_gemm_dgrad_f32(const float *output_grad, const float *weight, float *input_grad,
                              const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                              int64_t w_stride, void *stream);
int om_grouped_gemm_wgrad_f32(const float *output_grad, const float *input, float *weight_grad,
                              const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                              int64_t w_stride, void *stream);

/* Merged-MLP fusions, replacing the three GroupedGemmFunction calls and the two torch
 * elementwise ops of MergedMLP.forward (moe.py:396-405) and their autograd backward:
 *   om_merged_mlp_gate_up_fwd : g = x@Wg[e].T, u = x@Wu[e].T, h = silu(g)*u in one kernel
 *                               (x [rows,H]; Wg,Wu [G,I,H]; g,u,h [rows,I])
 *   om_merged_mlp_down_dgrad  : dh = dy@Wd[e] fused with the SwiGLU backward
 *                               du = dh*silu(g), dg = dh*u*sig(g)*(1+g*(1-sig(g)))
 *                               (dy [rows,H]; Wd [G,H,I]; g,u in; dg,du out [rows,I])
 *   om_merged_mlp_gate_up_dgrad: dx = dg@Wg[e] + du@Wu[e] with one accumulator.
 * Weight gradients use om_grouped_gemm_wgrad.                                             */
int om_merged_mlp_gate_up_fwd(const void *x, const void *w_gate, const void *w_up, void *g,
                              void *u, void *h, const int32_t *cum_token_counts, int64_t rows,
                              int G, int I, int H, int64_t w_stride, void *stream);
int om_merged_mlp_down_dgrad(const void *dy, const void *w_down, const void *g, const void *u,
                             void *dg, void *du, const int32_t *cum_token_counts, int64_t rows,
                             int G, int I, int H, int64_t w_stride, void *stream);
int om_merged_mlp_gate_up_dgrad(const void *dg, const void *du, const void *w_gate,
                                const void *w_up, void *dx, const int32_t *cum_token_counts,
                                int64_t rows, int G, int I, int H, int64_t w_stride,
                                void *stream);

/* The token gather folded into the GEMMs' operand loads: K4's
 *   ggemm_input = hidden_states[input_indices]        (PrepareInputForGroupGemmFunction.forward,
 *   optimus/models/common/moe.py:217-237; index_gather, sparse_moe_block.sycl:56-106)
 * is never materialised.  The kernels read row input_indices[r] of hidden_states [src_rows, H]
 * wherever the plain entry points read row r of ggemm_input [rows, H]; the arithmetic, and so
 * every output bit, is the same as index_gather followed by the plain entry point.
 *   om_merged_mlp_gate_up_fwd_gathered : as om_merged_mlp_gate_up_fwd with x = hidden_states,
 *                                        x_rows = input_indices [rows] int32 (device)
 *   om_grouped_gemm_wgrad_gathered     : as om_grouped_gemm_wgrad with input = hidden_states
 *                                        [src_rows, K], input_rows = input_indices [rows]
 *                                        (dW_gate = dg.T @ x[input_indices], same for up)
 * Indices must lie in [0, src_rows); they are not checked on the device.                   */
int om_merged_mlp_gate_up_fwd_gathered(const void *x, const int32_t *x_rows, int64_t src_rows,
                                       const void *w_gate, const void *w_up, void *g, void *u,
                                       void *h, const int32_t *cum_token_counts, int64_t rows,
                                       int G, int I, int H, int64_t w_stride, void *stream);
int om_grouped_gemm_wgrad_gathered(const void *output_grad, const void *input,
                                   const int32_t *input_rows, int64_t src_rows, void *weight_grad,
                                   const int32_t *cum_token_counts, int64_t rows, int G, int N,
                                   int K, int64_t w_stride, void *stream);

/* The combine's routing weight folded into the expert MLP.  The reference multiplies by w[t,k]
 * when it sums the experts' outputs (GroupGemmOutputReductionFunction, optimus/models/common/
 * moe.py:284-377) and its reduce_ggemm_output kernel already has a skip_weights_scaling switch
 * for rows that arrive scaled (sparse_moe_block.sycl:292-303).  Since the down projection is linear,
 *   w * ((silu(g) * u) @ Wd.T) = ((w * silu(g) * u) @ Wd.T),
 * the weight can be applied where h is formed, and in the backward pass the [rows, H] gradient of
 * the experts' output, w[t,k] * dfinal[t,:], never has to be written: the down projection's two
 * backward GEMMs read dfinal through input_indices, and the SwiGLU-backward epilogue applies w and
 * forms the routing weights' gradient.  Same mathematics as the reference's sequence; the bf16
 * roundings fall in different places (h is rounded after the weight, not before), so results agree
 * with the two-step form to bf16 accuracy, not bit for bit.
 *   om_moe_row_weights       : row_weights[pos] = w[t,k] for every routed entry rt (pos =
 *                              output_indices[rt], t = input_indices[pos], k = sel_idx[rt]); fp32 [RT];
 *                              RT may be an upper bound of the routed entries (T*K) when the index
 *                              arrays come from om_moe_sort: entries with pos < 0 are skipped
 *   om_merged_mlp_gate_up_fwd_weighted : as ..._gate_up_fwd_gathered, h = bf16(row_weights[r] *
 *                              silu(g) * u) (g and u are stored unweighted)
 *   om_sum_ggemm_output      : final[t,:] = (residual[t,:] +) bf16(sum of the token's rows), no weights;
 *                              residual may be null
 *   om_grouped_gemm_wgrad_gathered_out : as om_grouped_gemm_wgrad with output_grad = dfinal
 *                              [src_rows, N] read through output_grad_rows = input_indices [rows]
 *   om_merged_mlp_down_dgrad_weighted  : dh' = dfinal[dy_rows[r]] @ Wd[e];
 *                              row_dot[part][r] = sum over the part's 64 columns of dh' * silu(g) * u
 *                              (parts = om_merged_mlp_row_dot_parts(I) = ceil(I / 64), fp32 [parts, rows]);
 *                              then as om_merged_mlp_down_dgrad with dh = row_weights[r] * dh'
 *   om_moe_row_weights_grad  : dw[t,k] = sum over parts (in order) of row_dot[part][pos]; entries of
 *                              pairs outside the expert window are not written (pre-zero them)   */
int om_moe_row_weights(const void *routing_weights, const int32_t *selected_experts_indices,
                       const int32_t *input_indices, const int32_t *output_indices,
                       float *row_weights, int64_t RT, int K, int weights_dtype, void *stream);
int om_merged_mlp_gate_up_fwd_weighted(const void *x, const int32_t *x_rows, int64_t src_rows,
                                       const void *w_gate, const void *w_up, const float *row_weights,
                                       void *g, void *u, void *h, const int32_t *cum_token_counts,
                                       int64_t rows, int G, int I, int H, int64_t w_stride,
                                       void *stream);
int om_sum_ggemm_output(const void *ggemm_output, const int32_t *cum_expert_counts_ep,
                        const int32_t *output_indices, const void *residual,
                        void *final_hidden_states, int64_t T, int64_t E, int dtype, void *stream);
int om_grouped_gemm_wgrad_gathered_out(const void *output_grad, const int32_t *output_grad_rows,
                                       int64_t src_rows, const void *input, void *weight_grad,
                                       const int32_t *cum_token_counts, int64_t rows, int G, int N,
                                       int K, int64_t w_stride, void *stream);
int om_merged_mlp_row_dot_parts(int I);
int om_merged_mlp_down_dgrad_weighted(const void *dy, const int32_t *dy_rows, int64_t src_rows,
                                      const void *w_down, const void *g, const void *u,
                                      const float *row_weights, void *dg, void *du, float *row_dot,
                                      const int32_t *cum_token_counts, int64_t rows, int G, int I,
                                      int H, int64_t w_stride, void *stream);
int om_moe_row_weights_grad(const float *row_dot, int parts, const int32_t *selected_experts_indices,
                            const int32_t *input_indices, const int32_t *output_indices,
                            void *routing_weights_grad, int64_t RT, int K, int weights_dtype,
                            void *stream);

/* Weight gradients added to a gradient buffer in place.  In the reference's training set-up every
 * p.grad is a view of the optimizer's flat gradient buffer (optimus/optimizers.py:105-111) that is
 * zeroed in place (:117-118), and micro-batches accumulate into it (dist_train.py:154): autograd
 * ends every weight-gradient GEMM with `p.grad += dW`.  These forms do that sum in the GEMM's
 * epilogue:  weight_grad = cast(float(weight_grad) + float(cast(dW)))  in the gradient's dtype,
 * the bits of the in-place add on a freshly rounded dW, without dW being written or re-read.
 * Arguments as the entry points of the same name without the suffix; weight_grad is read and
 * written (every element, also those of experts without rows).                               */
int om_grouped_gemm_wgrad_accumulate(const void *output_grad, const void *input, void *weight_grad,
                                     const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                     int64_t w_stride, void *stream);
int om_grouped_gemm_wgrad_gathered_accumulate(const void *output_grad, const void *input,
                                              const int32_t *input_rows, int64_t src_rows,
                                              void *weight_grad, const int32_t *cum_token_counts,
                                              int64_t rows, int G, int N, int K, int64_t w_stride,
                                              void *stream);
int om_grouped_gemm_wgrad_gathered_out_accumulate(const void *output_grad, const int32_t *output_grad_rows,
                                                  int64_t src_rows, const void *input, void *weight_grad,
                                                  const int32_t *cum_token_counts, int64_t rows, int G,
                                                  int N, int K, int64_t w_stride, void *stream);
int om_grouped_gemm_wgrad_f32_accumulate(const float *output_grad, const float *input, float *weight_grad,
                                         const int32_t *cum_token_counts, int64_t rows, int G, int N,
                                         int K, int64_t w_stride, void *stream);

/* Stand-alone SwiGLU glue (moe.py:401-402 forward; moe.py:37-41 and :133-147 backward),
 * for callers that keep the three GEMMs separate.  n elements, dtype OM_F32 or OM_BF16.   */
int om_swiglu_fwd(const void *g, const void *u, void *h, int64_t n, int dtype, void *stream);
int om_swiglu_bwd(const void *dh, const void *g, const void *u, void *dg, void *du, int64_t n,
                  int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* OPTIMUS_MI355X_H */
