/*
 * ORACLE — test infrastructure only.  Nothing in the product path may link, load
 * or call this file; only tests, the smoke check and the benchmark's cpu_baseline
 * leg do.
 *
 * Plain-C restatement (scalar, one core) of the non-GEMM operators of the
 * Optimus-LM fast MoE block, following the reference kernels loop by loop:
 *   pytorch_xpu_extensions/pcl.xpu.customops/csrc/ops/sparse_moe_block.sycl
 * and of the index bookkeeping around them in optimus/models/common/moe.py.
 * Every function cites the lines it follows.  bf16 is carried as uint16_t with
 * round-to-nearest-even conversion from float, as at::BFloat16 does.
 *
 * Floating point: compiled with -ffp-contract=off, so "a += b * c" is a rounded
 * multiply followed by a rounded add.  The reference's own contraction behaviour
 * is compiler-defined; the checks that pin these functions are listed in
 * tests/test_oracle_moe.py (closed forms, adjoint identities, brute force).
 */
#include <stdint.h>
#include <string.h>
#include <math.h>

typedef uint16_t bf16_t;

static inline float bf16_to_f32(bf16_t h) {
    uint32_t u = ((uint32_t)h) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline bf16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)0x7fc0; /* NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (bf16_t)(u >> 16);
}

/* exported for tests that want the rounding rule itself */
void orc_f32_to_bf16(const float *in, bf16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_bf16(in[i]);
}
void orc_bf16_to_f32(const bf16_t *in, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = bf16_to_f32(in[i]);
}

/* ------------------------------------------------------------------------- */
/* K1  compute_partial_token_counts        sparse_moe_block.sycl:117-135      */
/* selected_experts [T,K] int64; partial_token_counts [NR,TH] (pre-zeroed);   */
/* expert_counts_ep [T]; TB = T / TH tokens per counting thread.              */
void orc_compute_partial_token_counts(const int64_t *selected_experts,
                                      int32_t *partial_token_counts,
                                      int32_t *expert_counts_ep,
                                      int expert_start_idx, int expert_end_idx,
                                      int64_t T, int64_t K, int64_t TH) {
    int64_t TB = T / TH;
    for (int64_t tid = 0; tid < TH; tid++) {
        for (int64_t lt = 0; lt < TB; lt++) {
            int32_t expert_count = 0;
            int64_t t = tid * TB + lt;
            for (int64_t k = 0; k < K; k++) {
                int64_t n = selected_experts[t * K + k];
                if (n >= expert_start_idx && n < expert_end_idx) {
                    partial_token_counts[(n - expert_start_idx) * TH + tid] += 1;
                    expert_count += 1;
                }
            }
            expert_counts_ep[t] = expert_count;
        }
    }
}

/* K2  the two cumsums and the strided read          moe.py:513-517           */
/* partial_cum_token_counts [NR*TH+1], cum_token_counts [NR+1],               */
/* cum_expert_counts_ep [T+1]; element 0 of each scan is 0.                   */
void orc_token_count_scans(const int32_t *partial_token_counts,
                           const int32_t *expert_counts_ep,
                           int32_t *partial_cum_token_counts,
                           int32_t *cum_token_counts,
                           int32_t *cum_expert_counts_ep,
                           int64_t NR, int64_t TH, int64_t T) {
    partial_cum_token_counts[0] = 0;
    for (int64_t i = 0; i < NR * TH; i++)
        partial_cum_token_counts[i + 1] = partial_cum_token_counts[i] + partial_token_counts[i];
    for (int64_t n = 0; n <= NR; n++)
        cum_token_counts[n] = partial_cum_token_counts[n * TH];
    cum_expert_counts_ep[0] = 0;
    for (int64_t t = 0; t < T; t++)
        cum_expert_counts_ep[t + 1] = cum_expert_counts_ep[t] + expert_counts_ep[t];
}

/* K3  compute_input_and_output_indices    sparse_moe_block.sycl:188-213      */
/* input_increment_buffer [NR,TH] pre-zeroed; outputs have TR entries.        */
void orc_compute_input_and_output_indices(const int64_t *selected_experts,
                                          const int32_t *partial_cum_token_counts,
                                          int32_t *input_increment_buffer,
                                          const int32_t *cum_expert_counts_ep,
                                          int32_t *selected_experts_indices,
                                          int32_t *input_indices,
                                          int32_t *output_indices,
                                          int expert_start_idx, int expert_end_idx,
                                          int64_t T, int64_t K, int64_t TH) {
    int64_t TB = T / TH;
    for (int64_t tid = 0; tid < TH; tid++) {
        for (int64_t t = tid * TB; t < (tid + 1) * TB; t++) {
            int32_t output_index = cum_expert_counts_ep[t];
            for (int64_t k = 0; k < K; k++) {
                int64_t n = selected_experts[t * K + k];
                if (n >= expert_start_idx && n < expert_end_idx) {
                    int64_t ln = n - expert_start_idx;
                    int32_t base = partial_cum_token_counts[ln * TH + tid];
                    int32_t offset = input_increment_buffer[ln * TH + tid];
                    int32_t input_index = base + offset;
                    input_indices[input_index] = (int32_t)t;
                    input_increment_buffer[ln * TH + tid] = offset + 1;
                    output_indices[output_index] = input_index;
                    selected_experts_indices[output_index] = (int32_t)k;
                    output_index += 1;
                }
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* index_add_op                             sparse_moe_block.sycl:12-21       */
/* output[indices[c],:] += input[c,:]; applied serially in c order (the       */
/* reference kernel is racy for duplicate indices; a serial pass is the only  */
/* well-defined reading).                                                     */
void orc_index_add_f32(const float *input, float *output, const int32_t *indices,
                       int64_t C, int64_t E) {
    for (int64_t c = 0; c < C; c++)
        for (int64_t e = 0; e < E; e++)
            output[(int64_t)indices[c] * E + e] += input[c * E + e];
}
void orc_index_add_bf16(const bf16_t *input, bf16_t *output, const int32_t *indices,
                        int64_t C, int64_t E) {
    /* at::BFloat16 operator+= : float add, one rounding per update */
    for (int64_t c = 0; c < C; c++)
        for (int64_t e = 0; e < E; e++) {
            int64_t o = (int64_t)indices[c] * E + e;
            output[o] = f32_to_bf16(bf16_to_f32(output[o]) + bf16_to_f32(input[c * E + e]));
        }
}

/* K4f index_gather                         sparse_moe_block.sycl:63-72       */
void orc_index_gather_f32(const float *input, const int32_t *indices, float *output,
                          int64_t O, int64_t E) {
    for (int64_t o = 0; o < O; o++)
        memcpy(output + o * E, input + (int64_t)indices[o] * E, (size_t)E * 4);
}
void orc_index_gather_bf16(const bf16_t *input, const int32_t *indices, bf16_t *output,
                           int64_t O, int64_t E) {
    for (int64_t o = 0; o < O; o++)
        memcpy(output + o * E, input + (int64_t)indices[o] * E, (size_t)E * 2);
}

/* K4b shuffle_sub_matrix_reduce            sparse_moe_block.sycl:487-501     */
void orc_shuffle_sub_matrix_reduce_f32(const float *ggemm_input_grad,
                                       const int32_t *cum_expert_counts_ep,
                                       const int32_t *output_indices,
                                       float *hidden_states_grad, int64_t T, int64_t E) {
    for (int64_t t = 0; t < T; t++)
        for (int64_t e = 0; e < E; e++) {
            float acc = 0.0f;
            for (int32_t i = cum_expert_counts_ep[t]; i < cum_expert_counts_ep[t + 1]; i++)
                acc += ggemm_input_grad[(int64_t)output_indices[i] * E + e];
            hidden_states_grad[t * E + e] = acc;
        }
}
void orc_shuffle_sub_matrix_reduce_bf16(const bf16_t *ggemm_input_grad,
                                        const int32_t *cum_expert_counts_ep,
                                        const int32_t *output_indices,
                                        bf16_t *hidden_states_grad, int64_t T, int64_t E) {
    for (int64_t t = 0; t < T; t++)
        for (int64_t e = 0; e < E; e++) {
            float acc = 0.0f;
            for (int32_t i = cum_expert_counts_ep[t]; i < cum_expert_counts_ep[t + 1]; i++)
                acc += bf16_to_f32(ggemm_input_grad[(int64_t)output_indices[i] * E + e]);
            hidden_states_grad[t * E + e] = f32_to_bf16(acc);
        }
}

/* K6f reduce_ggemm_output                  sparse_moe_block.sycl:294-310     */
/* wdtype: routing weights are float (w_is_f32 != 0) or bf16.                 */
void orc_reduce_ggemm_output_f32(const float *ggemm_output, const float *routing_weights,
                                 const int32_t *cum_expert_counts_ep,
                                 const int32_t *selected_experts_indices,
                                 const int32_t *output_indices, float *final_hidden_states,
                                 int64_t T, int64_t K, int64_t E, int skip_weights_scaling) {
    for (int64_t t = 0; t < T; t++)
        for (int64_t e = 0; e < E; e++) {
            float acc = 0.0f;
            for (int32_t i = cum_expert_counts_ep[t]; i < cum_expert_counts_ep[t + 1]; i++) {
                int32_t k = selected_experts_indices[i];
                int32_t index = output_indices[i];
                float scaling = skip_weights_scaling ? 1.0f : routing_weights[t * K + k];
                float output = ggemm_output[(int64_t)index * E + e];
                acc += (output * scaling);
            }
            final_hidden_states[t * E + e] = acc;
        }
}
void orc_reduce_ggemm_output_bf16(const bf16_t *ggemm_output, const void *routing_weights,
                                  int w_is_f32,
                                  const int32_t *cum_expert_counts_ep,
                                  const int32_t *selected_experts_indices,
                                  const int32_t *output_indices, bf16_t *final_hidden_states,
                                  int64_t T, int64_t K, int64_t E, int skip_weights_scaling) {
    const float *wf = (const float *)routing_weights;
    const bf16_t *wb = (const bf16_t *)routing_weights;
    for (int64_t t = 0; t < T; t++)
        for (int64_t e = 0; e < E; e++) {
            float acc = 0.0f;
            for (int32_t i = cum_expert_counts_ep[t]; i < cum_expert_counts_ep[t + 1]; i++) {
                int32_t k = selected_experts_indices[i];
                int32_t index = output_indices[i];
                float scaling = skip_weights_scaling ? 1.0f
                              : (w_is_f32 ? wf[t * K + k] : bf16_to_f32(wb[t * K + k]));
                float output = bf16_to_f32(ggemm_output[(int64_t)index * E + e]);
                acc += (output * scaling);
            }
            final_hidden_states[t * E + e] = f32_to_bf16(acc);
        }
}

/* K6b reduce_ggemm_output_backward         sparse_moe_block.sycl:378-397     */
/* routing_weights_grad must be pre-zeroed by the caller (moe.py:336).        */
void orc_reduce_ggemm_output_backward_f32(const float *final_hidden_states_grad,
                                          const float *ggemm_output,
                                          const float *routing_weights,
                                          const int32_t *selected_experts_indices,
                                          const int32_t *input_indices,
                                          const int32_t *output_indices,
                                          float *ggemm_output_grad, float *routing_weights_grad,
                                          int64_t RT, int64_t K, int64_t E) {
    for (int64_t rt = 0; rt < RT; rt++) {
        int32_t index = output_indices[rt];
        int32_t t = input_indices[index];
        int32_t k = selected_experts_indices[rt];
        float weight_grad_acc = 0.0f;
        for (int64_t e = 0; e < E; e++) {
            float scaling = routing_weights[(int64_t)t * K + k];
            float output_grad = final_hidden_states_grad[(int64_t)t * E + e];
            float input = ggemm_output[(int64_t)index * E + e];
            ggemm_output_grad[(int64_t)index * E + e] = scaling * output_grad;
            weight_grad_acc += input * output_grad;
        }
        routing_weights_grad[(int64_t)t * K + k] = weight_grad_acc;
    }
}
void orc_reduce_ggemm_output_backward_bf16(const bf16_t *final_hidden_states_grad,
                                           const bf16_t *ggemm_output,
                                           const void *routing_weights, int w_is_f32,
                                           const int32_t *selected_experts_indices,
                                           const int32_t *input_indices,
                                           const int32_t *output_indices,
                                           bf16_t *ggemm_output_grad, void *routing_weights_grad,
                                           int64_t RT, int64_t K, int64_t E) {
    const float *wf = (const float *)routing_weights;
    const bf16_t *wb = (const bf16_t *)routing_weights;
    for (int64_t rt = 0; rt < RT; rt++) {
        int32_t index = output_indices[rt];
        int32_t t = input_indices[index];
        int32_t k = selected_experts_indices[rt];
        float weight_grad_acc = 0.0f;
        float scaling = w_is_f32 ? wf[(int64_t)t * K + k] : bf16_to_f32(wb[(int64_t)t * K + k]);
        for (int64_t e = 0; e < E; e++) {
            float output_grad = bf16_to_f32(final_hidden_states_grad[(int64_t)t * E + e]);
            float input = bf16_to_f32(ggemm_output[(int64_t)index * E + e]);
            ggemm_output_grad[(int64_t)index * E + e] = f32_to_bf16(scaling * output_grad);
            weight_grad_acc += input * output_grad;
        }
        if (w_is_f32) ((float *)routing_weights_grad)[(int64_t)t * K + k] = weight_grad_acc;
        else ((bf16_t *)routing_weights_grad)[(int64_t)t * K + k] = f32_to_bf16(weight_grad_acc);
    }
}

/* ------------------------------------------------------------------------- */
/* SwiGLU glue of the merged MLP            moe.py:401-402 and moe.py:37-41   */
/* h = silu(g) * u with the reference's intermediate roundings for bf16:      */
/* silu output is rounded to bf16 before the multiply (two torch ops).        */
void orc_swiglu_fwd_f32(const float *g, const float *u, float *h, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        float s = g[i] / (1.0f + expf(-g[i]));
        h[i] = s * u[i];
    }
}
void orc_swiglu_bwd_f32(const float *dh, const float *g, const float *u,
                        float *dg, float *du, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        float sig = 1.0f / (1.0f + expf(-g[i]));
        du[i] = dh[i] * (g[i] * sig);
        dg[i] = (dh[i] * u[i]) * (sig * (1.0f + g[i] * (1.0f - sig)));
    }
}
