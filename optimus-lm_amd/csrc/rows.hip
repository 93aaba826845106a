// Row movers of the fast MoE block: gather, scatter-reduce, weighted combine and its backward,
// index_add.  All are HBM-bound; one wavefront streams a row with 16-byte accesses, fp32
// accumulation in the reference's summation order, one rounding per output element.
#include "common.h"

namespace {

#pragma clang fp contract(off)

constexpr int ROWS_PER_BLOCK = 4;  // 4 wavefronts per block, one row each

// output[o,:] = input[indices[o],:]
template <typename T>
__global__ __launch_bounds__(256) void index_gather_kernel(const T *__restrict__ input,
                                                           const int32_t *__restrict__ indices,
                                                           T *__restrict__ output, int64_t O,
                                                           int64_t E, bool vec_ok) {
    const int lane = threadIdx.x & 63;
    const int64_t o = static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK + (threadIdx.x >> 6);
    if (o >= O) return;
    const T *src = input + static_cast<int64_t>(indices[o]) * E;
    T *dst = output + o * E;
    if (vec_ok) {
        const int64_t nv = E / Elem<T>::VEC;
        const u32x4 *s4 = reinterpret_cast<const u32x4 *>(src);
        u32x4 *d4 = reinterpret_cast<u32x4 *>(dst);
        for (int64_t i = lane; i < nv; i += 64) d4[i] = s4[i];
    } else {
        for (int64_t i = lane; i < E; i += 64) dst[i] = src[i];
    }
}

// out = residual + round_to_T(sum): the two roundings of `residual + moe_output` on tensors of type T
template <typename T> __device__ __forceinline__ float round_as(float x);
template <> __device__ __forceinline__ float round_as<float>(float x) { return x; }
template <> __device__ __forceinline__ float round_as<uint16_t>(float x) {
    return bf16_bits_to_f32(f32_to_bf16_bits(x));
}

// hidden_grad[t,:] = sum_i ggemm_input_grad[output_indices[i],:],  i in [cum_ep[t], cum_ep[t+1])
// SCALE: final[t,:] = sum_i w[t, sel_idx[i]] * y[output_indices[i],:]
// residual != null: final[t,:] = residual[t,:] + T(that sum), the sum rounded to T first
template <typename T, typename TW, bool SCALE>
__global__ __launch_bounds__(256) void token_reduce_kernel(
    const T *__restrict__ rows, const TW *__restrict__ routing_weights,
    const int32_t *__restrict__ cum_expert_counts_ep,
    const int32_t *__restrict__ selected_experts_indices,
    const int32_t *__restrict__ output_indices, T *__restrict__ out, int64_t T_tokens, int K,
    int64_t E, bool vec_ok, const T *__restrict__ residual = nullptr) {
    const int lane = threadIdx.x & 63;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK + (threadIdx.x >> 6);
    if (t >= T_tokens) return;
    const int32_t i0 = cum_expert_counts_ep[t], i1 = cum_expert_counts_ep[t + 1];
    T *dst = out + t * E;
    const T *res = residual ? residual + t * E : nullptr;
    constexpr int V = Elem<T>::VEC;
    if (vec_ok) {
        // The token's row numbers and weights are fetched once, 64 at a time, one per lane, and
        // handed round with lane reads: the row loads then depend on no other load, and the four
        // column chunks a lane owns (4 KB of a row per pass) are in flight together.
        // Rows and result stream past the caches (nontemporal): measured 121 -> 99 us for 131072 rows
        // of 2048 bf16 (5.0 -> 6.1 TB/s); single-wavefront blocks or fewer resident wavefronts, which
        // help the AdamW streams, change nothing here.
        constexpr int CH = 4;
        const int64_t nv = E / V;
        for (int64_t c0 = 0; c0 < nv; c0 += 64 * CH) {
            float acc[CH][V];
#pragma unroll
            for (int u = 0; u < CH; u++)
#pragma unroll
                for (int j = 0; j < V; j++) acc[u][j] = 0.0f;
            for (int32_t ib = i0; ib < i1; ib += 64) {
                const int32_t n = min(64, i1 - ib);
                int32_t my_index = 0;
                float my_scale = 1.0f;
                if (lane < n) {
                    my_index = output_indices[ib + lane];
                    if (SCALE) my_scale = Elem<TW>::load(routing_weights + t * K + selected_experts_indices[ib + lane]);
                }
                for (int32_t i = 0; i < n; i++) {
                    const int32_t index = __shfl(my_index, i, 64);
                    const float scaling = __shfl(my_scale, i, 64);
                    const u32x4 *src = reinterpret_cast<const u32x4 *>(rows + static_cast<int64_t>(index) * E);
                    u32x4 q[CH];
#pragma unroll
                    for (int u = 0; u < CH; u++) {
                        const int64_t c = c0 + u * 64 + lane;
                        if (c < nv) q[u] = __builtin_nontemporal_load(src + c);   // every row is read once
                    }
#pragma unroll
                    for (int u = 0; u < CH; u++) {
                        if (c0 + u * 64 + lane < nv) {
                            float f[V];
                            Elem<T>::unpack(q[u], f);
#pragma unroll
                            for (int j = 0; j < V; j++) acc[u][j] += SCALE ? (f[j] * scaling) : f[j];
                        }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < CH; u++) {
                const int64_t c = c0 + u * 64 + lane;
                if (c >= nv) continue;
                if (res) {
                    float r[V];
                    Elem<T>::unpack(__builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(res) + c), r);
#pragma unroll
                    for (int j = 0; j < V; j++) acc[u][j] = r[j] + round_as<T>(acc[u][j]);
                }
                __builtin_nontemporal_store(Elem<T>::pack(acc[u]), reinterpret_cast<u32x4 *>(dst) + c);
            }
        }
    } else {
        for (int64_t e = lane; e < E; e += 64) {
            float acc = 0.0f;
            for (int32_t i = i0; i < i1; i++) {
                const int32_t index = output_indices[i];
                float scaling = 1.0f;
                if (SCALE) scaling = Elem<TW>::load(routing_weights + t * K + selected_experts_indices[i]);
                const float f = Elem<T>::load(rows + static_cast<int64_t>(index) * E + e);
                acc += SCALE ? (f * scaling) : f;
            }
            if (res) acc = Elem<T>::load(res + e) + round_as<T>(acc);
            Elem<T>::store(dst + e, acc);
        }
    }
}

// One wavefront per routed row rt:  pos = output_indices[rt]; t = input_indices[pos];
// k = sel_idx[rt];  dy[pos,:] = w[t,k]*dout[t,:];  dw[t,k] = <y[pos,:], dout[t,:]>.
template <typename T, typename TW>
__global__ __launch_bounds__(256) void combine_backward_kernel(
    const T *__restrict__ dout, const T *__restrict__ y, const TW *__restrict__ routing_weights,
    const int32_t *__restrict__ selected_experts_indices, const int32_t *__restrict__ input_indices,
    const int32_t *__restrict__ output_indices, T *__restrict__ dy, TW *__restrict__ dw, int64_t RT,
    int K, int64_t E, bool vec_ok) {
    const int lane = threadIdx.x & 63;
    const int64_t rt = static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK + (threadIdx.x >> 6);
    if (rt >= RT) return;
    const int32_t index = output_indices[rt];
    const int32_t t = input_indices[index];
    const int32_t k = selected_experts_indices[rt];
    const float scaling = Elem<TW>::load(routing_weights + static_cast<int64_t>(t) * K + k);
    const T *drow = dout + static_cast<int64_t>(t) * E;
    const T *yrow = y + static_cast<int64_t>(index) * E;
    T *dyrow = dy + static_cast<int64_t>(index) * E;
    constexpr int V = Elem<T>::VEC;
    float acc = 0.0f;
    if (vec_ok) {
        const int64_t nv = E / V;
        for (int64_t c = lane; c < nv; c += 64) {
            float d[V], in[V], o[V];
            Elem<T>::unpack(reinterpret_cast<const u32x4 *>(drow)[c], d);
            Elem<T>::unpack(reinterpret_cast<const u32x4 *>(yrow)[c], in);
#pragma unroll
            for (int j = 0; j < V; j++) {
                o[j] = scaling * d[j];
                acc += in[j] * d[j];
            }
            reinterpret_cast<u32x4 *>(dyrow)[c] = Elem<T>::pack(o);
        }
    } else {
        for (int64_t e = lane; e < E; e += 64) {
            const float d = Elem<T>::load(drow + e);
            Elem<T>::store(dyrow + e, scaling * d);
            acc += Elem<T>::load(yrow + e) * d;
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) Elem<TW>::store(dw + static_cast<int64_t>(t) * K + k, acc);
}

// The routing weight of every sorted row, for expert kernels that apply it themselves: routed
// entry rt -> row pos = output_indices[rt], token t = input_indices[pos], slot k = sel_idx[rt];
// row_weights[pos] = w[t,k].
template <typename TW>
__global__ __launch_bounds__(256) void row_weights_kernel(
    const TW *__restrict__ routing_weights, const int32_t *__restrict__ selected_experts_indices,
    const int32_t *__restrict__ input_indices, const int32_t *__restrict__ output_indices,
    float *__restrict__ row_weights, int64_t RT, int K) {
    const int64_t rt = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (rt >= RT) return;
    const int32_t pos = output_indices[rt];
    if (pos < 0) return;   // past the routed pairs (RT may be an upper bound: see om_moe_sort)
    const int32_t t = input_indices[pos];
    row_weights[pos] = Elem<TW>::load(routing_weights + static_cast<int64_t>(t) * K + selected_experts_indices[rt]);
}

// The way back: dw[t,k] = sum over the `parts` column ranges of row_dot[part][pos], added in order.
template <typename TW>
__global__ __launch_bounds__(256) void row_weights_grad_kernel(
    const float *__restrict__ row_dot, int parts, const int32_t *__restrict__ selected_experts_indices,
    const int32_t *__restrict__ input_indices, const int32_t *__restrict__ output_indices,
    TW *__restrict__ dw, int64_t RT, int K) {
    const int64_t rt = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (rt >= RT) return;
    const int32_t pos = output_indices[rt];
    if (pos < 0) return;
    const int32_t t = input_indices[pos];
    float s = 0.0f;
    for (int p0 = 0; p0 < parts; p0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = (p0 + u < parts) ? row_dot[(p0 + u) * RT + pos] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) s += v[u];
    }
    Elem<TW>::store(dw + static_cast<int64_t>(t) * K + selected_experts_indices[rt], s);
}

// output[indices[c],:] += input[c,:], atomically per element so duplicate indices add up.
__global__ void index_add_f32_kernel(const float *__restrict__ input, float *__restrict__ output,
                                     const int32_t *__restrict__ indices, int64_t C, int64_t E) {
    const int64_t c = blockIdx.x;
    if (c >= C) return;
    float *dst = output + static_cast<int64_t>(indices[c]) * E;
    for (int64_t e = threadIdx.x; e < E; e += blockDim.x) atomicAdd(dst + e, input[c * E + e]);
}
// bf16: compare-and-swap on the aligned 32-bit word that holds the element.
__global__ void index_add_bf16_kernel(const uint16_t *__restrict__ input, uint16_t *__restrict__ output,
                                      const int32_t *__restrict__ indices, int64_t C, int64_t E) {
    const int64_t c = blockIdx.x;
    if (c >= C) return;
    for (int64_t e = threadIdx.x; e < E; e += blockDim.x) {
        uint16_t *p = output + static_cast<int64_t>(indices[c]) * E + e;
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        unsigned int *word = reinterpret_cast<unsigned int *>(a & ~static_cast<uintptr_t>(3));
        const int shift = (a & 2) ? 16 : 0;
        const float add = bf16_bits_to_f32(input[c * E + e]);
        unsigned int old = *word, assumed;
        do {
            assumed = old;
            const uint16_t cur = static_cast<uint16_t>((assumed >> shift) & 0xffffu);
            const uint16_t upd = f32_to_bf16_bits(bf16_bits_to_f32(cur) + add);
            const unsigned int repl = (assumed & ~(0xffffu << shift)) | (static_cast<unsigned int>(upd) << shift);
            old = atomicCAS(word, assumed, repl);
        } while (old != assumed);
    }
}

template <typename T> bool row_vec_ok(const void *a, const void *b, const void *c, int64_t E) {
    return (E % Elem<T>::VEC) == 0 && om_aligned16(a) && om_aligned16(b) && (c == nullptr || om_aligned16(c));
}

inline unsigned row_blocks(int64_t rows) {
    return static_cast<unsigned>((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
}

}  // namespace

extern "C" int om_index_gather(const void *input, const int32_t *indices, void *output, int64_t O,
                               int64_t E, int dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    if (O < 0 || E < 0 || O > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (O == 0 || E == 0) return OM_OK;
    if (!input || !indices || !output) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    if (dtype == OM_F32)
        index_gather_kernel<float><<<row_blocks(O), 256, 0, st>>>(
            static_cast<const float *>(input), indices, static_cast<float *>(output), O, E,
            row_vec_ok<float>(input, output, nullptr, E));
    else
        index_gather_kernel<uint16_t><<<row_blocks(O), 256, 0, st>>>(
            static_cast<const uint16_t *>(input), indices, static_cast<uint16_t *>(output), O, E,
            row_vec_ok<uint16_t>(input, output, nullptr, E));
    return om_launch_status();
}

extern "C" int om_index_add(const void *input, void *output, const int32_t *indices, int64_t C,
                            int64_t E, int dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    if (C < 0 || E < 0 || C > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (C == 0 || E == 0) return OM_OK;
    if (!input || !indices || !output) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    if (dtype == OM_F32)
        index_add_f32_kernel<<<static_cast<unsigned>(C), 256, 0, st>>>(
            static_cast<const float *>(input), static_cast<float *>(output), indices, C, E);
    else
        index_add_bf16_kernel<<<static_cast<unsigned>(C), 256, 0, st>>>(
            static_cast<const uint16_t *>(input), static_cast<uint16_t *>(output), indices, C, E);
    return om_launch_status();
}

extern "C" int om_shuffle_sub_matrix_reduce(const void *ggemm_input_grad,
                                            const int32_t *cum_expert_counts_ep,
                                            const int32_t *output_indices, void *hidden_states_grad,
                                            int64_t T, int64_t E, int dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    if (T < 0 || E < 0 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (T == 0 || E == 0) return OM_OK;
    if (!cum_expert_counts_ep || !hidden_states_grad) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    if (dtype == OM_F32)
        token_reduce_kernel<float, float, false><<<row_blocks(T), 256, 0, st>>>(
            static_cast<const float *>(ggemm_input_grad), nullptr, cum_expert_counts_ep, nullptr,
            output_indices, static_cast<float *>(hidden_states_grad), T, 0, E,
            row_vec_ok<float>(ggemm_input_grad, hidden_states_grad, nullptr, E));
    else
        token_reduce_kernel<uint16_t, float, false><<<row_blocks(T), 256, 0, st>>>(
            static_cast<const uint16_t *>(ggemm_input_grad), nullptr, cum_expert_counts_ep, nullptr,
            output_indices, static_cast<uint16_t *>(hidden_states_grad), T, 0, E,
            row_vec_ok<uint16_t>(ggemm_input_grad, hidden_states_grad, nullptr, E));
    return om_launch_status();
}

namespace {
int reduce_ggemm_output_launch(const void *ggemm_output, const void *routing_weights,
                                      const int32_t *cum_expert_counts_ep,
                                      const int32_t *selected_experts_indices,
                                      const int32_t *output_indices, void *final_hidden_states,
                                      int64_t T, int K, int64_t E, int dtype, int weights_dtype,
                                      int skip_weights_scaling, const void *residual, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    if (weights_dtype != OM_F32 && weights_dtype != OM_BF16) return OM_ERR_DTYPE;
    if (dtype == OM_F32 && weights_dtype != OM_F32) return OM_ERR_DTYPE;
    if (T < 0 || E < 0 || K < 0 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (T == 0 || E == 0) return OM_OK;
    if (!cum_expert_counts_ep || !final_hidden_states) return OM_ERR_NULL;
    if (!skip_weights_scaling && !routing_weights) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = row_blocks(T);
#define OM_REDUCE(TT, TW, SC)                                                                      \
    token_reduce_kernel<TT, TW, SC><<<nb, 256, 0, st>>>(                                           \
        static_cast<const TT *>(ggemm_output), static_cast<const TW *>(routing_weights),           \
        cum_expert_counts_ep, selected_experts_indices, output_indices,                            \
        static_cast<TT *>(final_hidden_states), T, K, E,                                           \
        row_vec_ok<TT>(ggemm_output, final_hidden_states, residual, E),                           \
        static_cast<const TT *>(residual))
    if (skip_weights_scaling) {
        if (dtype == OM_F32) OM_REDUCE(float, float, false);
        else OM_REDUCE(uint16_t, float, false);
    } else if (dtype == OM_F32) {
        OM_REDUCE(float, float, true);
    } else if (weights_dtype == OM_F32) {
        OM_REDUCE(uint16_t, float, true);
    } else {
        OM_REDUCE(uint16_t, uint16_t, true);
    }
#undef OM_REDUCE
    return om_launch_status();
}
}  // namespace

extern "C" int om_reduce_ggemm_output(const void *ggemm_output, const void *routing_weights,
                                      const int32_t *cum_expert_counts_ep,
                                      const int32_t *selected_experts_indices,
                                      const int32_t *output_indices, void *final_hidden_states,
                                      int64_t T, int K, int64_t E, int dtype, int weights_dtype,
                                      int skip_weights_scaling, void *stream) {
    return reduce_ggemm_output_launch(ggemm_output, routing_weights, cum_expert_counts_ep,
                                      selected_experts_indices, output_indices, final_hidden_states, T, K,
                                      E, dtype, weights_dtype, skip_weights_scaling, nullptr, stream);
}

extern "C" int om_reduce_ggemm_output_residual(const void *ggemm_output, const void *routing_weights,
                                               const int32_t *cum_expert_counts_ep,
                                               const int32_t *selected_experts_indices,
                                               const int32_t *output_indices, const void *residual,
                                               void *final_hidden_states, int64_t T, int K, int64_t E,
                                               int dtype, int weights_dtype, void *stream) {
    if (T > 0 && E > 0 && !residual) return OM_ERR_NULL;
    return reduce_ggemm_output_launch(ggemm_output, routing_weights, cum_expert_counts_ep,
                                      selected_experts_indices, output_indices, final_hidden_states, T, K,
                                      E, dtype, weights_dtype, 0, residual, stream);
}

extern "C" int om_sum_ggemm_output(const void *ggemm_output, const int32_t *cum_expert_counts_ep,
                                   const int32_t *output_indices, const void *residual,
                                   void *final_hidden_states, int64_t T, int64_t E, int dtype,
                                   void *stream) {
    return reduce_ggemm_output_launch(ggemm_output, nullptr, cum_expert_counts_ep, nullptr, output_indices,
                                      final_hidden_states, T, 0, E, dtype, OM_F32, 1, residual, stream);
}

extern "C" int om_moe_row_weights(const void *routing_weights, const int32_t *selected_experts_indices,
                                  const int32_t *input_indices, const int32_t *output_indices,
                                  float *row_weights, int64_t RT, int K, int weights_dtype, void *stream) {
    if (weights_dtype != OM_F32 && weights_dtype != OM_BF16) return OM_ERR_DTYPE;
    if (RT < 0 || K < 1 || RT > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (RT == 0) return OM_OK;
    if (!routing_weights || !selected_experts_indices || !input_indices || !output_indices || !row_weights)
        return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = static_cast<unsigned>((RT + 255) / 256);
    if (weights_dtype == OM_F32)
        row_weights_kernel<float><<<nb, 256, 0, st>>>(static_cast<const float *>(routing_weights),
                                                      selected_experts_indices, input_indices,
                                                      output_indices, row_weights, RT, K);
    else
        row_weights_kernel<uint16_t><<<nb, 256, 0, st>>>(static_cast<const uint16_t *>(routing_weights),
                                                         selected_experts_indices, input_indices,
                                                         output_indices, row_weights, RT, K);
    return om_launch_status();
}

extern "C" int om_moe_row_weights_grad(const float *row_dot, int parts,
                                       const int32_t *selected_experts_indices,
                                       const int32_t *input_indices, const int32_t *output_indices,
                                       void *routing_weights_grad, int64_t RT, int K, int weights_dtype,
                                       void *stream) {
    if (weights_dtype != OM_F32 && weights_dtype != OM_BF16) return OM_ERR_DTYPE;
    if (RT < 0 || K < 1 || parts < 1 || RT > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (RT == 0) return OM_OK;
    if (!row_dot || !selected_experts_indices || !input_indices || !output_indices || !routing_weights_grad)
        return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = static_cast<unsigned>((RT + 255) / 256);
    if (weights_dtype == OM_F32)
        row_weights_grad_kernel<float><<<nb, 256, 0, st>>>(row_dot, parts, selected_experts_indices,
                                                           input_indices, output_indices,
                                                           static_cast<float *>(routing_weights_grad), RT, K);
    else
        row_weights_grad_kernel<uint16_t><<<nb, 256, 0, st>>>(row_dot, parts, selected_experts_indices,
                                                              input_indices, output_indices,
                                                              static_cast<uint16_t *>(routing_weights_grad), RT, K);
    return om_launch_status();
}

extern "C" int om_reduce_ggemm_output_backward(
    const void *final_hidden_states_grad, const void *ggemm_output, const void *routing_weights,
    const int32_t *selected_experts_indices, const int32_t *input_indices,
    const int32_t *output_indices, void *ggemm_output_grad, void *routing_weights_grad, int64_t RT,
    int K, int64_t E, int dtype, int weights_dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    if (weights_dtype != OM_F32 && weights_dtype != OM_BF16) return OM_ERR_DTYPE;
    if (dtype == OM_F32 && weights_dtype != OM_F32) return OM_ERR_DTYPE;
    if (RT < 0 || E < 0 || K < 0 || RT > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (RT == 0) return OM_OK;
    if (!final_hidden_states_grad || !ggemm_output || !routing_weights || !selected_experts_indices ||
        !input_indices || !output_indices || !ggemm_output_grad || !routing_weights_grad)
        return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = row_blocks(RT);
#define OM_CBWD(TT, TW)                                                                            \
    combine_backward_kernel<TT, TW><<<nb, 256, 0, st>>>(                                           \
        static_cast<const TT *>(final_hidden_states_grad), static_cast<const TT *>(ggemm_output),  \
        static_cast<const TW *>(routing_weights), selected_experts_indices, input_indices,         \
        output_indices, static_cast<TT *>(ggemm_output_grad),                                      \
        static_cast<TW *>(routing_weights_grad), RT, K, E,                                         \
        row_vec_ok<TT>(final_hidden_states_grad, ggemm_output, ggemm_output_grad, E))
    if (dtype == OM_F32) OM_CBWD(float, float);
    else if (weights_dtype == OM_F32) OM_CBWD(uint16_t, float);
    else OM_CBWD(uint16_t, uint16_t);
#undef OM_CBWD
    return om_launch_status();
}

// ---- stand-alone SwiGLU glue ---------------------------------------------------------------
namespace {
__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const T *__restrict__ g, const T *__restrict__ u,
                                                         T *__restrict__ h, int64_t n) {
    constexpr int V = Elem<T>::VEC;
    const int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t nv = n / V;
    if (c < nv) {
        float a[V], b[V], o[V];
        Elem<T>::unpack(reinterpret_cast<const u32x4 *>(g)[c], a);
        Elem<T>::unpack(reinterpret_cast<const u32x4 *>(u)[c], b);
#pragma unroll
        for (int j = 0; j < V; j++) o[j] = (a[j] / (1.0f + expf(-a[j]))) * b[j];
        reinterpret_cast<u32x4 *>(h)[c] = Elem<T>::pack(o);
    } else if (c == nv) {
        for (int64_t i = nv * V; i < n; i++) {
            const float a = Elem<T>::load(g + i);
            Elem<T>::store(h + i, (a / (1.0f + expf(-a))) * Elem<T>::load(u + i));
        }
    }
}
template <typename T>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T *__restrict__ dh, const T *__restrict__ g,
                                                         const T *__restrict__ u, T *__restrict__ dg,
                                                         T *__restrict__ du, int64_t n) {
    constexpr int V = Elem<T>::VEC;
    const int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t nv = n / V;
    if (c < nv) {
        float d[V], a[V], b[V], og[V], ou[V];
        Elem<T>::unpack(reinterpret_cast<const u32x4 *>(dh)[c], d);
        Elem<T>::unpack(reinterpret_cast<const u32x4 *>(g)[c], a);
        Elem<T>::unpack(reinterpret_cast<const u32x4 *>(u)[c], b);
#pragma unroll
        for (int j = 0; j < V; j++) {
            const float sg = sigmoidf_(a[j]);
            ou[j] = d[j] * (a[j] / (1.0f + expf(-a[j])));
            og[j] = (d[j] * b[j]) * (sg * (1.0f + a[j] * (1.0f - sg)));
        }
        reinterpret_cast<u32x4 *>(dg)[c] = Elem<T>::pack(og);
        reinterpret_cast<u32x4 *>(du)[c] = Elem<T>::pack(ou);
    } else if (c == nv) {
        for (int64_t i = nv * V; i < n; i++) {
            const float a = Elem<T>::load(g + i), d = Elem<T>::load(dh + i), b = Elem<T>::load(u + i);
            const float sg = sigmoidf_(a);
            Elem<T>::store(du + i, d * (a / (1.0f + expf(-a))));
            Elem<T>::store(dg + i, (d * b) * (sg * (1.0f + a * (1.0f - sg))));
        }
    }
}
}  // namespace

extern "C" int om_swiglu_fwd(const void *g, const void *u, void *h, int64_t n, int dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    if (n < 0) return OM_ERR_SHAPE;
    if (n == 0) return OM_OK;
    if (!g || !u || !h) return OM_ERR_NULL;
    if (!om_aligned16(g) || !om_aligned16(u) || !om_aligned16(h)) return OM_ERR_ALIGN;
    hipStream_t st = om_stream(stream);
    if (dtype == OM_F32) {
        const int64_t nb = (n / 4 + 1 + 255) / 256;
        swiglu_fwd_kernel<float><<<static_cast<unsigned>(nb), 256, 0, st>>>(
            static_cast<const float *>(g), static_cast<const float *>(u), static_cast<float *>(h), n);
    } else {
        const int64_t nb = (n / 8 + 1 + 255) / 256;
        swiglu_fwd_kernel<uint16_t><<<static_cast<unsigned>(nb), 256, 0, st>>>(
            static_cast<const uint16_t *>(g), static_cast<const uint16_t *>(u), static_cast<uint16_t *>(h), n);
    }
    return om_launch_status();
}

extern "C" int om_swiglu_bwd(const void *dh, const void *g, const void *u, void *dg, void *du,
                             int64_t n, int dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    if (n < 0) return OM_ERR_SHAPE;
    if (n == 0) return OM_OK;
    if (!dh || !g || !u || !dg || !du) return OM_ERR_NULL;
    if (!om_aligned16(dh) || !om_aligned16(g) || !om_aligned16(u) || !om_aligned16(dg) || !om_aligned16(du))
        return OM_ERR_ALIGN;
    hipStream_t st = om_stream(stream);
    if (dtype == OM_F32) {
        const int64_t nb = (n / 4 + 1 + 255) / 256;
        swiglu_bwd_kernel<float><<<static_cast<unsigned>(nb), 256, 0, st>>>(
            static_cast<const float *>(dh), static_cast<const float *>(g), static_cast<const float *>(u),
            static_cast<float *>(dg), static_cast<float *>(du), n);
    } else {
        const int64_t nb = (n / 8 + 1 + 255) / 256;
        swiglu_bwd_kernel<uint16_t><<<static_cast<unsigned>(nb), 256, 0, st>>>(
            static_cast<const uint16_t *>(dh), static_cast<const uint16_t *>(g),
            static_cast<const uint16_t *>(u), static_cast<uint16_t *>(dg), static_cast<uint16_t *>(du), n);
    }
    return om_launch_status();
}
