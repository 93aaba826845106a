// Gradient L2 norm over the flat gradient buffer, per parameter and total, and the clip
// coefficient that follows from it (reference optimus/optimizers.py:136-160, which calls
// torch.nn.utils.get_total_norm / clip_grads_with_norm_ on the parameters' gradient views).
//
// Three launches, all deterministic (no atomics):
//   1. grad_sumsq_kernel       one block per chunk of the flat buffer, fp32 sum of squares
//                              (HBM-bound: 2 B/element for bf16, 4 B for fp32, read once);
//   2. seg_norm_kernel         one block per parameter: sums its chunks' partials, takes the
//                              square root and rounds it to the gradient dtype;
//   3. total_norm_kernel       one block: norm of the per-parameter norms, rounded to the gradient
//                              dtype, and coef = min(1, max_norm * (1 / (total + 1e-6))) with every
//                              intermediate rounded to the gradient dtype, as torch does for a
//                              0-dim tensor of that dtype.
// A chunk never straddles two parameters; the host builds the chunk table once.
#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float round_to(float x);
template <> __device__ __forceinline__ float round_to<float>(float x) { return x; }
template <> __device__ __forceinline__ float round_to<uint16_t>(float x) {
    return bf16_bits_to_f32(f32_to_bf16_bits(x));
}

// Sum over the 256 threads of a block; every thread of wave 0 gets the result.
__device__ __forceinline__ float block_sum_256(float v, float *lds4) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds4[wave] = v;
    __syncthreads();
    return (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    for (int o = 32; o > 0; o >>= 1) {
        const long long bits = __double_as_longlong(v);
        const int lo = __shfl_xor(static_cast<int>(bits & 0xffffffffLL), o, 64);
        const int hi = __shfl_xor(static_cast<int>(bits >> 32), o, 64);
        v += __longlong_as_double((static_cast<long long>(hi) << 32) |
                                  static_cast<long long>(static_cast<unsigned int>(lo)));
    }
    return v;
}
__device__ __forceinline__ double block_sum_256_f64(double v, double *lds4) {
    v = wave_sum_f64(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds4[wave] = v;
    __syncthreads();
    return (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
}

#pragma clang fp contract(off)
template <typename T>
__global__ __launch_bounds__(256) void grad_sumsq_kernel(const T *__restrict__ grad,
                                                         const int64_t *__restrict__ chunk_offsets,
                                                         float *__restrict__ partials) {
    constexpr int V = Elem<T>::VEC;
    __shared__ float lds4[4];
    const int64_t begin = chunk_offsets[blockIdx.x];
    const int64_t end = chunk_offsets[blockIdx.x + 1];
    // [begin,a) scalar head, [a,b) whole 16-byte vectors, [b,end) scalar tail
    int64_t a = (begin + V - 1) / V * V;
    if (a > end) a = end;
    int64_t b = end / V * V;
    if (b < a) b = a;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    {
        int64_t i = begin + threadIdx.x;
        if (i < a) { const float g = Elem<T>::load(grad + i); acc[0] += g * g; }
        i = b + threadIdx.x;
        if (i < end) { const float g = Elem<T>::load(grad + i); acc[1] += g * g; }
    }
    const u32x4 *vp = reinterpret_cast<const u32x4 *>(grad + a);
    const int64_t nv = (b - a) / V;
    for (int64_t j = threadIdx.x; j < nv; j += 4 * 256) {
        u32x4 q[4];
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (j + u * 256 < nv) q[u] = __builtin_nontemporal_load(vp + j + u * 256);   // read once
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (j + u * 256 < nv) {
                float f[V];
                Elem<T>::unpack(q[u], f);
#pragma unroll
                for (int i = 0; i < V; i++) acc[u] += f[i] * f[i];
            }
    }
    const float total = block_sum_256((acc[0] + acc[1]) + (acc[2] + acc[3]), lds4);
    if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

template <typename T>
__global__ __launch_bounds__(256) void seg_norm_kernel(const float *__restrict__ partials,
                                                       const int64_t *__restrict__ seg_first_chunk,
                                                       float *__restrict__ seg_norms) {
    __shared__ double lds4[4];
    const int64_t c0 = seg_first_chunk[blockIdx.x], c1 = seg_first_chunk[blockIdx.x + 1];
    double acc = 0.0;
    for (int64_t c = c0 + threadIdx.x; c < c1; c += 256) acc += static_cast<double>(partials[c]);
    const double total = block_sum_256_f64(acc, lds4);
    if (threadIdx.x == 0) seg_norms[blockIdx.x] = round_to<T>(sqrtf(static_cast<float>(total)));
}

template <typename T>
__global__ __launch_bounds__(256) void total_norm_kernel(const float *__restrict__ seg_norms,
                                                         int64_t n_segs, float max_norm,
                                                         float *__restrict__ total_norm,
                                                         float *__restrict__ clip_coef) {
    __shared__ double lds4[4];
    double acc = 0.0;
    for (int64_t s = threadIdx.x; s < n_segs; s += 256) {
        const double x = static_cast<double>(seg_norms[s]);
        acc += x * x;
    }
    const double total_sq = block_sum_256_f64(acc, lds4);
    if (threadIdx.x == 0) {
        const float total = round_to<T>(sqrtf(static_cast<float>(total_sq)));
        *total_norm = total;
        if (clip_coef) {
            // max_norm / (total + 1e-6) evaluates as (total + 1e-6).reciprocal() * max_norm on a
            // 0-dim tensor of the gradient dtype; then clamp(max=1.0)
            const float x = round_to<T>(total + 1e-6f);
            const float r = round_to<T>(1.0f / x);
            const float c = round_to<T>(r * max_norm);
            *clip_coef = c > 1.0f ? 1.0f : c;   // NaN passes through, like torch.clamp
        }
    }
}

// Clip multiplier of the sharded optimizer (reference optimus/optimizers.py:398-432), one thread.
//   mode 0  no process group (:404-405): *value is this shard's norm, already rounded to the
//           gradient dtype, and max_norm / (norm + 1e-6) is evaluated on that 0-dim tensor: the sum,
//           the reciprocal and the product are each rounded to the gradient dtype;
//   mode 1  after the all-reduce (:399-403): *value is the sum over the ranks of the squared fp32
//           shard norms; norm = sqrt(value) and the coefficient are plain fp32.
// `flat_grad_shard.mul_(clip_coef)` runs only when clip_coef < 1 (:431-432) and, both operands being
// device tensors, casts the 0-dim coefficient to the gradient dtype before multiplying; hence
// *multiplier = coef < 1 ? round(coef) : 1 (a NaN coefficient compares false and scales nothing).
template <typename T>
__global__ void shard_clip_kernel(const float *__restrict__ value, int mode, float max_norm,
                                  float *__restrict__ grad_norm, float *__restrict__ multiplier) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    float norm, c;
    if (mode == 0) {
        norm = *value;
        const float x = round_to<T>(norm + 1e-6f);
        const float r = round_to<T>(1.0f / x);
        c = round_to<T>(r * max_norm);
    } else {
        norm = sqrtf(*value);
        const float x = norm + 1e-6f;
        const float r = 1.0f / x;
        c = r * max_norm;
    }
    *grad_norm = norm;
    *multiplier = c < 1.0f ? round_to<T>(c) : 1.0f;
}

// grad = cast(float(grad) * *coef), 16 bytes per lane, scalar tail.
template <typename T>
__global__ __launch_bounds__(256) void grad_scale_kernel(T *__restrict__ grad, int64_t n,
                                                         const float *__restrict__ coef) {
    constexpr int V = Elem<T>::VEC;
    const float c = *coef;
    const int64_t nv = n / V;
    u32x4 *vp = reinterpret_cast<u32x4 *>(grad);
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t j = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; j < nv; j += stride) {
        float f[V];
        Elem<T>::unpack(vp[j], f);
#pragma unroll
        for (int i = 0; i < V; i++) f[i] = f[i] * c;
        vp[j] = Elem<T>::pack(f);
    }
    if (blockIdx.x == 0) {
        const int64_t i = nv * V + threadIdx.x;
        if (i < n) Elem<T>::store(grad + i, Elem<T>::load(grad + i) * c);
    }
}

}  // namespace

extern "C" int om_grad_scale(void *grad, int64_t n, int grad_dtype, const float *coef, void *stream) {
    if (grad_dtype != OM_BF16 && grad_dtype != OM_F32) return OM_ERR_DTYPE;
    if (n < 0) return OM_ERR_SHAPE;
    if (n == 0) return OM_OK;
    if (!grad || !coef) return OM_ERR_NULL;
    if (!om_aligned16(grad)) return OM_ERR_ALIGN;
    const int vec = grad_dtype == OM_BF16 ? 8 : 4;
    int64_t blocks = (n / vec + 255) / 256;
    if (blocks < 1) blocks = 1;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipStream_t st = om_stream(stream);
    if (grad_dtype == OM_BF16)
        grad_scale_kernel<uint16_t><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st>>>(
            static_cast<uint16_t *>(grad), n, coef);
    else
        grad_scale_kernel<float><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st>>>(
            static_cast<float *>(grad), n, coef);
    return om_launch_status();
}

extern "C" int om_shard_clip_multiplier(const float *value, int mode, int grad_dtype, double max_norm,
                                        float *grad_norm, float *multiplier, void *stream) {
    if (grad_dtype != OM_BF16 && grad_dtype != OM_F32) return OM_ERR_DTYPE;
    if (mode != 0 && mode != 1) return OM_ERR_SHAPE;
    if (!value || !grad_norm || !multiplier) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const float mx = static_cast<float>(max_norm);
    if (grad_dtype == OM_BF16)
        shard_clip_kernel<uint16_t><<<dim3(1), dim3(64), 0, st>>>(value, mode, mx, grad_norm, multiplier);
    else
        shard_clip_kernel<float><<<dim3(1), dim3(64), 0, st>>>(value, mode, mx, grad_norm, multiplier);
    return om_launch_status();
}

extern "C" int om_grad_sumsq(const void *grad, int grad_dtype, const int64_t *chunk_offsets,
                             int64_t n_chunks, float *partials, void *stream) {
    if (grad_dtype != OM_BF16 && grad_dtype != OM_F32) return OM_ERR_DTYPE;
    if (n_chunks < 0 || n_chunks > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (n_chunks == 0) return OM_OK;
    if (!grad || !chunk_offsets || !partials) return OM_ERR_NULL;
    if (!om_aligned16(grad)) return OM_ERR_ALIGN;
    hipStream_t st = om_stream(stream);
    const dim3 grid(static_cast<unsigned>(n_chunks));
    if (grad_dtype == OM_BF16)
        grad_sumsq_kernel<uint16_t><<<grid, dim3(256), 0, st>>>(static_cast<const uint16_t *>(grad),
                                                                chunk_offsets, partials);
    else
        grad_sumsq_kernel<float><<<grid, dim3(256), 0, st>>>(static_cast<const float *>(grad),
                                                             chunk_offsets, partials);
    return om_launch_status();
}

extern "C" int om_grad_norm_clip_coef(const float *partials, const int64_t *seg_first_chunk,
                                      int64_t n_segs, int grad_dtype, double max_norm,
                                      float *seg_norms, float *total_norm, float *clip_coef,
                                      void *stream) {
    if (grad_dtype != OM_BF16 && grad_dtype != OM_F32) return OM_ERR_DTYPE;
    if (n_segs < 1 || n_segs > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (!partials || !seg_first_chunk || !seg_norms || !total_norm) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const dim3 grid(static_cast<unsigned>(n_segs));
    const float mx = static_cast<float>(max_norm);
    if (grad_dtype == OM_BF16) {
        seg_norm_kernel<uint16_t><<<grid, dim3(256), 0, st>>>(partials, seg_first_chunk, seg_norms);
        total_norm_kernel<uint16_t><<<dim3(1), dim3(256), 0, st>>>(seg_norms, n_segs, mx, total_norm,
                                                                  clip_coef);
    } else {
        seg_norm_kernel<float><<<grid, dim3(256), 0, st>>>(partials, seg_first_chunk, seg_norms);
        total_norm_kernel<float><<<dim3(1), dim3(256), 0, st>>>(seg_norms, n_segs, mx, total_norm,
                                                               clip_coef);
    }
    return om_launch_status();
}
