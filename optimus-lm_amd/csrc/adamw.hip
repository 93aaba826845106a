// Flat-buffer mixed-precision AdamW: one coalesced, vectorised pass (HBM-bound).
// Algorithmic traffic per element: read grad 2 + master 4 + m 4 + v 4, write master 4 + m 4 +
// v 4 + param 2 = 28 bytes (bf16 mode).  Each fp32 operation is rounded on its own (no FMA
// contraction) so the result is reproducible bit for bit by a scalar CPU loop.
#include "common.h"

namespace {

struct AdamScalars {
    float b1, b2, omb1, omb2, bc1, bc2, eps, neg_lr, neg_lr_wd;
    int use_wd;
};

#pragma clang fp contract(off)
__device__ __forceinline__ void adam_update(float g, float &m, float &v, float &w,
                                            const AdamScalars &s) {
    float mm = m * s.b1;
    mm = mm + s.omb1 * g;
    float vv = v * s.b2;
    vv = vv + (s.omb2 * g) * g;
    float mh = mm / s.bc1;
    float vh = vv / s.bc2;
    float d = sqrtf(vh) + s.eps;
    float ww = w + s.neg_lr * (mh / d);
    if (s.use_wd) ww = ww + s.neg_lr_wd * ww;
    m = mm; v = vv; w = ww;
}

// Streaming policy (both modes), from measurements at 6.9e9 elements on MI355X (same box, same run):
//   * one wavefront per block and one 16-byte vector per lane and stream: 64-thread blocks that own
//     1 KB of every fp32 stream reach 76 % of 8 TB/s where 256-thread blocks owning 16 KB reach 69 %
//     (a pure write stream: 87 % with 4 KB per block, 75 % with 16 KB; grid-stride and span-per-block
//     persistent grids: 65-66 %);
//   * nontemporal loads AND stores: each buffer is touched once per step and is far larger than any
//     cache; either hint alone gains nothing, both together 5-8 %.
//   * at most 12 such wavefronts resident per CU: with the 32 that fit by registers the same kernel
//     reaches 76.5 %, with 20 / 16 / 14 / 12 / 11 / 10: 79.2 / 79.8 / 81.0 / 82.0 / 81.8 / 79.6 % (fewer
//     requests queued at the memory controllers at once).  The launch asks for an LDS allocation it
//     never touches, sized so that 12 blocks fill a CU's 160 KB; nothing else in HIP bounds the
//     number of resident blocks.
// Every wavefront access is one contiguous span (512 B of the bf16 streams, 1 KB of the fp32 ones).
constexpr int ADAMW_THREADS = 64;
constexpr size_t ADAMW_OCCUPANCY_LDS = 13600;   // bytes of dynamic LDS per block: 12 blocks per CU

template <typename T> __device__ __forceinline__ T stream_load(const T *p) { return __builtin_nontemporal_load(p); }
template <typename T> __device__ __forceinline__ void stream_store(T *p, T v) { __builtin_nontemporal_store(v, p); }
// Keeps a value that is only copied from being recognised as "the value just loaded from there"
// (the traffic probe writes back what it read and must keep its stores).
__device__ __forceinline__ void opaque(f32x4 &v) { asm volatile("" : "+v"(v)); }

// CLIP selects what happens to the gradient before the update (reference optimizers.py:136-152,
// torch.nn.utils.clip_grads_with_norm_): 0 = used as is; 1 = multiplied by *grad_scale and rounded
// back to the gradient dtype, as the in-place multiply of the bf16 gradient views does; 2 = the
// same, and the scaled gradient is also stored (then `grad` is null and `grad_rw` is both the
// source and the destination).
// MATH = false is the traffic probe: the same loads and stores with the arithmetic left out (the
// fp32 states are written back as read, param = bf16(master)).
template <int CLIP, bool MATH>
__global__ __launch_bounds__(ADAMW_THREADS) void adamw_bf16_kernel(uint16_t *__restrict__ param,
                                                                      const uint16_t *__restrict__ grad,
                                                                      uint16_t *grad_rw,
                                                                      const float *__restrict__ grad_scale,
                                                                      float *__restrict__ master,
                                                                      float *__restrict__ exp_avg,
                                                                      float *__restrict__ exp_avg_sq,
                                                                      int64_t n_vec4, AdamScalars s) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * ADAMW_THREADS + threadIdx.x;
    if (c >= n_vec4) return;
    const uint16_t *gsrc = CLIP == 2 ? grad_rw : grad;
    float coef = 1.0f;
    if (CLIP) coef = *grad_scale;
    const u32x2 gq = stream_load(reinterpret_cast<const u32x2 *>(gsrc) + c);
    f32x4 m0 = stream_load(reinterpret_cast<const f32x4 *>(exp_avg) + c);
    f32x4 v0 = stream_load(reinterpret_cast<const f32x4 *>(exp_avg_sq) + c);
    f32x4 w0 = stream_load(reinterpret_cast<const f32x4 *>(master) + c);
    float g[4];
    g[0] = __uint_as_float(gq[0] << 16);
    g[1] = __uint_as_float(gq[0] & 0xffff0000u);
    g[2] = __uint_as_float(gq[1] << 16);
    g[3] = __uint_as_float(gq[1] & 0xffff0000u);
    if (CLIP) {
        uint16_t gb[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            gb[i] = f32_to_bf16_bits(g[i] * coef);
            g[i] = bf16_bits_to_f32(gb[i]);
        }
        if (CLIP == 2) {
            u32x2 gs;
            gs[0] = static_cast<uint32_t>(gb[0]) | (static_cast<uint32_t>(gb[1]) << 16);
            gs[1] = static_cast<uint32_t>(gb[2]) | (static_cast<uint32_t>(gb[3]) << 16);
            stream_store(reinterpret_cast<u32x2 *>(grad_rw) + c, gs);
        }
    }
    if (MATH) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float ma = m0[i], va = v0[i], wa = w0[i];
            adam_update(g[i], ma, va, wa, s);
            m0[i] = ma; v0[i] = va; w0[i] = wa;
        }
    } else {
        asm volatile("" : : "v"(g[0]), "v"(g[1]), "v"(g[2]), "v"(g[3]));   // the gradient load stays
        opaque(m0); opaque(v0); opaque(w0);
    }
    stream_store(reinterpret_cast<f32x4 *>(exp_avg) + c, m0);
    stream_store(reinterpret_cast<f32x4 *>(exp_avg_sq) + c, v0);
    stream_store(reinterpret_cast<f32x4 *>(master) + c, w0);
    u32x2 pk;
    pk[0] = static_cast<uint32_t>(f32_to_bf16_bits(w0[0])) | (static_cast<uint32_t>(f32_to_bf16_bits(w0[1])) << 16);
    pk[1] = static_cast<uint32_t>(f32_to_bf16_bits(w0[2])) | (static_cast<uint32_t>(f32_to_bf16_bits(w0[3])) << 16);
    stream_store(reinterpret_cast<u32x2 *>(param) + c, pk);
}

// Elements past the last full vector of 4 (at most 3).
__global__ void adamw_bf16_tail_kernel(uint16_t *param, uint16_t *grad, const float *grad_scale,
                                       int store_grad, float *master, float *exp_avg,
                                       float *exp_avg_sq, int64_t start, int64_t n, AdamScalars s) {
    const int64_t i = start + threadIdx.x;
    if (i < n) {
        float m = exp_avg[i], v = exp_avg_sq[i], w = master[i];
        float g = bf16_bits_to_f32(grad[i]);
        if (grad_scale) {
            const uint16_t gb = f32_to_bf16_bits(g * *grad_scale);
            g = bf16_bits_to_f32(gb);
            if (store_grad) grad[i] = gb;
        }
        adam_update(g, m, v, w, s);
        exp_avg[i] = m; exp_avg_sq[i] = v; master[i] = w;
        param[i] = f32_to_bf16_bits(w);
    }
}

// fp32 mode: the parameter buffer is the master buffer (16 B read, 12 B written per element).
template <int CLIP>
__global__ __launch_bounds__(ADAMW_THREADS) void adamw_f32_kernel(float *__restrict__ master,
                                                                  const float *__restrict__ grad,
                                                                  float *grad_rw,
                                                                  const float *__restrict__ grad_scale,
                                                                  float *__restrict__ exp_avg,
                                                                  float *__restrict__ exp_avg_sq,
                                                                  int64_t n_vec4, AdamScalars s) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * ADAMW_THREADS + threadIdx.x;
    if (c >= n_vec4) return;
    const float *gsrc = CLIP == 2 ? grad_rw : grad;
    float coef = 1.0f;
    if (CLIP) coef = *grad_scale;
    f32x4 g = stream_load(reinterpret_cast<const f32x4 *>(gsrc) + c);
    f32x4 m = stream_load(reinterpret_cast<const f32x4 *>(exp_avg) + c);
    f32x4 v = stream_load(reinterpret_cast<const f32x4 *>(exp_avg_sq) + c);
    f32x4 w = stream_load(reinterpret_cast<const f32x4 *>(master) + c);
    if (CLIP) {
#pragma unroll
        for (int i = 0; i < 4; i++) g[i] = g[i] * coef;
        if (CLIP == 2) stream_store(reinterpret_cast<f32x4 *>(grad_rw) + c, g);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float ma = m[i], va = v[i], wa = w[i];
        adam_update(g[i], ma, va, wa, s);
        m[i] = ma; v[i] = va; w[i] = wa;
    }
    stream_store(reinterpret_cast<f32x4 *>(exp_avg) + c, m);
    stream_store(reinterpret_cast<f32x4 *>(exp_avg_sq) + c, v);
    stream_store(reinterpret_cast<f32x4 *>(master) + c, w);
}
__global__ void adamw_f32_tail_kernel(float *master, float *grad, const float *grad_scale,
                                      int store_grad, float *exp_avg, float *exp_avg_sq,
                                      int64_t start, int64_t n, AdamScalars s) {
    const int64_t i = start + threadIdx.x;
    if (i < n) {
        float m = exp_avg[i], v = exp_avg_sq[i], w = master[i];
        float g = grad[i];
        if (grad_scale) {
            g = g * *grad_scale;
            if (store_grad) grad[i] = g;
        }
        adam_update(g, m, v, w, s);
        exp_avg[i] = m; exp_avg_sq[i] = v; master[i] = w;
    }
}

}  // namespace

// clip: 0 = gradient used as is, 1 = scaled by *grad_scale, 2 = scaled and stored back;
// ADAMW_PROBE = the bf16 kernel's loads and stores without the arithmetic.
constexpr int ADAMW_PROBE = 3;
static int adamw_launch(void *param, void *grad, float *master, float *exp_avg, float *exp_avg_sq,
                        int64_t n, double lr, double beta1, double beta2, double eps,
                        double weight_decay, int64_t step, int param_dtype, const float *grad_scale,
                        int clip, void *stream) {
    if (param_dtype != OM_BF16 && param_dtype != OM_F32) return OM_ERR_DTYPE;
    if (n < 0 || step < 1) return OM_ERR_SHAPE;
    if (n == 0) return OM_OK;
    if (!grad || !master || !exp_avg || !exp_avg_sq) return OM_ERR_NULL;
    if (param_dtype == OM_BF16 && !param) return OM_ERR_NULL;
    if ((clip == 1 || clip == 2) && !grad_scale) return OM_ERR_NULL;
    if (!om_aligned16(grad) || !om_aligned16(master) || !om_aligned16(exp_avg) ||
        !om_aligned16(exp_avg_sq) || (param_dtype == OM_BF16 && !om_aligned16(param)))
        return OM_ERR_ALIGN;
    // One launch gives every lane one 4-element vector and the runtime takes fewer than 2^32 threads
    // per launch, so buffers beyond 2^33 elements are updated in consecutive launches over
    // sub-ranges (the update is element-wise: the same bits as one pass).
    constexpr int64_t MAX_PER_LAUNCH = 1LL << 33;
    if (n > MAX_PER_LAUNCH) {
        const int64_t esz = param_dtype == OM_BF16 ? 2 : 4;
        for (int64_t lo = 0; lo < n; lo += MAX_PER_LAUNCH) {
            const int64_t len = n - lo < MAX_PER_LAUNCH ? n - lo : MAX_PER_LAUNCH;
            const int rc = adamw_launch(param ? static_cast<char *>(param) + lo * esz : nullptr,
                                        static_cast<char *>(grad) + lo * esz, master + lo, exp_avg + lo,
                                        exp_avg_sq + lo, len, lr, beta1, beta2, eps, weight_decay, step,
                                        param_dtype, grad_scale, clip, stream);
            if (rc != OM_OK) return rc;
        }
        return OM_OK;
    }

    // Scalars exactly as the reference forms them: Python doubles, narrowed to fp32 where they
    // meet an fp32 tensor (optimizers.py:193-202).
    AdamScalars s;
    s.b1 = static_cast<float>(beta1);
    s.b2 = static_cast<float>(beta2);
    s.omb1 = static_cast<float>(1.0 - beta1);
    s.omb2 = static_cast<float>(1.0 - beta2);
    s.bc1 = static_cast<float>(1.0 - pow(beta1, static_cast<double>(step)));
    s.bc2 = static_cast<float>(1.0 - pow(beta2, static_cast<double>(step)));
    s.eps = static_cast<float>(eps);
    s.neg_lr = static_cast<float>(-lr);
    s.neg_lr_wd = static_cast<float>(-lr * weight_decay);
    s.use_wd = weight_decay > 0.0 ? 1 : 0;

    hipStream_t st = om_stream(stream);
    const int64_t n_vec = n / 4;
    const int64_t blocks = (n_vec + ADAMW_THREADS - 1) / ADAMW_THREADS;
    if (blocks * ADAMW_THREADS >= (1LL << 32)) return OM_ERR_SHAPE;   // (not reached: see MAX_PER_LAUNCH)
    const dim3 grid(static_cast<unsigned>(blocks)), block(ADAMW_THREADS);
    if (param_dtype == OM_BF16) {
        uint16_t *p = static_cast<uint16_t *>(param), *g = static_cast<uint16_t *>(grad);
        if (n_vec > 0) {
            if (clip == ADAMW_PROBE)
                adamw_bf16_kernel<0, false><<<grid, block, ADAMW_OCCUPANCY_LDS, st>>>(p, g, nullptr, nullptr, master, exp_avg,
                                                                    exp_avg_sq, n_vec, s);
            else if (clip == 0)
                adamw_bf16_kernel<0, true><<<grid, block, ADAMW_OCCUPANCY_LDS, st>>>(p, g, nullptr, nullptr, master, exp_avg,
                                                                   exp_avg_sq, n_vec, s);
            else if (clip == 1)
                adamw_bf16_kernel<1, true><<<grid, block, ADAMW_OCCUPANCY_LDS, st>>>(p, g, nullptr, grad_scale, master, exp_avg,
                                                                   exp_avg_sq, n_vec, s);
            else
                adamw_bf16_kernel<2, true><<<grid, block, ADAMW_OCCUPANCY_LDS, st>>>(p, nullptr, g, grad_scale, master, exp_avg,
                                                                   exp_avg_sq, n_vec, s);
        }
        if (n_vec * 4 < n && clip != ADAMW_PROBE)
            adamw_bf16_tail_kernel<<<1, 64, 0, st>>>(p, g, clip ? grad_scale : nullptr, clip == 2,
                                                     master, exp_avg, exp_avg_sq, n_vec * 4, n, s);
    } else {
        if (clip == ADAMW_PROBE) return OM_ERR_DTYPE;
        float *g = static_cast<float *>(grad);
        if (n_vec > 0) {
            if (clip == 0)
                adamw_f32_kernel<0><<<grid, block, ADAMW_OCCUPANCY_LDS, st>>>(master, g, nullptr, nullptr, exp_avg, exp_avg_sq,
                                                            n_vec, s);
            else if (clip == 1)
                adamw_f32_kernel<1><<<grid, block, ADAMW_OCCUPANCY_LDS, st>>>(master, g, nullptr, grad_scale, exp_avg,
                                                            exp_avg_sq, n_vec, s);
            else
                adamw_f32_kernel<2><<<grid, block, ADAMW_OCCUPANCY_LDS, st>>>(master, nullptr, g, grad_scale, exp_avg,
                                                            exp_avg_sq, n_vec, s);
        }
        if (n_vec * 4 < n)
            adamw_f32_tail_kernel<<<1, 64, 0, st>>>(master, g, clip ? grad_scale : nullptr, clip == 2,
                                                    exp_avg, exp_avg_sq, n_vec * 4, n, s);
    }
    return om_launch_status();
}

extern "C" int om_adamw_step(void *param, const void *grad, float *master, float *exp_avg,
                             float *exp_avg_sq, int64_t n, double lr, double beta1, double beta2,
                             double eps, double weight_decay, int64_t step, int param_dtype,
                             void *stream) {
    return adamw_launch(param, const_cast<void *>(grad), master, exp_avg, exp_avg_sq, n, lr, beta1,
                        beta2, eps, weight_decay, step, param_dtype, nullptr, 0, stream);
}

extern "C" int om_adamw_step_clipped(void *param, void *grad, float *master, float *exp_avg,
                                     float *exp_avg_sq, int64_t n, double lr, double beta1,
                                     double beta2, double eps, double weight_decay, int64_t step,
                                     int param_dtype, const float *grad_scale, int store_scaled_grad,
                                     void *stream) {
    if (!grad_scale) return OM_ERR_NULL;
    return adamw_launch(param, grad, master, exp_avg, exp_avg_sq, n, lr, beta1, beta2, eps,
                        weight_decay, step, param_dtype, grad_scale, store_scaled_grad ? 2 : 1,
                        stream);
}

extern "C" int om_adamw_traffic_probe(void *param, const void *grad, float *master, float *exp_avg,
                                      float *exp_avg_sq, int64_t n, void *stream) {
    return adamw_launch(param, const_cast<void *>(grad), master, exp_avg, exp_avg_sq, n, 0.0, 0.0, 0.0,
                        0.0, 0.0, 1, OM_BF16, nullptr, ADAMW_PROBE, stream);
}
