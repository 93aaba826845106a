// The router's gate projection for float32 modules (the reference's small CPU-runnable
// configuration keeps the whole block in float32): logits = x W^T of the gate nn.Linear
// (optimus/models/common/moe.py:456, optimus/models/olmoe/modeling_olmoe.py:284) and the two
// products of its backward, in plain float32 arithmetic with sums in a fixed order.  This is the
// parity path at fp32 accuracy; nothing here is tuned (the bf16 gate runs on MFMA, gate_fwd.hip and
// gate_bwd.hip).
#include "common.h"

namespace {

// logits[t,n] = sum_h x[t,h] W[n,h]: one wavefront per token, lanes over h, the 64 partial sums
// added by a butterfly.
__global__ __launch_bounds__(256) void gate_logits_f32_kernel(const float *__restrict__ x,
                                                              const float *__restrict__ w, int64_t T,
                                                              int H, int N, float *__restrict__ logits) {
    const int lane = threadIdx.x & 63;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const float *xr = x + t * H;
    for (int n = 0; n < N; n++) {
        const float *wr = w + static_cast<int64_t>(n) * H;
        float s = 0.0f;
        for (int h = lane; h < H; h += 64) s += xr[h] * wr[h];
        s = wave_sum(s);
        if (lane == 0) logits[t * N + n] = s;
    }
}

// dx[t,h] = sum_n dlogits[t,n] W[n,h]: one thread per element, n ascending.
__global__ __launch_bounds__(256) void gate_dgrad_f32_kernel(const float *__restrict__ dlogits,
                                                             const float *__restrict__ w, int64_t T,
                                                             int H, int N, float *__restrict__ dx) {
    const int h = blockIdx.x * 256 + threadIdx.x;
    const int64_t t = blockIdx.y;
    if (h >= H) return;
    float s = 0.0f;
    for (int n = 0; n < N; n++) s += dlogits[t * N + n] * w[static_cast<int64_t>(n) * H + h];
    dx[t * H + h] = s;
}

// dW[n,h] = sum_t dlogits[t,n] x[t,h]: one thread per element, tokens ascending, the sum kept in
// double (thousands of terms) and rounded once.
__global__ __launch_bounds__(256) void gate_wgrad_f32_kernel(const float *__restrict__ x,
                                                             const float *__restrict__ dlogits,
                                                             int64_t T, int H, int N,
                                                             float *__restrict__ dw) {
    const int h = blockIdx.x * 256 + threadIdx.x;
    const int n = blockIdx.y;
    if (h >= H) return;
    double s = 0.0;
    for (int64_t t = 0; t < T; t++)
        s += static_cast<double>(dlogits[t * N + n]) * static_cast<double>(x[t * H + h]);
    dw[static_cast<int64_t>(n) * H + h] = static_cast<float>(s);
}

inline bool gate_f32_shape_ok(int64_t T, int H, int N) {
    return T >= 0 && T <= 0x7fffffffLL && H >= 1 && N >= 1 && N <= 65535;
}

}  // namespace

extern "C" int om_router_gate_logits_f32(const float *x, const float *gate_weight, int64_t T, int H, int N,
                                         float *logits_out, void *stream) {
    if (!gate_f32_shape_ok(T, H, N)) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!x || !gate_weight || !logits_out) return OM_ERR_NULL;
    gate_logits_f32_kernel<<<static_cast<unsigned>((T + 3) / 4), 256, 0, om_stream(stream)>>>(
        x, gate_weight, T, H, N, logits_out);
    return om_launch_status();
}

extern "C" int om_router_gate_dgrad_f32(const float *dlogits, const float *gate_weight, int64_t T, int H,
                                        int N, float *dx, void *stream) {
    if (!gate_f32_shape_ok(T, H, N) || T > 65535LL * 32768) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!dlogits || !gate_weight || !dx) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    // the grid's y extent is limited to 65535: tokens go in slabs
    for (int64_t t0 = 0; t0 < T; t0 += 65535) {
        const int64_t nt = T - t0 < 65535 ? T - t0 : 65535;
        gate_dgrad_f32_kernel<<<dim3((H + 255) / 256, static_cast<unsigned>(nt)), 256, 0, st>>>(
            dlogits + t0 * N, gate_weight, nt, H, N, dx + t0 * H);
    }
    return om_launch_status();
}

extern "C" int om_router_gate_wgrad_f32(const float *x, const float *dlogits, int64_t T, int H, int N,
                                        float *dweight, void *stream) {
    if (!gate_f32_shape_ok(T, H, N)) return OM_ERR_SHAPE;
    if (!dweight) return OM_ERR_NULL;
    if (T > 0 && (!x || !dlogits)) return OM_ERR_NULL;
    gate_wgrad_f32_kernel<<<dim3((H + 255) / 256, N), 256, 0, om_stream(stream)>>>(x, dlogits, T, H, N, dweight);
    return om_launch_status();
}
