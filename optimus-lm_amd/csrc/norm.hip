// RMSNorm of the decoder layer, optionally fused with the residual add that precedes it
// (reference optimus/models/olmoe/modeling_olmoe.py:93-104 and the layer body :402-409;
// optimus/models/deepseek_v3/modeling_deepseek_v3.py:29-41 is the same expression):
//     h  = x (+ residual)                      rounded to the model dtype, as the tensor add is
//     v  = mean(float(h)^2);  r = rsqrt(v + eps)
//     y  = weight * cast(float(h) * r)         two roundings in bf16: the normalised value, then
//                                              the product with the bf16 weight
// One wavefront per row, 16-byte accesses, the row stays in registers between the two passes
// (rows up to 64 * 16 * ROW_VECS / sizeof(T) elements), HBM-bound.  Backward: per row
//     dxn = dy * weight;  dx = r * (dxn - xn * mean(dxn * xn)),  xn = float(h) * r
// in fp32 (one wavefront per row), and the weight gradient sum_rows dy * cast(xn) column-wise in
// chunks of rows whose partial sums a last kernel adds in chunk order (deterministic).
#include "common.h"

namespace {

#pragma clang fp contract(off)

constexpr int NORM_ROWS = 4;     // rows (wavefronts) per block
constexpr int ROW_VECS = 4;      // 16-byte vectors a lane keeps per pass: 4 KB of a row per pass

template <typename T> __device__ __forceinline__ float round_like(float x);
template <> __device__ __forceinline__ float round_like<float>(float x) { return x; }
template <> __device__ __forceinline__ float round_like<uint16_t>(float x) {
    return bf16_bits_to_f32(f32_to_bf16_bits(x));
}

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const T *__restrict__ x,
                                                          const T *__restrict__ residual,
                                                          const T *__restrict__ weight, float eps,
                                                          T *__restrict__ out, T *__restrict__ h_out,
                                                          float *__restrict__ rstd_out, int64_t rows,
                                                          int64_t E) {
    constexpr int V = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * NORM_ROWS + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t nv = E / V;
    const u32x4 *xr = reinterpret_cast<const u32x4 *>(x + row * E);
    const u32x4 *rr = residual ? reinterpret_cast<const u32x4 *>(residual + row * E) : nullptr;
    u32x4 *hr = h_out ? reinterpret_cast<u32x4 *>(h_out + row * E) : nullptr;
    // pass 1: h = x + residual (kept when the row fits the registers), sum of squares
    u32x4 keep[ROW_VECS];
    const bool fits = nv <= 64 * ROW_VECS;
    float ss = 0.0f;
    for (int64_t c0 = 0; c0 < nv; c0 += 64 * ROW_VECS) {
#pragma unroll
        for (int u = 0; u < ROW_VECS; u++) {
            const int64_t c = c0 + u * 64 + lane;
            if (c < nv) {
                u32x4 q = xr[c];
                if (rr) {
                    float a[V], b[V];
                    Elem<T>::unpack(q, a);
                    Elem<T>::unpack(rr[c], b);
#pragma unroll
                    for (int j = 0; j < V; j++) a[j] = a[j] + b[j];
                    q = Elem<T>::pack(a);       // the sum as the model dtype holds it
                }
                if (hr) hr[c] = q;
                float f[V];
                Elem<T>::unpack(q, f);
#pragma unroll
                for (int j = 0; j < V; j++) ss += f[j] * f[j];
                if (fits) keep[u] = q;
            }
        }
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / static_cast<float>(E) + eps);
    if (lane == 0 && rstd_out) rstd_out[row] = r;
    // pass 2: y = weight * cast(h * r)
    const u32x4 *wr = reinterpret_cast<const u32x4 *>(weight);
    u32x4 *orow = reinterpret_cast<u32x4 *>(out + row * E);
    for (int64_t c0 = 0; c0 < nv; c0 += 64 * ROW_VECS) {
#pragma unroll
        for (int u = 0; u < ROW_VECS; u++) {
            const int64_t c = c0 + u * 64 + lane;
            if (c < nv) {
                u32x4 q;
                if (fits) q = keep[u];
                else if (hr) q = hr[c];
                else {
                    q = xr[c];
                    if (rr) {
                        float a[V], b[V];
                        Elem<T>::unpack(q, a);
                        Elem<T>::unpack(rr[c], b);
#pragma unroll
                        for (int j = 0; j < V; j++) a[j] = a[j] + b[j];
                        q = Elem<T>::pack(a);
                    }
                }
                float f[V], w[V], y[V];
                Elem<T>::unpack(q, f);
                Elem<T>::unpack(wr[c], w);
#pragma unroll
                for (int j = 0; j < V; j++) y[j] = w[j] * round_like<T>(f[j] * r);
                orow[c] = Elem<T>::pack(y);
            }
        }
    }
}

// dx, one wavefront per row.  Rows that fit the registers are read once; longer ones twice.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_dx_kernel(const T *__restrict__ dy,
                                                         const T *__restrict__ h,
                                                         const T *__restrict__ weight,
                                                         const float *__restrict__ rstd,
                                                         T *__restrict__ dx, int64_t rows, int64_t E) {
    constexpr int V = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * NORM_ROWS + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t nv = E / V;
    const bool fits = nv <= 64 * ROW_VECS;
    const float r = rstd[row];
    const u32x4 *wr = reinterpret_cast<const u32x4 *>(weight);
    const u32x4 *dyr = reinterpret_cast<const u32x4 *>(dy + row * E);
    const u32x4 *hr = reinterpret_cast<const u32x4 *>(h + row * E);
    u32x4 *dxr = reinterpret_cast<u32x4 *>(dx + row * E);
    float dxn[ROW_VECS][V], xn[ROW_VECS][V];
    float dot = 0.0f;
    for (int64_t c0 = 0; c0 < nv; c0 += 64 * ROW_VECS) {
#pragma unroll
        for (int u = 0; u < ROW_VECS; u++) {
            const int64_t c = c0 + u * 64 + lane;
            if (c < nv) {
                float g[V], f[V], w[V];
                Elem<T>::unpack(dyr[c], g);
                Elem<T>::unpack(hr[c], f);
                Elem<T>::unpack(wr[c], w);
#pragma unroll
                for (int j = 0; j < V; j++) {
                    xn[u][j] = f[j] * r;
                    dxn[u][j] = g[j] * w[j];
                    dot += dxn[u][j] * xn[u][j];
                }
            }
        }
    }
    dot = wave_sum(dot) / static_cast<float>(E);
    for (int64_t c0 = 0; c0 < nv; c0 += 64 * ROW_VECS) {
#pragma unroll
        for (int u = 0; u < ROW_VECS; u++) {
            const int64_t c = c0 + u * 64 + lane;
            if (c < nv) {
                if (!fits) {
                    float g[V], f[V], w[V];
                    Elem<T>::unpack(dyr[c], g);
                    Elem<T>::unpack(hr[c], f);
                    Elem<T>::unpack(wr[c], w);
#pragma unroll
                    for (int j = 0; j < V; j++) { xn[u][j] = f[j] * r; dxn[u][j] = g[j] * w[j]; }
                }
                float o[V];
#pragma unroll
                for (int j = 0; j < V; j++) o[j] = r * (dxn[u][j] - xn[u][j] * dot);
                dxr[c] = Elem<T>::pack(o);
            }
        }
    }
}

// Partial weight gradient of a chunk of DW_ROWS rows for 64 * V columns: a lane owns V columns,
// the four wavefronts of the block take the rows in turn and are added through LDS.
constexpr int DW_ROWS = 128;
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_dw_kernel(const T *__restrict__ dy,
                                                         const T *__restrict__ h,
                                                         const float *__restrict__ rstd,
                                                         float *__restrict__ dw_part, int64_t rows,
                                                         int64_t E) {
    constexpr int V = Elem<T>::VEC;
    __shared__ float lds_dw[4][64 * V];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t c = static_cast<int64_t>(blockIdx.x) * 64 + lane;      // 16-byte column
    const int64_t r0 = static_cast<int64_t>(blockIdx.y) * DW_ROWS;
    float dw[V];
#pragma unroll
    for (int j = 0; j < V; j++) dw[j] = 0.0f;
    if (c * V < E) {
        for (int i = wave; i < DW_ROWS; i += 4) {
            const int64_t row = r0 + i;
            if (row >= rows) break;
            const float r = rstd[row];
            float g[V], f[V];
            Elem<T>::unpack(reinterpret_cast<const u32x4 *>(dy + row * E)[c], g);
            Elem<T>::unpack(reinterpret_cast<const u32x4 *>(h + row * E)[c], f);
#pragma unroll
            for (int j = 0; j < V; j++) dw[j] += g[j] * round_like<T>(f[j] * r);
        }
    }
#pragma unroll
    for (int j = 0; j < V; j++) lds_dw[wave][lane * V + j] = dw[j];
    __syncthreads();
    for (int t = threadIdx.x; t < 64 * V; t += 256) {
        const int64_t e = static_cast<int64_t>(blockIdx.x) * 64 * V + t;
        if (e < E)
            dw_part[static_cast<int64_t>(blockIdx.y) * E + e] =
                (lds_dw[0][t] + lds_dw[1][t]) + (lds_dw[2][t] + lds_dw[3][t]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce_kernel(const float *__restrict__ dw_part,
                                                                int n_blocks, int64_t E,
                                                                T *__restrict__ dweight) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= E) return;
    float s = 0.0f;
    for (int b = 0; b < n_blocks; b++) s += dw_part[static_cast<int64_t>(b) * E + e];
    Elem<T>::store(dweight + e, s);
}

}  // namespace

extern "C" int om_rmsnorm_fwd(const void *x, const void *residual, const void *weight, double eps,
                              void *out, void *h_out, float *rstd_out, int64_t rows, int64_t E,
                              int dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    const int V = dtype == OM_F32 ? 4 : 8;
    if (rows < 0 || E < 1 || E % V != 0 || rows > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!x || !weight || !out) return OM_ERR_NULL;
    if (!om_aligned16(x) || !om_aligned16(weight) || !om_aligned16(out) ||
        (residual && !om_aligned16(residual)) || (h_out && !om_aligned16(h_out)))
        return OM_ERR_ALIGN;
    hipStream_t st = om_stream(stream);
    const unsigned nb = static_cast<unsigned>((rows + NORM_ROWS - 1) / NORM_ROWS);
    if (dtype == OM_BF16)
        rmsnorm_fwd_kernel<uint16_t><<<nb, 256, 0, st>>>(
            static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(residual),
            static_cast<const uint16_t *>(weight), static_cast<float>(eps), static_cast<uint16_t *>(out),
            static_cast<uint16_t *>(h_out), rstd_out, rows, E);
    else
        rmsnorm_fwd_kernel<float><<<nb, 256, 0, st>>>(
            static_cast<const float *>(x), static_cast<const float *>(residual),
            static_cast<const float *>(weight), static_cast<float>(eps), static_cast<float *>(out),
            static_cast<float *>(h_out), rstd_out, rows, E);
    return om_launch_status();
}

extern "C" int64_t om_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t E) {
    if (rows < 0 || E < 1) return 0;
    return ((rows + DW_ROWS - 1) / DW_ROWS) * E * 4;
}

extern "C" int om_rmsnorm_bwd(const void *dy, const void *h, const void *weight, const float *rstd,
                              void *dx, void *dweight, void *workspace, int64_t workspace_bytes,
                              int64_t rows, int64_t E, int dtype, void *stream) {
    if (dtype != OM_F32 && dtype != OM_BF16) return OM_ERR_DTYPE;
    const int V = dtype == OM_F32 ? 4 : 8;
    if (rows < 1 || E < 1 || E % V != 0 || rows > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (!dy || !h || !weight || !rstd || !dx || !dweight || !workspace) return OM_ERR_NULL;
    if (!om_aligned16(dy) || !om_aligned16(h) || !om_aligned16(weight) || !om_aligned16(dx))
        return OM_ERR_ALIGN;
    if (workspace_bytes < om_rmsnorm_bwd_workspace_bytes(rows, E)) return OM_ERR_WORKSPACE;
    hipStream_t st = om_stream(stream);
    const unsigned nb = static_cast<unsigned>((rows + NORM_ROWS - 1) / NORM_ROWS);
    const int chunks = static_cast<int>((rows + DW_ROWS - 1) / DW_ROWS);
    const dim3 dwgrid(static_cast<unsigned>((E / V + 63) / 64), static_cast<unsigned>(chunks));
    float *part = static_cast<float *>(workspace);
    if (dtype == OM_BF16) {
        const uint16_t *g = static_cast<const uint16_t *>(dy), *hh = static_cast<const uint16_t *>(h);
        rmsnorm_dx_kernel<uint16_t><<<nb, 256, 0, st>>>(g, hh, static_cast<const uint16_t *>(weight), rstd,
                                                        static_cast<uint16_t *>(dx), rows, E);
        rmsnorm_dw_kernel<uint16_t><<<dwgrid, 256, 0, st>>>(g, hh, rstd, part, rows, E);
        rmsnorm_dw_reduce_kernel<uint16_t><<<static_cast<unsigned>((E + 255) / 256), 256, 0, st>>>(
            part, chunks, E, static_cast<uint16_t *>(dweight));
    } else {
        const float *g = static_cast<const float *>(dy), *hh = static_cast<const float *>(h);
        rmsnorm_dx_kernel<float><<<nb, 256, 0, st>>>(g, hh, static_cast<const float *>(weight), rstd,
                                                     static_cast<float *>(dx), rows, E);
        rmsnorm_dw_kernel<float><<<dwgrid, 256, 0, st>>>(g, hh, rstd, part, rows, E);
        rmsnorm_dw_reduce_kernel<float><<<static_cast<unsigned>((E + 255) / 256), 256, 0, st>>>(
            part, chunks, E, static_cast<float *>(dweight));
    }
    return om_launch_status();
}
