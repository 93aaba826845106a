// Router gate projection for many experts, logits[t,n] = sum_h x[t,h] * W[n,h] in fp32 from bf16
// operands (the DeepSeek-V3 router: optimus/models/deepseek_v3/modeling_deepseek_v3.py:160 casts
// both operands to float32 and calls F.linear; bf16 x bf16 products are exact in fp32, so this is
// that value up to the order of the sum).
//
// With a few hundred experts the gate weight is megabytes (256 x 7168 bf16 = 3.7 MB).  A block that
// covers 32 tokens re-reads all of it from L2, and that traffic, not the read of x, bounds the
// launch.  Here a block covers 128 tokens (four wavefronts of 32) and a slice of H; the weight tile
// of a 64-wide step is fetched once per block into LDS with direct loads and shared by the four
// wavefronts, the token fragments come straight from global memory in MFMA layout, and the slices
// of H are added by a second kernel in slice order (deterministic).  Weight traffic falls by 4x,
// the blocks still fill the chip through the split of H.
#include "common.h"

namespace {

typedef const __attribute__((address_space(1))) void *glb_ptr;
typedef __attribute__((address_space(3))) void *lds_ptr;

constexpr int GT = 128;   // tokens per block
constexpr int GK = 64;    // columns of H per LDS stage

// W tile [rows][64 h] as 128-byte rows, 16-byte chunk c of row r stored at c ^ ((r >> 1) & 7):
// conflict-free for 16-byte fragment reads of 32 consecutive rows per half-wavefront.
__device__ __forceinline__ int w_off(int row, int ch) { return row * 128 + ((ch ^ ((row >> 1) & 7)) << 4); }

// grid (ceil(T / 128), splits); 256 threads; NB = ceil(N / 32) accumulators per wavefront
template <int NB>
__global__ __launch_bounds__(256) void gate_logits_split_kernel(const uint16_t *__restrict__ x,
                                                                const uint16_t *__restrict__ w,
                                                                int64_t T, int H, int N, int h_per_split,
                                                                float *__restrict__ partial) {
    constexpr int NP = NB * 32;                 // experts rounded up to MFMA blocks
    constexpr int W_LOADS = NP / 8 / 4;         // 1 KB direct loads per wavefront per stage
    __shared__ __attribute__((aligned(1024))) char ws[2][NP * 128];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * GT + wave * 32;
    const int h_begin = blockIdx.y * h_per_split;
    const int steps = h_per_split / GK;
    // H is any multiple of 8: the last step of the last slice may hold fewer than 64 columns.  Its token
    // fragments past the end are zeros, its weight loads past the end re-read the last 8 columns.
    const int h_len = min(H - h_begin, h_per_split);
    // token fragment: lane l holds token t0 + l % 32, 8 consecutive h starting at 8 * (l / 32)
    int64_t ta = t0 + (lane & 31);
    if (ta >= T) ta = T - 1;                    // rows past the end: valid memory, result unused
    const uint16_t *xp = x + ta * H + h_begin + (lane >> 5) * 8;
    // weight loads: load i of this wavefront fills LDS rows (wave * W_LOADS + i) * 8 .. + 7; lane l
    // fetches row + l / 8, chunk (l % 8) ^ swizzle, so that the chunk lands at its swizzled place
    const uint16_t *wp[W_LOADS];
#pragma unroll
    for (int i = 0; i < W_LOADS; i++) {
        const int row = (wave * W_LOADS + i) * 8 + (lane >> 3);
        const int ch = (lane & 7) ^ ((row >> 1) & 7);
        const int src = row < N ? row : N - 1;  // padding rows repeat the last expert (never stored)
        wp[i] = w + static_cast<int64_t>(src) * H + h_begin + ch * 8;
    }
    auto issue_w = [&](int s, int stage) {
        const bool tail = (s + 1) * GK > h_len;          // block-uniform
        const int chunks = (h_len - s * GK) >> 3;         // 8-column chunks the step holds
#pragma unroll
        for (int i = 0; i < W_LOADS; i++) {
            const uint16_t *src = wp[i] + s * GK;
            if (tail) {
                const int row = (wave * W_LOADS + i) * 8 + (lane >> 3);
                const int ch = (lane & 7) ^ ((row >> 1) & 7);
                src -= max(ch - (chunks - 1), 0) * 8;
            }
            __builtin_amdgcn_global_load_lds((glb_ptr)src, (lds_ptr)(ws[stage] + (wave * W_LOADS + i) * 1024), 16, 0, 0);
        }
    };
    f32x16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][r] = 0.0f;
    u32x4 xa[2][GK / 16];
    auto fetch_x = [&](int s, int buf) {
        if ((s + 1) * GK > h_len) {                       // block-uniform
#pragma unroll
            for (int u = 0; u < GK / 16; u++) {
                const bool inside = s * GK + u * 16 + (lane >> 5) * 8 < h_len;
                xa[buf][u] = inside ? *reinterpret_cast<const u32x4 *>(xp + s * GK + u * 16) : u32x4{0, 0, 0, 0};
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < GK / 16; u++) xa[buf][u] = *reinterpret_cast<const u32x4 *>(xp + s * GK + u * 16);
    };
    auto multiply = [&](int stage, int buf) {
#pragma unroll
        for (int u = 0; u < GK / 16; u++) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const u32x4 wf = *reinterpret_cast<const u32x4 *>(ws[stage] + w_off(b * 32 + (lane & 31), u * 2 + (lane >> 5)));
                // lane l then holds token l % 32 and experts b*32 + 8*(r/4) + 4*(l/32) + r%4
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wf),
                                                                 __builtin_bit_cast(bf16x8, xa[buf][u]),
                                                                 acc[b], 0, 0, 0);
            }
        }
    };
    if (steps > 0) {
        issue_w(0, 0);
        fetch_x(0, 0);
    }
    for (int s = 0; s < steps; s += 2) {
        // stage 0 holds step s; fetch step s+1 into stage 1 while step s is multiplied
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's part of step s has landed
        __syncthreads();                      // everyone's has; stage 1 is free (step s-1 was read)
        if (s + 1 < steps) { issue_w(s + 1, 1); fetch_x(s + 1, 1); }
        multiply(0, 0);
        if (s + 1 >= steps) break;
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (s + 2 < steps) { issue_w(s + 2, 0); fetch_x(s + 2, 0); }
        multiply(1, 1);
    }
    const int64_t t = t0 + (lane & 31);
    if (t < T) {
        float *out = partial + (static_cast<int64_t>(blockIdx.y) * T + t) * N;
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int n = b * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (n < N) out[n] = acc[b][r];
            }
    }
}

// logits = sum over the slices of H, in slice order
__global__ __launch_bounds__(256) void gate_logits_reduce_kernel(const float *__restrict__ partial,
                                                                 int splits, int64_t tn,
                                                                 float *__restrict__ logits) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= tn) return;
    float s = 0.0f;
    for (int k0 = 0; k0 < splits; k0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = (k0 + u < splits) ? partial[(k0 + u) * tn + i] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) s += v[u];
    }
    logits[i] = s;
}

inline bool gate_split_shape_ok(int64_t T, int H, int N) {
    return T >= 0 && T <= 0x7fffffffLL && N >= 1 && N <= 256 && H >= 8 && H % 8 == 0;
}

// Slices of H: enough blocks for one per CU when the token count alone does not give them, each
// slice a whole number of 64-wide steps, the last of which may be partial (the fp32 partials cost
// 8 B per logit and slice).
inline int gate_split_count(int64_t T, int H) {
    const int64_t token_blocks = (T + GT - 1) / GT;
    const int steps = (H + GK - 1) / GK;
    int best = 1;
    for (int s = 1; s <= 16 && s <= steps; s++)
        if (steps % s == 0) {
            best = s;
            if (token_blocks * s >= 256) break;
        }
    return best;
}

}  // namespace

extern "C" int64_t om_router_gate_logits_split_workspace_bytes(int64_t T, int H, int N) {
    if (!gate_split_shape_ok(T, H, N)) return OM_ERR_SHAPE;
    return static_cast<int64_t>(gate_split_count(T, H)) * T * N * 4;
}

extern "C" int om_router_gate_logits_split(const void *x, const void *gate_weight, int64_t T, int H, int N,
                                           float *logits_out, void *workspace, int64_t workspace_bytes,
                                           void *stream) {
    if (!gate_split_shape_ok(T, H, N)) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!x || !gate_weight || !logits_out || !workspace) return OM_ERR_NULL;
    if (!om_aligned16(x) || !om_aligned16(gate_weight) || !om_aligned16(workspace)) return OM_ERR_ALIGN;
    const int splits = gate_split_count(T, H);
    const int64_t tn = T * N;
    if (workspace_bytes < splits * tn * 4) return OM_ERR_WORKSPACE;
    hipStream_t st = om_stream(stream);
    const dim3 grid(static_cast<unsigned>((T + GT - 1) / GT), splits);
    const uint16_t *xp = static_cast<const uint16_t *>(x), *wp = static_cast<const uint16_t *>(gate_weight);
    float *ws = static_cast<float *>(workspace);
    const int hps = (H + GK - 1) / GK / splits * GK;   // a whole number of steps; the last slice may end early
    if (N <= 64) gate_logits_split_kernel<2><<<grid, dim3(256), 0, st>>>(xp, wp, T, H, N, hps, ws);
    else if (N <= 128) gate_logits_split_kernel<4><<<grid, dim3(256), 0, st>>>(xp, wp, T, H, N, hps, ws);
    else gate_logits_split_kernel<8><<<grid, dim3(256), 0, st>>>(xp, wp, T, H, N, hps, ws);
    gate_logits_reduce_kernel<<<dim3(static_cast<unsigned>((tn + 255) / 256)), dim3(256), 0, st>>>(ws, splits, tn, logits_out);
    return om_launch_status();
}
