// Grouped expert GEMMs in float32 (v_mfma_f32_32x32x2_f32, fp32 operands and accumulation), for
// modules kept in float32 like the reference's small CPU-runnable configuration
// (GroupedGemmFunction, optimus/models/common/moe.py:163-215, runs torch.matmul per expert in
// whatever dtype the module has).  Same three products and the same variable-rows-per-expert
// contract as the bf16 kernels; this path is for parity at fp32 accuracy, not for speed: one
// 64x64 output tile per 256-thread block, contraction steps of 16 staged through LDS from
// registers, one stage.
//
// An operand tile is always kept in LDS as [row][c] (c = contraction index, 17-float row pitch).
// CONTIG operands ([row][c] in memory) are copied as float4 along c; STRIDED operands ([c][row] in
// memory: the weight in dgrad, both operands in wgrad) are read as float4 along the rows (coalesced)
// and written to LDS transposed.
#include "common.h"

namespace {

constexpr int TB = 64;      // tile rows and columns
constexpr int KS = 16;      // contraction step
constexpr int PITCH = KS + 1;
typedef __attribute__((ext_vector_type(4))) float f4;

enum { F_CONTIG = 0, F_STRIDED = 1 };

struct F32Params {
    const float *A, *B;
    float *C;
    const int32_t *cum;
    int64_t lda, ldb, ldc, strideB, strideC;
    int n_experts, n_cols, kc;
    int accumulate;   // wgrad: C += product instead of C = product
};

// Fill tile[row][c] (64 x 16) from an operand.  CONTIG: element (row, c) at base[(r0+row)*ld + c0+c];
// STRIDED: element (row, c) at base[(c0+c)*ld + r0+row].  Rows >= r_end and contraction indices
// >= c_end read as zero (extents are multiples of 4, so a float4 is inside or outside as a whole).
template <int KIND>
__device__ __forceinline__ void load_tile(float (*tile)[PITCH], const float *base, int64_t ld, int64_t r0,
                                          int64_t r_end, int64_t c0, int64_t c_end, int tid) {
    if (KIND == F_CONTIG) {
        const int row = tid >> 2, c4 = (tid & 3) * 4;
        f4 v = {0.f, 0.f, 0.f, 0.f};
        if (r0 + row < r_end && c0 + c4 < c_end) v = *reinterpret_cast<const f4 *>(base + (r0 + row) * ld + c0 + c4);
        tile[row][c4] = v[0]; tile[row][c4 + 1] = v[1]; tile[row][c4 + 2] = v[2]; tile[row][c4 + 3] = v[3];
    } else {
        const int c = tid >> 4, row4 = (tid & 15) * 4;
        f4 v = {0.f, 0.f, 0.f, 0.f};
        if (c0 + c < c_end && r0 + row4 < r_end) v = *reinterpret_cast<const f4 *>(base + (c0 + c) * ld + r0 + row4);
        tile[row4][c] = v[0]; tile[row4 + 1][c] = v[1]; tile[row4 + 2][c] = v[2]; tile[row4 + 3][c] = v[3];
    }
}

// One 64x64 tile: C[m0.., n0..] = sum over c in [c0, c1) of A(m, c) * B(n, c); rows >= m_end and
// columns >= n_end are not stored.
template <int AKIND, int BKIND>
__device__ __forceinline__ void tile_product(const float *A, int64_t lda, int64_t a_r0, int64_t a_rend,
                                             const float *B, int64_t ldb, int64_t b_r0, int64_t b_rend,
                                             int64_t c0, int64_t c1, float *C, int64_t ldc, int64_t m0,
                                             int64_t m_end, int64_t n0, int64_t n_end, bool accumulate = false) {
    __shared__ float ta[TB][PITCH], tb[TB][PITCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    for (int64_t c = c0; c < c1; c += KS) {
        __syncthreads();
        load_tile<AKIND>(ta, A, lda, a_r0, a_rend, c, c1, tid);
        load_tile<BKIND>(tb, B, ldb, b_r0, b_rend, c, c1, tid);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < KS; k += 2) {
            const float a = ta[wm + (lane & 31)][k + (lane >> 5)];
            const float b = tb[wn + (lane & 31)][k + (lane >> 5)];
            // operands swapped: lane l then holds output row wm + l%32 and columns
            // wn + 8*(r/4) + 4*(l/32) + r%4
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, acc, 0, 0, 0);
        }
    }
    const int64_t m = m0 + wm + (lane & 31);
    if (m < m_end) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            f4 v = {acc[q * 4], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]};
            const int64_t n = n0 + wn + q * 8 + (lane >> 5) * 4;
            if (n >= n_end) continue;
            f4 *dst = reinterpret_cast<f4 *>(C + m * ldc + n);
            if (accumulate) v += *dst;
            *dst = v;
        }
    }
}

// blockIdx.x = row tile (cut per expert, located by a scan of cum), blockIdx.y = column tile
template <int BKIND>
__global__ __launch_bounds__(256) void ggemm_f32_rows_kernel(const F32Params p) {
    __shared__ int s_expert, s_begin, s_end;
    if (threadIdx.x == 0) {
        int tile = blockIdx.x, found = -1, begin = 0, end = 0;
        for (int e = 0; e < p.n_experts; e++) {
            const int s = p.cum[e], cnt = p.cum[e + 1] - s;
            const int tiles = (cnt + TB - 1) / TB;
            if (tile < tiles) { found = e; begin = s + tile * TB; end = s + cnt; break; }
            tile -= tiles;
        }
        s_expert = found; s_begin = begin; s_end = end;
    }
    __syncthreads();
    const int expert = s_expert;
    if (expert < 0) return;
    const int64_t m0 = s_begin, m_end = s_end, n0 = static_cast<int64_t>(blockIdx.y) * TB;
    const float *B = p.B + expert * p.strideB;
    // fwd:   B = W[g] [n][k], operand rows n0.., contraction k
    // dgrad: B = W[g] [c][col] with c the contraction index, operand rows n0..
    tile_product<F_CONTIG, BKIND>(p.A, p.lda, m0, m_end, B, p.ldb, n0, p.n_cols, 0, p.kc, p.C, p.ldc, m0,
                                  m_end, n0, p.n_cols);
}

// blockIdx = (column tile of dW, row tile of dW, expert): dW[g][n][k] = sum_r dout[r][n] * in[r][k]
__global__ __launch_bounds__(256) void ggemm_f32_wgrad_kernel(const F32Params p) {
    const int expert = blockIdx.z;
    const int64_t r0 = p.cum[expert], r1 = p.cum[expert + 1];
    const int64_t n0 = static_cast<int64_t>(blockIdx.y) * TB, k0 = static_cast<int64_t>(blockIdx.x) * TB;
    float *C = p.C + expert * p.strideC;
    const int64_t n_end = p.kc < n0 + TB ? p.kc : n0 + TB;   // rows of dW: the N extent
    tile_product<F_STRIDED, F_STRIDED>(p.A, p.lda, n0, p.kc, p.B, p.ldb, k0, p.n_cols, r0, r1, C, p.ldc,
                                       n0, n_end, k0, p.n_cols, p.accumulate != 0);
}

inline bool mult8(int64_t v) { return v > 0 && v % 8 == 0; }
inline unsigned tiles_of(int v) { return static_cast<unsigned>((v + TB - 1) / TB); }
inline bool fits31(int64_t v) { return v >= 0 && v < (1LL << 31); }

}  // namespace

extern "C" int om_grouped_gemm_fwd_f32(const float *input, const float *weight, float *output,
                                       const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                       int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult8(N) || !mult8(K)) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!input || !weight || !output || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(input) || !om_aligned16(weight) || !om_aligned16(output)) return OM_ERR_ALIGN;
    F32Params p = {};
    p.A = input; p.B = weight; p.C = output; p.cum = cum_token_counts;
    p.lda = K; p.ldb = K; p.ldc = N;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(N) * K;
    if (p.strideB % 4 != 0) return OM_ERR_ALIGN;
    if (!fits31(rows * K) || !fits31(rows * N) || !fits31(p.strideB * G)) return OM_ERR_SHAPE;
    p.n_experts = G; p.n_cols = N; p.kc = K;
    const int64_t m_tiles = (rows + TB - 1) / TB + G;
    if (m_tiles > 0x7fffffffLL || tiles_of(N) > 65535) return OM_ERR_SHAPE;
    ggemm_f32_rows_kernel<F_CONTIG><<<dim3(static_cast<unsigned>(m_tiles), tiles_of(N)), dim3(256), 0, om_stream(stream)>>>(p);
    return om_launch_status();
}

extern "C" int om_grouped_gemm_dgrad_f32(const float *output_grad, const float *weight, float *input_grad,
                                         const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                         int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult8(N) || !mult8(K)) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!output_grad || !weight || !input_grad || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(output_grad) || !om_aligned16(weight) || !om_aligned16(input_grad)) return OM_ERR_ALIGN;
    F32Params p = {};
    p.A = output_grad; p.B = weight; p.C = input_grad; p.cum = cum_token_counts;
    p.lda = N; p.ldb = K; p.ldc = K;   // din[r][k] = sum_n dout[r][n] * W[n][k]: B is [c = n][row = k]
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(N) * K;
    if (p.strideB % 4 != 0) return OM_ERR_ALIGN;
    if (!fits31(rows * K) || !fits31(rows * N) || !fits31(p.strideB * G)) return OM_ERR_SHAPE;
    p.n_experts = G; p.n_cols = K; p.kc = N;
    const int64_t m_tiles = (rows + TB - 1) / TB + G;
    if (m_tiles > 0x7fffffffLL || tiles_of(K) > 65535) return OM_ERR_SHAPE;
    ggemm_f32_rows_kernel<F_STRIDED><<<dim3(static_cast<unsigned>(m_tiles), tiles_of(K)), dim3(256), 0, om_stream(stream)>>>(p);
    return om_launch_status();
}

namespace {
int wgrad_f32_launch(const float *output_grad, const float *input, float *weight_grad,
                     const int32_t *cum_token_counts, int64_t rows, int G, int N, int K, int64_t w_stride,
                     void *stream, bool accumulate) {
    if (rows < 0 || G < 1 || G > 65535 || !mult8(N) || !mult8(K)) return OM_ERR_SHAPE;
    if (!weight_grad || !cum_token_counts || (rows > 0 && (!output_grad || !input))) return OM_ERR_NULL;
    if (!om_aligned16(output_grad) || !om_aligned16(input) || !om_aligned16(weight_grad)) return OM_ERR_ALIGN;
    F32Params p = {};
    p.A = output_grad; p.B = input; p.C = weight_grad; p.cum = cum_token_counts;
    p.lda = N; p.ldb = K; p.ldc = K;
    p.strideC = w_stride ? w_stride : static_cast<int64_t>(N) * K;
    if (p.strideC % 4 != 0) return OM_ERR_ALIGN;
    if (!fits31(rows * K) || !fits31(rows * N) || !fits31(p.strideC * G) || tiles_of(N) > 65535) return OM_ERR_SHAPE;
    p.n_experts = G; p.n_cols = K; p.kc = N;
    p.accumulate = accumulate ? 1 : 0;
    ggemm_f32_wgrad_kernel<<<dim3(tiles_of(K), tiles_of(N), G), dim3(256), 0, om_stream(stream)>>>(p);
    return om_launch_status();
}
}  // namespace

extern "C" int om_grouped_gemm_wgrad_f32(const float *output_grad, const float *input, float *weight_grad,
                                         const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                         int64_t w_stride, void *stream) {
    return wgrad_f32_launch(output_grad, input, weight_grad, cum_token_counts, rows, G, N, K, w_stride, stream,
                            false);
}

extern "C" int om_grouped_gemm_wgrad_f32_accumulate(const float *output_grad, const float *input,
                                                    float *weight_grad, const int32_t *cum_token_counts,
                                                    int64_t rows, int G, int N, int K, int64_t w_stride,
                                                    void *stream) {
    return wgrad_f32_launch(output_grad, input, weight_grad, cum_token_counts, rows, G, N, K, w_stride, stream,
                            true);
}
