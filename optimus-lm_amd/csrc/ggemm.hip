// Grouped expert GEMMs on bf16 MFMA (v_mfma_f32_32x32x16_bf16), fp32 accumulation.
//
// One kernel template covers every product of the merged MLP.  An output tile BM x BN is
// computed by WAVES_M x WAVES_N wavefronts; each wavefront owns a (BM/WAVES_M) x (BN/WAVES_N)
// sub-tile as a grid of 32x32 MFMA accumulators.  Operands are staged through LDS in steps of
// 64 along the contraction index c, double buffered, one barrier per step.
//
// An operand is either
//   CONTIG  — stored [row][c] with c contiguous (activations in fwd/dgrad, weights in fwd):
//             LDS keeps 128-byte rows with the 16-byte chunks XOR-permuted per row; a fragment
//             is one ds_read_b128 per lane;
//   STRIDED — stored [c][row] with row contiguous (weights in dgrad, both operands in wgrad):
//             LDS keeps the tile as it lies in memory; fragments come from the gfx950
//             transposing LDS read (ds_read_b64_tr_b16), two per lane.
// The per-lane order of the 8 contraction indices is the same for both kinds, so they can be
// mixed in one MFMA.
//
// Variable rows per expert: the M extent of fwd/dgrad is cut into tiles per expert; a block finds
// its (expert, row block) from the device-resident cum_token_counts with a wavefront scan, so no
// host copy of the counts and no max-rows-per-expert is needed.  In wgrad the rows are the
// contraction range of expert g and rows past its end are zero-filled.
#include "common.h"

namespace {

enum { CONTIG = 0, STRIDED = 1 };
enum {
    EPI_STORE = 0,        // C = acc
    EPI_SWIGLU = 1,       // even 32-col accumulators = gate, odd = up: store g, u, h
    EPI_SWIGLU_BWD = 2,   // acc = dh: read g,u, store dg, du
    EPI_WGRAD = 3         // C[g] = acc, no row masking
};

constexpr int BK = 64;  // contraction step, elements

struct GemmParams {
    // operands; for the two-phase products (gate+up) index 1 is the second pair
    const uint16_t *A[2];
    const uint16_t *B[2];
    uint16_t *C;         // EPI_STORE / EPI_WGRAD output;  EPI_SWIGLU: g ; EPI_SWIGLU_BWD: dg
    uint16_t *C1;        // EPI_SWIGLU: u ; EPI_SWIGLU_BWD: du
    uint16_t *C2;        // EPI_SWIGLU: h
    const uint16_t *G;   // EPI_SWIGLU_BWD: saved g
    const uint16_t *U;   // EPI_SWIGLU_BWD: saved u
    const int32_t *cum;  // [G+1] device
    int64_t lda, ldb, ldc;      // leading dimensions, elements
    int64_t strideB, strideC;   // per-expert strides, elements
    int64_t rows;               // allocated activation rows (upper bound of cum[G])
    int n_experts;
    int n_cols;                 // output columns (fwd/dgrad) — tiles along N = n_cols / BN_OUT
    int kc;                     // contraction length per phase (fwd/dgrad), multiple of 64
    int phases;                 // 1 or 2
    int m_tiles_max;            // fwd/dgrad: upper bound on row tiles
};

__device__ __forceinline__ int swz(int row) { return (row + (row >> 3)) & 7; }

// LDS byte offset of 16-byte chunk `ch` of row `row` in a CONTIG tile.
__device__ __forceinline__ int contig_off(int row, int ch) { return row * 128 + ((ch ^ swz(row)) << 4); }

template <int R> struct StridedTile {
    static constexpr int PITCH = R * 2 + 64;  // bytes per c-row; +64 spreads rows over the banks
    static constexpr int BYTES = BK * PITCH;
};
template <int R> struct ContigTile {
    static constexpr int BYTES = R * 128;
};
template <int KIND, int R> struct TileBytes {
    static constexpr int value = KIND == CONTIG ? ContigTile<R>::BYTES : StridedTile<R>::BYTES;
};

typedef __attribute__((address_space(3))) s16x4 *lds_s16x4_ptr;

__device__ __forceinline__ bf16x8 lds_read_frag_contig(const char *tile, int row, int ch) {
    const u32x4 v = *reinterpret_cast<const u32x4 *>(tile + contig_off(row, ch));
    return __builtin_bit_cast(bf16x8, v);
}

// Transposing read: lanes 4r..4r+3 of a 16-lane group address c-row r, 4 consecutive rows-of-the-
// operand each; lane i receives operand row i at c-rows 0..3.
template <int R>
__device__ __forceinline__ bf16x8 lds_read_frag_strided(const char *tile, int c0, int m0, int lane) {
    const int i = lane & 15;
    const int r = i >> 2, q = i & 3;
    const int mb = ((lane >> 4) & 1) * 16;
    const int g2 = lane >> 5;
    const char *p = tile + (c0 + 8 * g2 + r) * StridedTile<R>::PITCH + (m0 + mb + 4 * q) * 2;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * StridedTile<R>::PITCH));
    typedef __attribute__((ext_vector_type(8))) short s16x8;
    s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, v);
}

__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    f32x2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ void unpack4_bf16(u32x2 v, float *f) {
    f[0] = __uint_as_float(v[0] << 16);
    f[1] = __uint_as_float(v[0] & 0xffff0000u);
    f[2] = __uint_as_float(v[1] << 16);
    f[3] = __uint_as_float(v[1] & 0xffff0000u);
}

// Which expert owns row tile `tile` (tiles are BM rows, cut per expert)?  Wavefront scan over
// cum_token_counts.  Returns false when `tile` is past the last tile.
template <int BM>
__device__ __forceinline__ bool find_tile(const int32_t *cum, int n_experts, int tile, int lane,
                                          int &expert, int &row_begin, int &row_end) {
    int base_tiles = 0;
    for (int e0 = 0; e0 < n_experts; e0 += 64) {
        const int e = e0 + lane;
        int s = 0, cnt = 0;
        if (e < n_experts) { s = cum[e]; cnt = cum[e + 1] - s; }
        const int tiles = (cnt + BM - 1) / BM;
        int incl = tiles;  // inclusive scan over the wavefront
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o, 64);
            if (lane >= o) incl += v;
        }
        const int excl = incl - tiles;
        const bool mine = (tile >= base_tiles + excl) && (tile < base_tiles + incl);
        const unsigned long long vote = __ballot(mine);
        if (vote) {
            const int src = __ffsll(static_cast<long long>(vote)) - 1;
            const int local = tile - (base_tiles + __shfl(excl, src, 64));
            const int s_src = __shfl(s, src, 64);
            const int cnt_src = __shfl(cnt, src, 64);
            expert = e0 + src;
            row_begin = s_src + local * BM;
            row_end = s_src + cnt_src;
            return true;
        }
        base_tiles += __shfl(incl, 63, 64);
    }
    return false;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int AKIND, int BKIND, int EPI>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void ggemm_kernel(const GemmParams p) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wavefront sub-tile
    constexpr int TM = WM / 32, TN = WN / 32;            // 32x32 accumulators per wavefront
    constexpr int A_BYTES = TileBytes<AKIND, BM>::value;
    constexpr int B_BYTES = TileBytes<BKIND, BN>::value;
    constexpr int STAGE = A_BYTES + B_BYTES;
    extern __shared__ __attribute__((aligned(16))) char smem[];  // 2 stages

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // ---- which tile ---------------------------------------------------------------------
    int expert, row_begin, row_end;  // fwd/dgrad: rows of this tile's expert segment
    int n0;                          // first output column (LDS B row 0)
    int64_t c_begin, c_len;          // contraction range
    if (EPI == EPI_WGRAD) {
        // grid: x = (N/BM) * (K/BN) tiles of dW[g], y = expert
        const int tiles_n = p.n_cols / BN;  // n_cols = K_orig (columns of dW), rows of dW = p.kc
        expert = blockIdx.y;
        const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
        row_begin = tm * BM;  // row of dW
        row_end = 0;
        n0 = tn * BN;
        c_begin = p.cum[expert];
        c_len = p.cum[expert + 1] - c_begin;
    } else {
        constexpr int BN_OUT = (EPI == EPI_SWIGLU) ? BN / 2 : BN;
        const int tiles_n = p.n_cols / BN_OUT;
        const int tile_m = blockIdx.x / tiles_n;
        const int tile_n = blockIdx.x % tiles_n;
        if (!find_tile<BM>(p.cum, p.n_experts, tile_m, lane, expert, row_begin, row_end)) return;
        n0 = tile_n * BN_OUT;
        c_begin = 0;
        c_len = p.kc;
    }
    const int phases = p.phases;
    const int steps_per_phase = static_cast<int>((c_len + BK - 1) / BK);
    const int total_steps = steps_per_phase * phases;

    // ---- global -> register staging ---------------------------------------------------------
    constexpr int A_CHUNKS = BM * 8 / NT;  // 16-byte chunks per thread per step
    constexpr int B_CHUNKS = BN * 8 / NT;
    static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile/thread mismatch");
    u32x4 ra[A_CHUNKS], rb[B_CHUNKS];

    auto load_tiles = [&](int step) {
        const int ph = step / steps_per_phase;
        const int64_t c0 = static_cast<int64_t>(step - ph * steps_per_phase) * BK;
        const uint16_t *Ap = p.A[ph];
        const uint16_t *Bp = p.B[ph];
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            const int q = tid + i * NT;
            if (AKIND == CONTIG) {
                const int row = q >> 3, ch = q & 7;
                int64_t m = static_cast<int64_t>(row_begin) + row;
                if (m >= row_end) m = row_end - 1;  // rows past the segment: valid memory, result unused
                ra[i] = *reinterpret_cast<const u32x4 *>(Ap + m * p.lda + c0 + ch * 8);
            } else {
                constexpr int CPR = BM / 8;
                const int crow = q / CPR, ch = q % CPR;
                const int64_t c = c0 + crow;
                if (c < c_len)
                    ra[i] = *reinterpret_cast<const u32x4 *>(Ap + (c_begin + c) * p.lda + row_begin + ch * 8);
                else
                    ra[i] = u32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) {
            const int q = tid + i * NT;
            if (BKIND == CONTIG) {
                const int row = q >> 3, ch = q & 7;
                int64_t n;
                const uint16_t *Bq = Bp;
                if (EPI == EPI_SWIGLU) {
                    // LDS rows alternate 32 gate rows / 32 up rows
                    const int blk = row >> 5;
                    n = n0 + (blk >> 1) * 32 + (row & 31);
                    Bq = (blk & 1) ? p.B[1] : p.B[0];
                } else {
                    n = n0 + row;
                }
                rb[i] = *reinterpret_cast<const u32x4 *>(Bq + expert * p.strideB + n * p.ldb + c0 + ch * 8);
            } else {
                constexpr int CPR = BN / 8;
                const int crow = q / CPR, ch = q % CPR;
                const int64_t c = c0 + crow;
                if (EPI == EPI_WGRAD) {
                    if (c < c_len)
                        rb[i] = *reinterpret_cast<const u32x4 *>(Bp + (c_begin + c) * p.ldb + n0 + ch * 8);
                    else
                        rb[i] = u32x4{0, 0, 0, 0};
                } else {
                    rb[i] = *reinterpret_cast<const u32x4 *>(Bp + expert * p.strideB + c * p.ldb + n0 + ch * 8);
                }
            }
        }
    };
    auto store_tiles = [&](int stage) {
        char *sa = smem + stage * STAGE;
        char *sb = sa + A_BYTES;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            const int q = tid + i * NT;
            if (AKIND == CONTIG) {
                *reinterpret_cast<u32x4 *>(sa + contig_off(q >> 3, q & 7)) = ra[i];
            } else {
                constexpr int CPR = BM / 8;
                *reinterpret_cast<u32x4 *>(sa + (q / CPR) * StridedTile<BM>::PITCH + (q % CPR) * 16) = ra[i];
            }
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) {
            const int q = tid + i * NT;
            if (BKIND == CONTIG) {
                *reinterpret_cast<u32x4 *>(sb + contig_off(q >> 3, q & 7)) = rb[i];
            } else {
                constexpr int CPR = BN / 8;
                *reinterpret_cast<u32x4 *>(sb + (q / CPR) * StridedTile<BN>::PITCH + (q % CPR) * 16) = rb[i];
            }
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    if (total_steps > 0) {
        load_tiles(0);
        store_tiles(0);
    }
    __syncthreads();

    for (int step = 0; step < total_steps; step++) {
        const int stage = step & 1;
        if (step + 1 < total_steps) load_tiles(step + 1);
        const char *sa = smem + stage * STAGE;
        const char *sb = sa + A_BYTES;
#pragma unroll
        for (int kk = 0; kk < BK / 16; kk++) {
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) {
                if (AKIND == CONTIG)
                    fa[i] = lds_read_frag_contig(sa, wm * WM + i * 32 + (lane & 31), kk * 2 + (lane >> 5));
                else
                    fa[i] = lds_read_frag_strided<BM>(sa, kk * 16, wm * WM + i * 32, lane);
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (BKIND == CONTIG)
                    fb[j] = lds_read_frag_contig(sb, wn * WN + j * 32 + (lane & 31), kk * 2 + (lane >> 5));
                else
                    fb[j] = lds_read_frag_strided<BN>(sb, kk * 16, wn * WN + j * 32, lane);
            }
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    // operands swapped: the lane then holds 4 consecutive output columns per row
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
        if (step + 1 < total_steps) store_tiles(stage ^ 1);
        __syncthreads();
    }

    // ---- epilogue ------------------------------------------------------------------------------
    // accumulator element r of lane l: output row (l % 32), column (r/4)*8 + (l/32)*4 + (r%4).
    const int lrow = lane & 31;
    const int lcol = (lane >> 5) * 4;
    if (EPI == EPI_STORE || EPI == EPI_WGRAD) {
        uint16_t *Cb = p.C + (EPI == EPI_WGRAD ? expert * p.strideC : 0);
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int64_t m = static_cast<int64_t>(row_begin) + wm * WM + i * 32 + lrow;
            if (EPI == EPI_STORE && m >= row_end) continue;
#pragma unroll
            for (int j = 0; j < TN; j++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int n = n0 + wn * WN + j * 32 + rq * 8 + lcol;
                    u32x2 v;
                    v[0] = pack2_bf16(acc[i][j][rq * 4 + 0], acc[i][j][rq * 4 + 1]);
                    v[1] = pack2_bf16(acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3]);
                    *reinterpret_cast<u32x2 *>(Cb + m * p.ldc + n) = v;
                }
            }
        }
    } else if (EPI == EPI_SWIGLU) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int64_t m = static_cast<int64_t>(row_begin) + wm * WM + i * 32 + lrow;
            if (m >= row_end) continue;
#pragma unroll
            for (int j = 0; j < TN; j += 2) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int n = n0 + (wn * WN + j * 32) / 2 + rq * 8 + lcol;
                    float hv[4];
#pragma unroll
                    for (int x = 0; x < 4; x++) {
                        const float gv = acc[i][j][rq * 4 + x], uv = acc[i][j + 1][rq * 4 + x];
                        hv[x] = (gv / (1.0f + __expf(-gv))) * uv;
                    }
                    u32x2 vg, vu, vh;
                    vg[0] = pack2_bf16(acc[i][j][rq * 4 + 0], acc[i][j][rq * 4 + 1]);
                    vg[1] = pack2_bf16(acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3]);
                    vu[0] = pack2_bf16(acc[i][j + 1][rq * 4 + 0], acc[i][j + 1][rq * 4 + 1]);
                    vu[1] = pack2_bf16(acc[i][j + 1][rq * 4 + 2], acc[i][j + 1][rq * 4 + 3]);
                    vh[0] = pack2_bf16(hv[0], hv[1]);
                    vh[1] = pack2_bf16(hv[2], hv[3]);
                    *reinterpret_cast<u32x2 *>(p.C + m * p.ldc + n) = vg;
                    *reinterpret_cast<u32x2 *>(p.C1 + m * p.ldc + n) = vu;
                    *reinterpret_cast<u32x2 *>(p.C2 + m * p.ldc + n) = vh;
                }
            }
        }
    } else {  // EPI_SWIGLU_BWD
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int64_t m = static_cast<int64_t>(row_begin) + wm * WM + i * 32 + lrow;
            if (m >= row_end) continue;
#pragma unroll
            for (int j = 0; j < TN; j++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int n = n0 + wn * WN + j * 32 + rq * 8 + lcol;
                    float gv[4], uv[4], dg[4], du[4];
                    unpack4_bf16(*reinterpret_cast<const u32x2 *>(p.G + m * p.ldc + n), gv);
                    unpack4_bf16(*reinterpret_cast<const u32x2 *>(p.U + m * p.ldc + n), uv);
#pragma unroll
                    for (int x = 0; x < 4; x++) {
                        const float dh = acc[i][j][rq * 4 + x];
                        const float sg = 1.0f / (1.0f + __expf(-gv[x]));
                        du[x] = dh * (gv[x] * sg);
                        dg[x] = (dh * uv[x]) * (sg * (1.0f + gv[x] * (1.0f - sg)));
                    }
                    u32x2 vg, vu;
                    vg[0] = pack2_bf16(dg[0], dg[1]);
                    vg[1] = pack2_bf16(dg[2], dg[3]);
                    vu[0] = pack2_bf16(du[0], du[1]);
                    vu[1] = pack2_bf16(du[2], du[3]);
                    *reinterpret_cast<u32x2 *>(p.C + m * p.ldc + n) = vg;
                    *reinterpret_cast<u32x2 *>(p.C1 + m * p.ldc + n) = vu;
                }
            }
        }
    }
}

// ---- host side ---------------------------------------------------------------------------------

template <int BM, int BN, int WAVES_M, int WAVES_N, int AKIND, int BKIND, int EPI>
int launch(const GemmParams &p, dim3 grid, hipStream_t st) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int lds = 2 * (TileBytes<AKIND, BM>::value + TileBytes<BKIND, BN>::value);
    auto kern = ggemm_kernel<BM, BN, WAVES_M, WAVES_N, AKIND, BKIND, EPI>;
    static bool attr_set = false;  // one-time opt-in to > 64 KiB of dynamic LDS
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return OM_ERR_LAUNCH;
        attr_set = true;
    }
    kern<<<grid, dim3(NT), lds, st>>>(p);
    return om_launch_status();
}

inline bool mult(int64_t v, int m) { return v > 0 && v % m == 0; }

}  // namespace

// Tile shape used by the fwd / dgrad launches.
#define OM_BM 128
#define OM_BN 128

extern "C" int om_grouped_gemm_fwd(const void *input, const void *weight, void *output,
                                   const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                   int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(N, OM_BN) || !mult(K, BK)) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!input || !weight || !output || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(input) || !om_aligned16(weight) || !om_aligned16(output)) return OM_ERR_ALIGN;
    GemmParams p = {};
    p.A[0] = static_cast<const uint16_t *>(input);
    p.B[0] = static_cast<const uint16_t *>(weight);
    p.C = static_cast<uint16_t *>(output);
    p.cum = cum_token_counts;
    p.lda = K; p.ldb = K; p.ldc = N;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(N) * K;
    p.rows = rows; p.n_experts = G; p.n_cols = N; p.kc = K; p.phases = 1;
    p.m_tiles_max = static_cast<int>((rows + OM_BM - 1) / OM_BM + G);
    dim3 grid(static_cast<unsigned>(p.m_tiles_max) * (N / OM_BN));
    return launch<OM_BM, OM_BN, 2, 2, CONTIG, CONTIG, EPI_STORE>(p, grid, om_stream(stream));
}

extern "C" int om_grouped_gemm_dgrad(const void *output_grad, const void *weight, void *input_grad,
                                     const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                     int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(N, BK) || !mult(K, OM_BN)) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!output_grad || !weight || !input_grad || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(output_grad) || !om_aligned16(weight) || !om_aligned16(input_grad)) return OM_ERR_ALIGN;
    GemmParams p = {};
    p.A[0] = static_cast<const uint16_t *>(output_grad);
    p.B[0] = static_cast<const uint16_t *>(weight);
    p.C = static_cast<uint16_t *>(input_grad);
    p.cum = cum_token_counts;
    p.lda = N; p.ldb = K; p.ldc = K;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(N) * K;
    p.rows = rows; p.n_experts = G; p.n_cols = K; p.kc = N; p.phases = 1;
    p.m_tiles_max = static_cast<int>((rows + OM_BM - 1) / OM_BM + G);
    dim3 grid(static_cast<unsigned>(p.m_tiles_max) * (K / OM_BN));
    return launch<OM_BM, OM_BN, 2, 2, CONTIG, STRIDED, EPI_STORE>(p, grid, om_stream(stream));
}

extern "C" int om_grouped_gemm_wgrad(const void *output_grad, const void *input, void *weight_grad,
                                     const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                     int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(N, OM_BM) || !mult(K, OM_BN)) return OM_ERR_SHAPE;
    if (!output_grad || !input || !weight_grad || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(output_grad) || !om_aligned16(input) || !om_aligned16(weight_grad)) return OM_ERR_ALIGN;
    GemmParams p = {};
    p.A[0] = static_cast<const uint16_t *>(output_grad);  // [rows, N]: operand rows = n, c = row
    p.B[0] = static_cast<const uint16_t *>(input);        // [rows, K]
    p.C = static_cast<uint16_t *>(weight_grad);           // [G, N, K]
    p.cum = cum_token_counts;
    p.lda = N; p.ldb = K; p.ldc = K;
    p.strideC = w_stride ? w_stride : static_cast<int64_t>(N) * K;
    p.rows = rows; p.n_experts = G; p.n_cols = K; p.kc = N; p.phases = 1;
    dim3 grid(static_cast<unsigned>((N / OM_BM) * (K / OM_BN)), static_cast<unsigned>(G));
    return launch<OM_BM, OM_BN, 2, 2, STRIDED, STRIDED, EPI_WGRAD>(p, grid, om_stream(stream));
}

extern "C" int om_merged_mlp_gate_up_fwd(const void *x, const void *w_gate, const void *w_up, void *g,
                                         void *u, void *h, const int32_t *cum_token_counts,
                                         int64_t rows, int G, int I, int H, int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(I, OM_BN / 2) || !mult(H, BK)) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!x || !w_gate || !w_up || !g || !u || !h || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(x) || !om_aligned16(w_gate) || !om_aligned16(w_up) || !om_aligned16(g) ||
        !om_aligned16(u) || !om_aligned16(h))
        return OM_ERR_ALIGN;
    GemmParams p = {};
    p.A[0] = static_cast<const uint16_t *>(x);
    p.B[0] = static_cast<const uint16_t *>(w_gate);
    p.B[1] = static_cast<const uint16_t *>(w_up);
    p.C = static_cast<uint16_t *>(g);
    p.C1 = static_cast<uint16_t *>(u);
    p.C2 = static_cast<uint16_t *>(h);
    p.cum = cum_token_counts;
    p.lda = H; p.ldb = H; p.ldc = I;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(I) * H;
    p.rows = rows; p.n_experts = G; p.n_cols = I; p.kc = H; p.phases = 1;
    p.m_tiles_max = static_cast<int>((rows + OM_BM - 1) / OM_BM + G);
    dim3 grid(static_cast<unsigned>(p.m_tiles_max) * (I / (OM_BN / 2)));
    return launch<OM_BM, OM_BN, 2, 2, CONTIG, CONTIG, EPI_SWIGLU>(p, grid, om_stream(stream));
}

extern "C" int om_merged_mlp_down_dgrad(const void *dy, const void *w_down, const void *g, const void *u,
                                        void *dg, void *du, const int32_t *cum_token_counts,
                                        int64_t rows, int G, int I, int H, int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(I, OM_BN) || !mult(H, BK)) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!dy || !w_down || !g || !u || !dg || !du || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(dy) || !om_aligned16(w_down) || !om_aligned16(g) || !om_aligned16(u) ||
        !om_aligned16(dg) || !om_aligned16(du))
        return OM_ERR_ALIGN;
    GemmParams p = {};
    p.A[0] = static_cast<const uint16_t *>(dy);      // [rows, H]
    p.B[0] = static_cast<const uint16_t *>(w_down);  // [G, H, I]: c = h, operand row = i
    p.C = static_cast<uint16_t *>(dg);
    p.C1 = static_cast<uint16_t *>(du);
    p.G = static_cast<const uint16_t *>(g);
    p.U = static_cast<const uint16_t *>(u);
    p.cum = cum_token_counts;
    p.lda = H; p.ldb = I; p.ldc = I;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(H) * I;
    p.rows = rows; p.n_experts = G; p.n_cols = I; p.kc = H; p.phases = 1;
    p.m_tiles_max = static_cast<int>((rows + OM_BM - 1) / OM_BM + G);
    dim3 grid(static_cast<unsigned>(p.m_tiles_max) * (I / OM_BN));
    return launch<OM_BM, OM_BN, 2, 2, CONTIG, STRIDED, EPI_SWIGLU_BWD>(p, grid, om_stream(stream));
}

extern "C" int om_merged_mlp_gate_up_dgrad(const void *dg, const void *du, const void *w_gate,
                                           const void *w_up, void *dx, const int32_t *cum_token_counts,
                                           int64_t rows, int G, int I, int H, int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(I, BK) || !mult(H, OM_BN)) return OM_ERR_SHAPE;
    if (rows == 0) return OM_OK;
    if (!dg || !du || !w_gate || !w_up || !dx || !cum_token_counts) return OM_ERR_NULL;
    if (!om_aligned16(dg) || !om_aligned16(du) || !om_aligned16(w_gate) || !om_aligned16(w_up) ||
        !om_aligned16(dx))
        return OM_ERR_ALIGN;
    GemmParams p = {};
    p.A[0] = static_cast<const uint16_t *>(dg);
    p.A[1] = static_cast<const uint16_t *>(du);
    p.B[0] = static_cast<const uint16_t *>(w_gate);  // [G, I, H]: c = i, operand row = h
    p.B[1] = static_cast<const uint16_t *>(w_up);
    p.C = static_cast<uint16_t *>(dx);
    p.cum = cum_token_counts;
    p.lda = I; p.ldb = H; p.ldc = H;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(I) * H;
    p.rows = rows; p.n_experts = G; p.n_cols = H; p.kc = I; p.phases = 2;
    p.m_tiles_max = static_cast<int>((rows + OM_BM - 1) / OM_BM + G);
    dim3 grid(static_cast<unsigned>(p.m_tiles_max) * (H / OM_BN));
    return launch<OM_BM, OM_BN, 2, 2, CONTIG, STRIDED, EPI_STORE>(p, grid, om_stream(stream));
}
