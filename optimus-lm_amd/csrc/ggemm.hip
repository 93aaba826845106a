// Grouped expert GEMMs on bf16 MFMA (v_mfma_f32_32x32x16_bf16), fp32 accumulation.
//
// One kernel template covers every product of the merged MLP.  An output tile BM x BN is
// computed by WAVES_M x WAVES_N wavefronts; each wavefront owns a (BM/WAVES_M) x (BN/WAVES_N)
// sub-tile as a grid of 32x32 MFMA accumulators.  Operands are staged through LDS in steps of
// 64 along the contraction index c with direct global->LDS loads (global_load_lds_dwordx4: no
// register staging, no ds_write), two LDS stages, one barrier per step: the loads of step s+1
// are in flight while step s is multiplied.
//
// An operand is either
//   CONTIG  — stored [row][c] with c contiguous (activations in fwd/dgrad, weights in fwd):
//             LDS keeps 128-byte rows with the 16-byte chunks XOR-permuted per row; a fragment
//             is one ds_read_b128 per lane;
//   STRIDED — stored [c][row] with row contiguous (weights in dgrad, both operands in wgrad):
//             LDS keeps the tile as it lies in memory (chunks XOR-permuted per c-row); fragments
//             come from the gfx950 transposing LDS read (ds_read_b64_tr_b16), two per lane.
// A direct load writes LDS at (wave-uniform base + lane*16), so the permutation is applied by
// choosing which global chunk each lane fetches.  The per-lane order of the 8 contraction
// indices is the same for both kinds, so they can be mixed in one MFMA.
//
// Variable rows per expert: the M extent of fwd/dgrad is cut into tiles per expert.  Each block
// scans the device-resident cum_token_counts once into an LDS table (row tiles up to and including
// each expert) and looks its (expert, row block) up there per tile, so no host copy of the counts
// and no max-rows-per-expert is needed, and the blocks share out the tiles that really exist.  In wgrad the rows are the
// contraction range of expert g; rows past its end are zero-filled in LDS.
//
// Block order: consecutive block ids go to different XCDs (8 per chip, each with its own L2), so
// block ids are remapped to give every XCD a contiguous run of tiles, which share operand tiles.
//
// Two things that surround the expert GEMMs in the layer are folded into them (template parameters
// GATHER and ROWW): the token gather (an operand's rows are fetched through an index: the A rows of
// fwd/dgrad, or the contraction rows of either operand in wgrad), and the routing weight of the
// combine (the SwiGLU epilogue scales h by the weight of its row; the SwiGLU-backward epilogue
// scales dh by it and produces the per-row sums that make up the weight's gradient).
#include "common.h"

namespace {

enum { CONTIG = 0, STRIDED = 1 };
// An operand's rows can be taken through an index instead of in order: the token gather that
// precedes the expert GEMMs (ggemm_input = hidden_states[input_indices]) folded into the loads.
enum {
    GATHER_NONE = 0,
    GATHER_A = 1,    // fwd/dgrad: A rows
    GATHER_B = 2,    // wgrad: contraction rows of B
    GATHER_WA = 3    // wgrad: contraction rows of A
};
enum {
    EPI_STORE = 0,        // C = acc
    EPI_SWIGLU = 1,       // even 32-col accumulators = gate, odd = up: store g, u, h
    EPI_SWIGLU_BWD = 2,   // acc = dh: read g,u, store dg, du
    EPI_WGRAD = 3         // C[g] = acc, no row masking
};

constexpr int BK = 64;  // contraction step, elements
// Shares (in eighths) of a step's direct loads issued after the barrier / with 16-slices 0, 1, 2 of
// the step.  Forward and input-gradient products (row-major activations): the A loads right after
// the barrier, the B loads behind the first MFMAs.  Weight gradients (both operands read along the
// contraction rows): the A loads behind the first MFMAs, the B loads one slice later.  Measured per
// kernel on one box: the weight gradients gain 4 % with their split and the others lose 1-2 % with
// it; an even spread over the step, everything in one place, or cutting through the A loads are
// all 2-7 % worse on the whole layer.
constexpr int LD_SHARE_T = 4, LD_SHARE_0 = 4, LD_SHARE_1 = 0, LD_SHARE_2 = 0;       // fwd / dgrad
constexpr int LDW_SHARE_T = 0, LDW_SHARE_0 = 4, LDW_SHARE_1 = 4, LDW_SHARE_2 = 0;   // wgrad
constexpr int NUM_XCD = 8;

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
    const int32_t *row_index;   // GATHER_A: A row of sorted row r; GATHER_B / GATHER_WA: B / A row of contraction row c
    // ROWW kernels (the routing weight folded into the expert MLP):
    const float *row_scale;     // [rows] weight of each sorted row
    float *row_dot;             // EPI_SWIGLU_BWD: [n_cols / COLS][rows] partial sums of dh * silu(g) * u
    int64_t lda, ldb, ldc;      // leading dimensions, elements
    int64_t strideB, strideC;   // per-expert strides, elements
    int64_t rows;               // allocated activation rows (upper bound of cum[G])
    int n_experts;
    int n_cols;                 // output columns (fwd/dgrad) — tiles along N = n_cols / BN_OUT
    int kc;                     // contraction length per phase (fwd/dgrad), multiple of 8
    int phases;                 // 1 or 2
    int m_tiles_max;            // fwd/dgrad: upper bound on row tiles
    int total_tiles;            // logical tiles of the launch (the blocks loop over them)
    int tiles_e;                // wgrad: tiles per expert
};

typedef __attribute__((address_space(3))) s16x4 *lds_s16x4_ptr;
typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef const __attribute__((address_space(1))) void *glb_void_ptr;

// 16 bytes global -> LDS; LDS address = lds_base (wave-uniform) + lane*16.
__device__ __forceinline__ void load16_to_lds(const void *gptr, char *lds_base) {
    __builtin_amdgcn_global_load_lds((glb_void_ptr)gptr, (lds_void_ptr)lds_base, 16, 0, 0);
}

// A block-uniform 64-bit value, pinned to scalar registers (the compiler cannot always prove that
// per-tile state carried around the tile loop is uniform).
__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(static_cast<uint64_t>(v) >> 32));
    return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

// ---- CONTIG tile: R rows x 64 c; 128-byte rows; chunk position = chunk ^ swz(row) ----------
// (row >> 1) & 7: measured conflict-free for ds_read_b128 with 32 consecutive rows per half-wave
// (counter SQ_LDS_BANK_CONFLICT = 0, 4 cycles per read); period 16, so rows 32 apart share it.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int contig_off(int row, int ch) { return row * 128 + ((ch ^ swz(row)) << 4); }

// The chunk (8 contraction indices) that lane `lane` of direct load `grp` of a CONTIG tile fetches: the
// load fills LDS rows grp*8 .. grp*8+7, lane -> (row grp*8 + lane/8, position lane%8 = chunk ^ swz(row)).
__device__ __forceinline__ int contig_chunk(int grp, int lane) { return (lane & 7) ^ ((grp * 4 + (lane >> 4)) & 7); }

// ---- STRIDED tile: 64 c-rows x R rows-of-the-operand; R*2-byte c-rows; chunk position =
//      chunk ^ ((crow & 3) << 2): the four c-rows a transposing read touches land in four
//      different 64-byte bank windows -------------------------------------------------------
template <int R> __device__ __forceinline__ int strided_off(int crow, int ch) {
    return crow * (R * 2) + ((ch ^ ((crow & 3) << 2)) << 4);
}

template <int KIND, int R> struct TileBytes { static constexpr int value = R * 128; };  // both kinds

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
    const int m = m0 + mb + 4 * q;
    const int cr = c0 + 8 * g2 + r;  // (cr & 3) == (cr + 4) & 3
    const char *p = tile + strided_off<R>(cr, m >> 3) + (m & 7) * 2;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * R * 2));
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

// 1 / (1 + e^-x) with the hardware exponential and reciprocal (about 1 ulp each, far inside one
// bf16 rounding of the results it feeds).  An IEEE division here costs ten instructions per
// element, and the SwiGLU epilogues are bound by vector-ALU issue.
__device__ __forceinline__ float fast_sigmoid(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}

// Sum over aligned groups of N neighbouring lanes (N = 4, 8 or 16); every lane of the group gets
// it.  DPP: swap within pairs, swap pairs within quads, mirror within 8, mirror within 16.
template <int CTRL> __device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
template <int N> __device__ __forceinline__ float lane_group_sum(float v) {
    static_assert(N == 4 || N == 8 || N == 16, "group size");
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    if (N >= 8) v += dpp_move<0x141>(v);
    if (N >= 16) v += dpp_move<0x140>(v);
    return v;
}

__device__ __forceinline__ void unpack4_bf16(u32x2 v, float *f) {
    f[0] = __uint_as_float(v[0] << 16);
    f[1] = __uint_as_float(v[0] & 0xffff0000u);
    f[2] = __uint_as_float(v[1] << 16);
    f[3] = __uint_as_float(v[1] & 0xffff0000u);
}

// Row tiles of fwd/dgrad are cut per expert (BM rows each, the last one of an expert partial).
// One wavefront builds, once per block, a table in LDS from the device-resident cum_token_counts:
// tile_end[e] = number of row tiles of experts 0..e, seg[e] = cum_token_counts[e].
constexpr int MAX_EXPERTS = 1024;
template <int BM>
__device__ __forceinline__ void build_tile_table(const int32_t *cum, int n_experts, int lane,
                                                 int *tile_end, int *seg) {
    int base_tiles = 0;
    for (int e0 = 0; e0 < n_experts; e0 += 64) {
        const int e = e0 + lane;
        int s = 0, cnt = 0;
        if (e < n_experts) { s = cum[e]; cnt = cum[e + 1] - s; }
        int incl = (cnt + BM - 1) / BM;  // inclusive scan over the wavefront
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o, 64);
            if (lane >= o) incl += v;
        }
        if (e < n_experts) {
            tile_end[e] = base_tiles + incl;
            seg[e] = s;
            if (e == n_experts - 1) seg[n_experts] = s + cnt;
        }
        base_tiles += __shfl(incl, 63, 64);
    }
}

// Which expert owns row tile `tile`, and which rows are the tile's?  False past the last tile.
template <int BM>
__device__ __forceinline__ bool find_tile(const int *tile_end, const int *seg, int n_experts, int tile,
                                          int lane, int &expert, int &row_begin, int &row_end) {
    for (int e0 = 0; e0 < n_experts; e0 += 64) {
        const int e = e0 + lane;
        const bool mine = e < n_experts && tile < tile_end[e];   // tile_end is non-decreasing
        const unsigned long long vote = __ballot(mine);
        if (vote) {
            expert = e0 + __ffsll(static_cast<long long>(vote)) - 1;
            const int first = expert > 0 ? tile_end[expert - 1] : 0;
            row_begin = seg[expert] + (tile - first) * BM;
            row_end = seg[expert + 1];
            return true;
        }
    }
    return false;
}

// Weight gradient: the tiles of expert e cost about (contraction steps of e + a few steps' worth of
// epilogue) each, so with skewed routing equal tile counts per XCD are far from equal work.  The
// tiles are numbered expert-major; boundary j of 0..8 is the tile at which j/8 of the launch's work
// lies behind, and XCD x takes the run [boundary x, boundary x+1).  A boundary that falls within an
// eighth of an XCD's share of an expert's first or last tile moves there: all tiles of dW[g] share
// the expert's rows of both operands, and with near-uniform routing whole experts per XCD (what
// equal tile counts give) is the better cut.  Every wavefront computes the two boundaries it needs
// by itself from cum_token_counts (two strided passes, no LDS, no barrier).
constexpr int WGRAD_EPILOGUE_STEPS = 3;   // a tile's stores take about as long as 3 steps
constexpr int WGRAD_BALANCE_MAX_EXPERTS = 4096;
__device__ __forceinline__ int wgrad_tile_units(int rows, int bk) {
    const int steps = (rows + bk - 1) / bk;
    return steps + WGRAD_EPILOGUE_STEPS;
}
__device__ __forceinline__ void wgrad_xcd_run(const int32_t *cum, int n_experts, int tiles_e, int bk, int xcd,
                                              int n_xcd, int lane, int &lo, int &hi) {
    int mine = 0;
    for (int e = lane; e < n_experts; e += 64) mine += wgrad_tile_units(cum[e + 1] - cum[e], bk);
    const long long work = static_cast<long long>(wave_sum_i(mine)) * tiles_e;
    const long long t_lo = work * xcd / n_xcd, t_hi = work * (xcd + 1) / n_xcd;
    lo = 0;
    hi = n_experts * tiles_e;
    int base = 0;   // units of the experts before this chunk
    for (int e0 = 0; e0 < n_experts; e0 += 64) {
        const int e = e0 + lane;
        const int u = e < n_experts ? wgrad_tile_units(cum[e + 1] - cum[e], bk) : 0;
        int incl = u;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o, 64);
            if (lane >= o) incl += v;
        }
        const long long before = static_cast<long long>(base + incl - u) * tiles_e;
        const long long after = before + static_cast<long long>(u) * tiles_e;
        // exactly one expert of the launch holds a target below the total; the total itself
        // (boundary n_xcd) keeps the initial value of hi
        const bool has_lo = u > 0 && t_lo >= before && t_lo < after;
        const bool has_hi = u > 0 && t_hi >= before && t_hi < after;
        const long long snap = work / (n_xcd * 8);
        auto cut = [&](long long t) -> int {   // tile of this expert at which work t lies behind
            if (t - before <= after - t) {
                if (t - before <= snap) return e * tiles_e;
            } else if (after - t <= snap) {
                return (e + 1) * tiles_e;
            }
            return e * tiles_e + static_cast<int>((t - before) / (u > 0 ? u : 1));
        };
        const int tile_lo = cut(t_lo), tile_hi = cut(t_hi);
        const unsigned long long m_lo = __ballot(has_lo), m_hi = __ballot(has_hi);
        if (m_lo) lo = __shfl(tile_lo, __ffsll(static_cast<long long>(m_lo)) - 1, 64);
        if (m_hi) hi = __shfl(tile_hi, __ffsll(static_cast<long long>(m_hi)) - 1, 64);
        base += __shfl(incl, 63, 64);
    }
    if (xcd == 0) lo = 0;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int AKIND, int BKIND, int EPI, int GATHER = GATHER_NONE,
          bool ROWW = false, bool ACCUM = false, bool KTAIL = false, bool REGLOAD = false>
// (second launch bound: two wavefronts per SIMD, i.e. at most 256 registers, for the 128x128 tile, whose two
// blocks per CU depend on it; the 256x256 tile's 8 wavefronts imply it already)
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64, BM == 128 ? 2 : 1) void ggemm_kernel(const GemmParams p) {
    static_assert(!ACCUM || EPI == EPI_WGRAD, "only the weight gradient adds into its output");
    // KTAIL: forward / input-gradient products whose contraction length is not a multiple of 64 (the last
    // step of a phase is partial); a kernel of its own, so that the others carry none of its handling
    static_assert(!KTAIL || (BM == 128 && EPI != EPI_WGRAD && AKIND == CONTIG), "partial last contraction step: 128x128 forward / input gradient");
    // REGLOAD: forward / input-gradient products whose experts hold few rows, where a launch is a stream of
    // weights that are used once.  Both operands go through registers instead of direct global->LDS loads: the
    // weights (B) are fetched TWO contraction steps ahead into two register sets, the activations (A, which
    // mostly hit in L2) one step ahead, and are written to the LDS stage that has become free before the
    // barrier that ends a step.  With direct loads the look-ahead cannot exceed one step: the compiler
    // waits for every outstanding load before a barrier, since it cannot tell which LDS bytes a direct load
    // in flight will write.  Same LDS layout, same order of the sums: bit-identical results.
    static_assert(!REGLOAD || (BM == 128 && EPI != EPI_WGRAD && !KTAIL), "register-staged operands: 128x128 forward / input gradient");
    static_assert(GATHER == GATHER_NONE || (GATHER == GATHER_A && AKIND == CONTIG && EPI != EPI_WGRAD) ||
                      (GATHER == GATHER_B && BKIND == STRIDED && EPI == EPI_WGRAD) ||
                      (GATHER == GATHER_WA && AKIND == STRIDED && EPI == EPI_WGRAD), "gather variants");
    static_assert(!ROWW || EPI == EPI_SWIGLU || EPI == EPI_SWIGLU_BWD, "row weights belong to the SwiGLU epilogues");
    constexpr int NW = WAVES_M * WAVES_N;
    // The 128x128 tile takes output extents that are any multiple of 8: its last tile along an
    // extent may be partial (loads past the extent are clamped, stores masked).  The 256x256 tile is
    // only launched on whole tiles and carries none of that.
    constexpr bool EDGE = BM == 128;
    // Contraction steps are taken in pairs (static stage names).  The weight gradient, whose step
    // count follows the expert's rows, and the 128x128 tile end an odd count with a single step; the
    // 256x256 forward / input-gradient kernels are only launched on even counts.
    constexpr bool ANY_STEPS = EPI == EPI_WGRAD || EDGE;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wavefront sub-tile
    constexpr int TM = WM / 32, TN = WN / 32;            // 32x32 accumulators per wavefront
    constexpr int A_BYTES = TileBytes<AKIND, BM>::value;
    constexpr int B_BYTES = TileBytes<BKIND, BN>::value;
    constexpr int A_LOADS = BM / 8 / NW;                 // direct loads per wavefront per step
    constexpr int B_LOADS = BN / 8 / NW;
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile/wave mismatch");
    // two statically distinct stages: the compiler can then tell that a fragment read of one
    // stage does not depend on the loads in flight to the other
    __shared__ __attribute__((aligned(1024))) char stage0[A_BYTES + B_BYTES];
    __shared__ __attribute__((aligned(1024))) char stage1[A_BYTES + B_BYTES];
    // wgrad through an index: the current expert's slice of the index is kept in LDS (filled when
    // the block moves to another expert) for the look-up that a tile's first loads wait for; the
    // look-ups inside the main loop run one step ahead and go to global memory (reading them from
    // LDS measured 20 % slower: they queue with the fragment reads)
    constexpr bool GATHER_W = GATHER == GATHER_B || GATHER == GATHER_WA;
    constexpr int IDX_CACHE = GATHER_W ? (BM == 256 ? 4096 : 2048) : 1;
    __shared__ int idx_cache[IDX_CACHE];
    int cached_expert = -1;
    __shared__ int tile_end[EPI == EPI_WGRAD ? 1 : MAX_EXPERTS];   // see build_tile_table
    __shared__ int seg[EPI == EPI_WGRAD ? 1 : MAX_EXPERTS + 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);   // the same value in a scalar register

    // ---- per-tile state (set by setup_tile) ---------------------------------------------------
    int expert = 0, row_begin = 0, row_end = 0;  // fwd/dgrad: rows of this tile's expert segment
    int n0 = 0;                                  // first output column (LDS B row 0)
    int c_begin = 0, c_len = 0;                  // contraction range
    int steps_per_phase = 0, total_steps = 0;
    int loop_steps = 0;   // steps the main loop takes (see setup_tile)
    // Tiles that run together on an XCD share operand slices.  Walking the contraction index from
    // 0 in all of them makes them ask L2 for the same lines at the same time, and all wait for the
    // same fill; a small per-tile offset `rot` lets one tile fetch a slice and the sharers hit it.
    int rot = 0;
    auto rotated = [&](int sp) {   // sp in [0, steps_per_phase)
        const int r = sp + rot;
        return r >= steps_per_phase ? r - steps_per_phase : r;
    };

    // ---- per-lane source offsets of the direct loads (elements, without the c0 term) ------------
    // CONTIG : lane -> (row = group*8 + lane/8, chunk = (lane%8) ^ swz(row))
    // STRIDED: lane -> (crow = group*(64/CPR) + lane/CPR, chunk = (lane%CPR) ^ ((crow&3)<<2))
    // A load's address is (operand pointer + block-uniform 64-bit tile base) + a 32-bit per-lane
    // offset: the wide part stays in scalar registers (the load takes a scalar base and a 32-bit
    // vector offset), so operands of any size cost no vector arithmetic.  The per-lane part covers
    // one tile (BM rows, or 64 contraction rows) — except for rows fetched through an index, whose
    // lane offset is index * pitch: such a source must span < 2^31 elements (checked on the host).
    int a_off[A_LOADS], b_off[B_LOADS];
    int64_t a_base = 0, b_base = 0;   // elements, block-uniform
    int a_crow[A_LOADS];  // STRIDED A in wgrad: c-row of the lane's slot (for the zero fill)
    int b_crow[B_LOADS];
    int b_src[GATHER == GATHER_B ? B_LOADS : 1];   // GATHER_B: source rows of the next B loads
    int a_src[GATHER == GATHER_WA ? A_LOADS : 1];  // GATHER_WA: source rows of the next A loads
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
        constexpr int CPR = BM / 8;
        a_crow[i] = (AKIND == CONTIG) ? 0 : (wave * A_LOADS + i) * (64 / CPR) + lane / CPR;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
        constexpr int CPR = BN / 8;
        const int grp = wave * B_LOADS + i;
        b_crow[i] = (BKIND == CONTIG) ? 0 : grp * (64 / CPR) + lane / CPR;
    }

    const int lda32 = static_cast<int>(p.lda), ldb32 = static_cast<int>(p.ldb);
    // GATHER_B: the B rows that contraction step `step` needs, looked up one step ahead of the
    // loads that use them (plain loads: they land before the next wait for the direct loads).
    auto index_of = [&](int step, int c0, int c) -> int {   // c0: the step's first row (block-uniform)
        if (step == 0 && c0 + BK <= IDX_CACHE) return idx_cache[GATHER_W ? c : 0];
        return p.row_index[c_begin + c];
    };
    auto load_b_src = [&](int step) {
        if (GATHER != GATHER_B || step >= loop_steps) return;
        const int c0 = (step < steps_per_phase ? rotated(step) : step) * BK;
        // One 4-byte read per B load (measured faster than one read per wavefront plus lane
        // permutes, which queue behind the fragment reads).  Kept as read: any arithmetic on the
        // value here would put the wait for it here too.
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) {
            const int c = min(c0 + b_crow[i], c_len - 1);   // past the segment: any valid row (A is zeroed)
            b_src[GATHER == GATHER_B ? i : 0] = index_of(step, c0, c);
        }
    };

    auto load_a_src = [&](int step) {   // GATHER_WA: the same for the A rows
        if (GATHER != GATHER_WA || step >= loop_steps) return;
        const int c0 = (step < steps_per_phase ? rotated(step) : step) * BK;
#pragma unroll
        for (int i = 0; i < A_LOADS; i++) {
            const int c = min(c0 + a_crow[i], c_len - 1);   // past the segment: any valid row (zeroed in LDS)
            a_src[GATHER == GATHER_WA ? i : 0] = index_of(step, c0, c);
        }
    };

    // Which tile `logical` is, and the load offsets for it.  False: the tile lies past the last
    // row block (the launch sizes the tile count from an upper bound on the routed rows).
    auto setup_tile = [&](int logical) -> bool {
        int rot_a, rot_b;  // position among the tiles sharing this tile's A / B operand
        // lane-derived terms are recomputed per tile rather than kept live across the main loop
        int lane_s = lane;
        asm volatile("" : "+v"(lane_s));
        if (EPI == EPI_WGRAD) {
            // tiles are numbered expert-major: an XCD works on whole experts (all tiles of dW[g]
            // share the expert's rows of both operands)
            const int tiles_n = (p.n_cols + BN - 1) / BN;
            expert = logical / p.tiles_e;
            const int tile = logical - expert * p.tiles_e;
            const int tm = tile / tiles_n, tn = tile % tiles_n;
            rot_a = tn; rot_b = tm;
            row_begin = tm * BM;  // row of dW
            row_end = 0;
            n0 = tn * BN;
            c_begin = p.cum[expert];
            c_len = p.cum[expert + 1] - c_begin;
        } else {
            constexpr int BN_OUT = (EPI == EPI_SWIGLU) ? BN / 2 : BN;
            const int tiles_n = (p.n_cols + BN_OUT - 1) / BN_OUT;
            const int tile_m = logical / tiles_n;
            const int tile_n = logical % tiles_n;
            rot_a = tile_n; rot_b = tile_m & 7;
            if (!find_tile<BM>(tile_end, seg, p.n_experts, tile_m, lane_s, expert, row_begin, row_end)) return false;
            n0 = tile_n * BN_OUT;
            c_begin = 0;
            c_len = p.kc;
        }
        // block-uniform values: keep them in scalar registers
        expert = __builtin_amdgcn_readfirstlane(expert);
        row_begin = __builtin_amdgcn_readfirstlane(row_begin);
        row_end = __builtin_amdgcn_readfirstlane(row_end);
        n0 = __builtin_amdgcn_readfirstlane(n0);
        c_begin = __builtin_amdgcn_readfirstlane(c_begin);
        c_len = __builtin_amdgcn_readfirstlane(c_len);
        steps_per_phase = (c_len + BK - 1) / BK;
        total_steps = steps_per_phase * p.phases;
        loop_steps = ANY_STEPS ? total_steps : ((total_steps + 1) & ~1);
        rot = (rot_a + rot_b) % (steps_per_phase > 0 ? steps_per_phase : 1);
#pragma unroll
        for (int i = 0; i < A_LOADS; i++) {
            const int grp = wave * A_LOADS + i;
            if (AKIND == CONTIG) {
                const int row = grp * 8 + (lane_s >> 3);
                const int ch = (lane_s & 7) ^ swz(row);
                int m = row_begin + row;
                if (m >= row_end) m = row_end - 1;  // rows past the segment: valid memory, result unused
                if (GATHER == GATHER_A) m = p.row_index[m];
                else m -= row_begin;                // the tile's first row is part of a_base
                a_off[i] = m * lda32 + ch * 8;
            } else {
                constexpr int CPR = BM / 8;
                const int ch = (lane_s % CPR) ^ ((a_crow[i] & 3) << 2);
                // (a partial last tile: chunks past the extent re-read its last chunk; masked on store)
                a_off[i] = EDGE ? min(row_begin + ch * 8, p.kc - 8) : row_begin + ch * 8;  // + (contraction row within the step) * lda per step
            }
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) {
            const int grp = wave * B_LOADS + i;
            if (BKIND == CONTIG) {
                const int row = grp * 8 + (lane_s >> 3);
                const int ch = (lane_s & 7) ^ swz(row);
                // output columns past n_cols (a partial last column tile) re-read the last one; their
                // results are masked on store
                const int n_last = EDGE ? p.n_cols - 1 - n0 : BN;
                if (EPI == EPI_SWIGLU) {
                    // LDS rows alternate 32 gate rows / 32 up rows; the up matrix is B[1]
                    const int blk = row >> 5;
                    const int n = (blk >> 1) * 32 + (row & 31);
                    b_off[i] = min(n, n_last) * ldb32 + ch * 8;
                } else {
                    b_off[i] = min(row, n_last) * ldb32 + ch * 8;
                }
            } else {
                constexpr int CPR = BN / 8;
                const int ch = (lane_s % CPR) ^ ((b_crow[i] & 3) << 2);
                const int col8 = EDGE ? min(ch * 8, p.n_cols - 8 - n0) : ch * 8;   // (partial last column tile, as above)
                // fwd/dgrad: the lane's contraction row within a step never changes, so it is part of
                // the offset; wgrad clamps the row into the expert's segment per step
                b_off[i] = col8 + (EPI == EPI_WGRAD ? 0 : b_crow[i] * ldb32);
            }
        }
        // block-uniform parts of the addresses (scalar registers)
        if (AKIND == CONTIG) a_base = GATHER == GATHER_A ? 0 : static_cast<int64_t>(row_begin) * p.lda;
        else a_base = 0;   // wgrad: the contraction rows enter per step (step_base)
        if (BKIND == CONTIG) b_base = expert * p.strideB + static_cast<int64_t>(n0) * p.ldb;
        else b_base = (EPI == EPI_WGRAD ? 0 : expert * p.strideB) + n0;
        if (GATHER_W && expert != cached_expert) {
            // every wavefront is past the barrier that ends the previous tile's main loop, so no
            // one still reads the cache; `expert` is block-uniform, so all take this branch together
            const int n_cached = min(c_len, IDX_CACHE);
            for (int i = tid; i < n_cached; i += NW * 64) idx_cache[GATHER_W ? i : 0] = p.row_index[c_begin + i];
            cached_expert = expert;
            __syncthreads();
        }
        load_b_src(0);
        load_a_src(0);
        return true;
    };

    // Loads of contraction step `step` into `stage`.
    // Loads [lo, hi) of the step's list (A loads first, then B loads); lo and hi are constants
    // after unrolling.
    u32x4 rb[REGLOAD ? 2 : 1][REGLOAD ? B_LOADS : 1];   // REGLOAD: B of steps s+1 and s+2 (set = step % 2)
    u32x4 ra[REGLOAD ? A_LOADS : 1];                    //          A of step s+1
    auto issue_part = [&](int step, char *stage, int lo, int hi) {
        if (REGLOAD) return;                               // (no direct loads in these kernels)
        if (step >= loop_steps) return;                    // nothing left to fetch for this tile
        const int ph = (step >= steps_per_phase) ? 1 : 0;  // at most two phases
        const int sp = step - ph * steps_per_phase;
        int c0 = (sp < steps_per_phase ? rotated(sp) : sp) * BK;
        if (!ANY_STEPS && c0 > c_len - BK) c0 = c_len - BK;
        // KTAIL kernels take contraction lengths that are any multiple of 8: the last step of a phase
        // may hold fewer than 64 indices.  Its loads past the end re-read the last valid 8 indices (c-row)
        // instead, and the A slots they fill are zeroed in LDS before the step is multiplied (zero_tail).
        const bool c_tail = KTAIL && c0 + BK > c_len;   // block-uniform
        const int c_chunks = (c_len - c0) >> 3;                           // 8-index chunks the step holds
        // first contraction row that this step's STRIDED loads may touch, folded into the scalar base
        // (rows are clamped into the segment, so the base is clamped the same way)
        const int c_lo = (EPI == EPI_WGRAD) ? max(min(c0, c_len - 1), 0) : c0;
        const int64_t a_step = uniform64(a_base + ((AKIND == STRIDED && GATHER != GATHER_WA) ? static_cast<int64_t>(c_begin + c_lo) * p.lda : 0));
        const int64_t b_step = uniform64(b_base + ((BKIND == STRIDED && GATHER != GATHER_B) ? static_cast<int64_t>(c_begin + c_lo) * p.ldb : 0));
        const char *Ap = reinterpret_cast<const char *>((p.phases > 1 && ph ? p.A[1] : p.A[0]) + a_step);
        const char *Bp = reinterpret_cast<const char *>(
            ((EPI != EPI_SWIGLU && p.phases > 1 && ph) ? p.B[1] : p.B[0]) + b_step);
        const char *Bup = reinterpret_cast<const char *>(p.B[1] + b_step);
        char *sa = stage + wave * (A_LOADS * 1024);
        char *sb = stage + A_BYTES + wave * (B_LOADS * 1024);
#pragma unroll
        for (int i = 0; i < A_LOADS; i++) {
            if (i < lo || i >= hi) continue;
            uint32_t off;  // bytes from the step's scalar base
            if (AKIND == CONTIG) {
                off = static_cast<uint32_t>(a_off[i] + c0) * 2u;
                if (c_tail) off -= static_cast<uint32_t>(max(contig_chunk(wave_u * A_LOADS + i, lane) - (c_chunks - 1), 0)) * 16u;
            } else {
                int c = c0 + a_crow[i];
                if (EPI == EPI_WGRAD) c = min(c, c_len - 1);  // stay in the segment; zeroed below
                if (GATHER == GATHER_WA)
                    off = static_cast<uint32_t>(a_off[i] + a_src[GATHER == GATHER_WA ? i : 0] * lda32) * 2u;
                else
                    off = static_cast<uint32_t>(a_off[i] + (c - c_lo) * lda32) * 2u;
            }
            load16_to_lds(Ap + off, sa + i * 1024);
        }
        if (hi >= A_LOADS && lo < A_LOADS) load_a_src(step + 1);   // this step's A loads are out
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) {
            if (A_LOADS + i < lo || A_LOADS + i >= hi) continue;
            uint32_t off;
            if (BKIND == CONTIG) {
                off = static_cast<uint32_t>(b_off[i] + c0) * 2u;
                if (c_tail) off -= static_cast<uint32_t>(max(contig_chunk(wave_u * B_LOADS + i, lane) - (c_chunks - 1), 0)) * 16u;
            } else {
                if (GATHER == GATHER_B) {
                    off = static_cast<uint32_t>(b_off[i] + b_src[GATHER == GATHER_B ? i : 0] * ldb32) * 2u;
                } else if (EPI == EPI_WGRAD) {
                    const int c = min(c0 + b_crow[i], c_len - 1);
                    off = static_cast<uint32_t>(b_off[i] + (c - c_lo) * ldb32) * 2u;
                } else {
                    // loop-invariant: kept opaque so that it stays a 32-bit register next to a scalar
                    // base (hoisted, it becomes a zero-extended 64-bit pair per load)
                    int o = b_off[i];
                    asm volatile("" : "+v"(o));
                    off = static_cast<uint32_t>(o) * 2u;
                    if (c_tail) off -= static_cast<uint32_t>(max(c0 + b_crow[i] - (c_len - 1), 0) * ldb32) * 2u;
                }
            }
            // EPI_SWIGLU: a load covers 8 LDS rows inside one 32-row block, all gate or all up rows, so
            // the choice of the matrix is uniform over the wavefront (scalar base, 32-bit lane offset)
            const bool up_rows = EPI == EPI_SWIGLU && ((((wave_u * B_LOADS + i) * 8) >> 5) & 1);
            load16_to_lds((up_rows ? Bup : Bp) + off, sb + i * 1024);
        }
        if (hi >= A_LOADS + B_LOADS && lo < A_LOADS + B_LOADS) load_b_src(step + 1);   // this step's B loads are out
    };
    constexpr int NL = A_LOADS + B_LOADS;
    auto issue_loads = [&](int step, char *stage) { issue_part(step, stage, 0, NL); };
    // REGLOAD: the loads of a step into registers, and from there into an LDS stage.  The loads are issued
    // unconditionally (past a tile's last step they re-read its last step, unused): inside a branch they
    // would make the compiler wait for all loads at the join, and the look-ahead would be gone.
    auto fetch_a = [&](int step) {
        if (!REGLOAD) return;
        step = min(step, loop_steps - 1);
        const int ph = (step >= steps_per_phase) ? 1 : 0;
        const int c0 = rotated(step - ph * steps_per_phase) * BK;
        const char *Ap = reinterpret_cast<const char *>((p.phases > 1 && ph ? p.A[1] : p.A[0]) + uniform64(a_base));
#pragma unroll
        for (int i = 0; i < A_LOADS; i++)
            ra[REGLOAD ? i : 0] = *reinterpret_cast<const u32x4 *>(Ap + static_cast<uint32_t>(a_off[i] + c0) * 2u);
    };
    auto fetch_b = [&](int step, int set) {
        if (!REGLOAD) return;
        step = min(step, loop_steps - 1);
        const int ph = (step >= steps_per_phase) ? 1 : 0;
        const int c0 = rotated(step - ph * steps_per_phase) * BK;
        const int64_t b_step = uniform64(b_base + (BKIND == STRIDED ? static_cast<int64_t>(c_begin + c0) * p.ldb : 0));
        const char *Bp = reinterpret_cast<const char *>(
            ((EPI != EPI_SWIGLU && p.phases > 1 && ph) ? p.B[1] : p.B[0]) + b_step);
        const char *Bup = reinterpret_cast<const char *>(p.B[1] + b_step);
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) {
            uint32_t off;
            if (BKIND == CONTIG) {
                off = static_cast<uint32_t>(b_off[i] + c0) * 2u;
            } else {
                int o = b_off[i];
                asm volatile("" : "+v"(o));
                off = static_cast<uint32_t>(o) * 2u;
            }
            const bool up_rows = EPI == EPI_SWIGLU && ((((wave_u * B_LOADS + i) * 8) >> 5) & 1);
            rb[REGLOAD ? set : 0][REGLOAD ? i : 0] = *reinterpret_cast<const u32x4 *>((up_rows ? Bup : Bp) + off);
        }
    };
    // (a wavefront writes the 1 KB blocks that its direct loads would fill: base + lane * 16)
    auto commit_a = [&](int step, char *stage) {
        if (!REGLOAD || step >= loop_steps) return;
        char *sa = stage + wave * (A_LOADS * 1024) + lane * 16;
#pragma unroll
        for (int i = 0; i < A_LOADS; i++) *reinterpret_cast<u32x4 *>(sa + i * 1024) = ra[REGLOAD ? i : 0];
    };
    auto commit_b = [&](int step, char *stage, int set) {
        if (!REGLOAD || step >= loop_steps) return;
        char *sb = stage + A_BYTES + wave * (B_LOADS * 1024) + lane * 16;
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) *reinterpret_cast<u32x4 *>(sb + i * 1024) = rb[REGLOAD ? set : 0][REGLOAD ? i : 0];
    };
    // The direct loads of a step are spread over the MFMAs of a whole step rather than issued in
    // one burst: the texture path of a CU accepts about one 1 KB load per wavefront every ~220
    // cycles, and a wavefront that has to wait for it cannot issue its MFMAs meanwhile.  Shares of
    // the NL loads: after the barrier of step s (stage free), then with slices 0, 1, 2 of step s+1.
    constexpr bool WG = EPI == EPI_WGRAD;
    constexpr int LD_T = NL * (WG ? LDW_SHARE_T : LD_SHARE_T) / 8, LD_0 = NL * (WG ? LDW_SHARE_0 : LD_SHARE_0) / 8;
    constexpr int LD_1 = NL * (WG ? LDW_SHARE_1 : LD_SHARE_1) / 8;
    constexpr int LD_2 = NL - LD_T - LD_0 - LD_1;
    static_assert(LD_SHARE_T + LD_SHARE_0 + LD_SHARE_1 + LD_SHARE_2 == 8 &&
                      LDW_SHARE_T + LDW_SHARE_0 + LDW_SHARE_1 + LDW_SHARE_2 == 8 && LD_2 >= 0, "load shares");
    // wgrad: zero the A c-rows past the end of the expert's rows (after the loads have landed,
    // before the barrier).  B holds finite in-segment data there, so the products vanish.
    auto zero_tail = [&](int step, char *stage) {
        if ((EPI != EPI_WGRAD && !KTAIL) || step >= loop_steps) return;   // (nothing was fetched for a step past the last)
        if (EPI != EPI_WGRAD) {
            // KTAIL: the last step of a phase holds fewer than 64 indices (A is CONTIG here): zero the
            // chunks past the end
            const int ph = (step >= steps_per_phase) ? 1 : 0;
            const int c0 = rotated(step - ph * steps_per_phase) * BK;
            if (c0 + BK <= c_len) return;
            const int c_chunks = (c_len - c0) >> 3;
            char *sa = stage + wave * (A_LOADS * 1024);
#pragma unroll
            for (int i = 0; i < A_LOADS; i++)
                if (contig_chunk(wave_u * A_LOADS + i, lane) >= c_chunks)
                    *reinterpret_cast<u32x4 *>(sa + i * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
            return;
        }
        const int c0 = (step < steps_per_phase ? rotated(step) : step) * BK;
        if (c0 + BK <= c_len) return;
        char *sa = stage + wave * (A_LOADS * 1024);
#pragma unroll
        for (int i = 0; i < A_LOADS; i++)
            if (c0 + a_crow[i] >= c_len)
                *reinterpret_cast<u32x4 *>(sa + i * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
    };

    f32x16 acc[TM][TN];

    // ---- fragment addresses (bytes within a stage), loop-invariant ------------------------------
    // CONTIG : addr(i, kk) = c_base + i*4096 + c_kofs[kk]      (rows i*32 apart share the swizzle)
    // STRIDED: addr(i, kk) = s_base[i] + kk*16*R*2 (+ 4*R*2 for the second transposing read)
    const int lrow32 = lane & 31, g2 = lane >> 5;
    int c_kofs[BK / 16];
#pragma unroll
    for (int kk = 0; kk < BK / 16; kk++) c_kofs[kk] = ((kk * 2 + g2) ^ swz(lrow32)) << 4;
    const int a_cbase = (wm * WM + lrow32) * 128;
    const int b_cbase = A_BYTES + (wn * WN + lrow32) * 128;
    int a_sbase[TM], b_sbase[TN];
    {
        const int i16 = lane & 15;
        const int r = i16 >> 2, q = i16 & 3, mb = ((lane >> 4) & 1) * 16;
        const int cr = 8 * g2 + r;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int m = wm * WM + i * 32 + mb + 4 * q;
            a_sbase[i] = strided_off<BM>(cr, m >> 3) + (m & 7) * 2;
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int m = wn * WN + j * 32 + mb + 4 * q;
            b_sbase[j] = A_BYTES + strided_off<BN>(cr, m >> 3) + (m & 7) * 2;
        }
    }
    typedef __attribute__((ext_vector_type(8))) short s16x8;
    auto read_a = [&](const char *stage, int i, int kk) -> bf16x8 {
        if (AKIND == CONTIG) {
            return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(stage + a_cbase + i * 4096 + c_kofs[kk]));
        } else {
            const char *ptr = stage + a_sbase[i] + kk * (16 * BM * 2);
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ptr));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ptr + 4 * BM * 2));
            return __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
    };
    auto read_b = [&](const char *stage, int j, int kk) -> bf16x8 {
        if (BKIND == CONTIG) {
            return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(stage + b_cbase + j * 4096 + c_kofs[kk]));
        } else {
            const char *ptr = stage + b_sbase[j] + kk * (16 * BN * 2);
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ptr));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ptr + 4 * BN * 2));
            return __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
    };

    // ---- main loop ------------------------------------------------------------------------------
    // Two LDS stages; the loads of step s+2 are issued as soon as every wavefront has taken its
    // last fragments of step s out of LDS.  Fragments are double buffered in registers: the reads
    // of 16-slice kk+1 are interleaved with the MFMAs of slice kk, and the first slice of the next
    // stage is read under the MFMAs of the last slice of this one, so the wavefront never waits on
    // LDS latency with an empty MFMA pipe.
    bf16x8 fa[2][TM], fb[2][TN];
    auto read_group = [&](const char *stage, int kk, int buf) {
#pragma unroll
        for (int i = 0; i < TM; i++) fa[buf][i] = read_a(stage, i, kk);
#pragma unroll
        for (int j = 0; j < TN; j++) fb[buf][j] = read_b(stage, j, kk);
    };
    auto mfma_group = [&](int buf) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                // operands swapped: the lane then holds 4 consecutive output columns per row
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
    };
    // Scheduling hint for one 16-slice: MFMA first, then the LDS reads of the next slice two at a
    // time behind the leading MFMAs, `nl` direct loads spread evenly, the remaining MFMAs last.
    // The wait for the previous slice's fragments then sits ahead of the first MFMA with no newer
    // LDS read in front of it (the compiler always waits for a zero LDS counter here because the
    // direct loads count as possible LDS accesses), and the last read of a slice has several MFMAs
    // behind it to hide its latency.
    constexpr int DS_READS = TM * (AKIND == CONTIG ? 1 : 2) + TN * (BKIND == CONTIG ? 1 : 2);
    auto interleave_loads = [&](int nl) {
        constexpr int NM = TM * TN;
        constexpr int DS_PER = (DS_READS + NM - 2) / (NM - 1) < 2 ? 2 : (DS_READS + NM - 2) / (NM - 1);
        int placed = 0, ds_left = DS_READS;
#pragma unroll
        for (int r = 0; r < NM; r++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                    // 1 MFMA
            // (the builtin wants literal counts; the conditions fold after unrolling)
#pragma unroll
            for (int q = 0; q < DS_PER; q++)
                if (ds_left > 0) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); ds_left--; }
            const int want = ((r + 1) * nl + NM - 1) / NM;   // loads due by now
            if (want - placed >= 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // 1 VMEM read
            if (want - placed >= 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            if (want - placed >= 3) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            if (want - placed >= 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            placed = want;
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto interleave = [&]() { interleave_loads(0); };
    // one contraction step on `cur`; `nxt` holds step s+1 when this returns (par = s % 2)
    auto half_step = [&](char *cur, char *nxt, int s, int par) {
#pragma unroll
        for (int kk = 0; kk < BK / 16 - 1; kk++) {
            // the rest of the loads of step s+1 (their stage was released in the previous step)
            const int lo = LD_T + (kk > 0 ? LD_0 : 0) + (kk > 1 ? LD_1 : 0);
            const int n = kk == 0 ? LD_0 : (kk == 1 ? LD_1 : LD_2);
            issue_part(s + 1, nxt, lo, lo + n);
            // REGLOAD: B of step s+2 into the register set that held B of step s (written to LDS a step ago);
            // issued after the A loads of step s+1 (below, behind the barrier of the previous step), so that
            // the wait for those leaves these in flight
            if (REGLOAD && kk == 0) fetch_b(s + 2, par);
            read_group(cur, kk + 1, (kk + 1) & 1);
            mfma_group(kk & 1);
            if (REGLOAD) { if (kk == 0) interleave_loads(B_LOADS); else interleave(); }
            else if (n > 0) interleave_loads(n); else interleave();
        }
        if (!REGLOAD) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's loads of step s+1 landed
        commit_a(s + 1, nxt);                // (REGLOAD: the compiler's own waits: all loads but the B_LOADS youngest)
        commit_b(s + 1, nxt, par ^ 1);
        zero_tail(s + 1, nxt);
        __syncthreads();                     // everyone's did, and nobody reads `cur` any more
        issue_part(s + 2, cur, 0, LD_T);
        fetch_a(s + 2);
        read_group(nxt, 0, 0);
        mfma_group((BK / 16 - 1) & 1);
        if (REGLOAD) interleave_loads(A_LOADS); else if (LD_T > 0) interleave_loads(LD_T); else interleave();
    };
    // ---- persistent block: walks its share of the logical tiles --------------------------------
    // Hardware places block b on XCD b % 8.  XCD x owns the contiguous run [x*per, (x+1)*per) of
    // tiles and its blocks take them round-robin, so the tiles in flight on an XCD at any moment
    // are neighbours and share operand slices in that XCD's L2; the total % 8 tiles left over go
    // one each to the blocks of the least loaded slot.
    // fwd/dgrad: the launch is sized for an upper bound on the row tiles; the tiles that exist are
    // counted here from cum_token_counts, so that all XCDs get equal shares of real work.
    int total_tiles = p.total_tiles;
    if (EPI != EPI_WGRAD) {
        if (wave == 0) build_tile_table<BM>(p.cum, p.n_experts, lane, tile_end, seg);
        __syncthreads();
        constexpr int BN_OUT = (EPI == EPI_SWIGLU) ? BN / 2 : BN;
        total_tiles = __builtin_amdgcn_readfirstlane(tile_end[p.n_experts - 1]) * ((p.n_cols + BN_OUT - 1) / BN_OUT);
    }
    const int nbx = gridDim.x / NUM_XCD;
    const int xcd = blockIdx.x % NUM_XCD, slot = blockIdx.x / NUM_XCD;
    int per = total_tiles / NUM_XCD, rem = total_tiles - per * NUM_XCD;
    int run_lo = xcd * per;   // first tile of this XCD's run
    if (EPI == EPI_WGRAD && p.n_experts <= WGRAD_BALANCE_MAX_EXPERTS) {
        int lo, hi;
        wgrad_xcd_run(p.cum, p.n_experts, p.tiles_e, BK, xcd, NUM_XCD, lane, lo, hi);
        run_lo = __builtin_amdgcn_readfirstlane(lo);
        per = __builtin_amdgcn_readfirstlane(hi) - run_lo;
        rem = 0;
    }
    const int n_mine = slot < per ? (per - slot + nbx - 1) / nbx : 0;
    const int n_all = n_mine + ((xcd < rem && slot == per % nbx) ? 1 : 0);
    int it = 0;
    // moves the per-tile state to this block's next tile that has rows; false when there is none
    auto next_tile = [&]() -> bool {
        while (it < n_all) {
            const int logical = it < n_mine ? run_lo + slot + it * nbx : total_tiles - rem + xcd;
            it++;
            if (setup_tile(logical)) return true;
        }
        return false;
    };
    bool have = next_tile();
    bool prefetched = false;   // the loads of step 0 of the current tile are already in flight
    while (have) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    // Steps are taken in pairs so the stage names are static; an odd step count ends with a single
    // step.
    if (loop_steps > 0) {
        if (!prefetched) { issue_loads(0, stage0); fetch_a(0); fetch_b(0, 0); fetch_b(1, 1); }
        if (!REGLOAD) __builtin_amdgcn_s_waitcnt(0x0F70);
        commit_a(0, stage0);
        commit_b(0, stage0, 0);
        zero_tail(0, stage0);
        __syncthreads();
        issue_part(1, stage1, 0, LD_T);
        fetch_a(1);
        read_group(stage0, 0, 0);
        const int n_steps = loop_steps;
        for (int step = 0; step < n_steps; step += 2) {
            half_step(stage0, stage1, step, 0);
            if (!ANY_STEPS || step + 1 < n_steps) half_step(stage1, stage0, step + 1, 1);
        }
    }
    __syncthreads();  // the stages are dead: stage 1 becomes the strips, stage 0 the next tile's

    // The next tile's first contraction step is fetched into stage 0 while this tile's results go
    // out (the strips live in stage 1), which takes the cold-miss latency of a tile's first loads
    // off the critical path.
    const int e_expert = expert, e_row_begin = row_begin, e_row_end = row_end, e_n0 = n0;
    have = next_tile();
    prefetched = have && loop_steps > 0;
    if (prefetched) { issue_loads(0, stage0); fetch_a(0); fetch_b(0, 0); fetch_b(1, 1); }

    // ---- epilogue ------------------------------------------------------------------------------
    // Accumulator element r of lane l is output row (l % 32), column (r/4)*8 + (l/32)*4 + (r%4) of
    // its 32x32 block: a lane holds 4 consecutive columns of ONE row, and the 64 lanes of a store
    // would touch 32 different rows.  Each wavefront therefore turns its results around through a
    // private LDS strip (32 rows x COLS bf16, row pitch COLS*2+8 bytes so that both the 8-byte
    // writes in accumulator layout and the 8-byte reads in row layout are conflict-free) and moves
    // 16 bytes per lane to and from global memory, 64 lanes covering whole 256-byte row segments.
    // The fused SwiGLU backward reads g and u in the same row layout.
    // The epilogue's lane-derived addresses are the same for every tile; recompute them per tile
    // (a few VALU ops) instead of letting them be hoisted out of the tile loop, where they would
    // stay live across the main loop and spill.
    int lane_e = lane, wave_e = __builtin_amdgcn_readfirstlane(wave);
    asm volatile("" : "+v"(lane_e), "+s"(wave_e));
    constexpr int COLS = (EPI == EPI_SWIGLU) ? WN / 2 : WN;   // output columns of this wavefront
    constexpr int PITCH = COLS * 2 + 8;
    constexpr int STRIP = 32 * PITCH;
    constexpr int NSTRIP = (EPI == EPI_SWIGLU) ? 3 : 1;
    static_assert(NW * NSTRIP * STRIP <= A_BYTES + B_BYTES, "strips must fit in one stage");
    const int wm_e = wave_e / WAVES_N, wn_e = wave_e % WAVES_N;
    char *strip = stage1 + wave_e * (NSTRIP * STRIP);
    const int lrow = lane_e & 31;
    const int lcol = (lane_e >> 5) * 4;
    constexpr int CPRW = COLS / 8;            // 16-byte chunks per strip row
    constexpr int ITS = 32 * CPRW / 64;       // chunks per lane per strip
    // write 4 consecutive columns (as bf16) of row lrow at column `col` of strip `which`
    auto strip_put = [&](int which, int col, float v0, float v1, float v2, float v3) {
        u32x2 v;
        v[0] = pack2_bf16(v0, v1);
        v[1] = pack2_bf16(v2, v3);
        *reinterpret_cast<u32x2 *>(strip + which * STRIP + lrow * PITCH + col * 2) = v;
    };
    auto strip_get = [&](int which, int row, int cc) -> u32x4 {
        const char *q = strip + which * STRIP + row * PITCH + cc * 16;
        const u32x2 lo = *reinterpret_cast<const u32x2 *>(q);
        const u32x2 hi = *reinterpret_cast<const u32x2 *>(q + 8);
        return u32x4{lo[0], lo[1], hi[0], hi[1]};
    };
    auto strip_sync = [&]() {  // LDS operations of one wavefront are performed in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    const int col0 = (EPI == EPI_SWIGLU) ? e_n0 + (wn_e * WN) / 2 : e_n0 + wn_e * WN;   // first output column
    uint16_t *Cb = p.C + (EPI == EPI_WGRAD ? e_expert * p.strideC : 0);
    // Rows this wavefront may touch in global memory: the expert's rows (the weight gradient: the
    // rows of dW), none at all for a lane whose 8 columns lie past the last output column (a partial
    // last column tile; extents are multiples of 8, so a lane's 16-byte chunk is in or out as a whole).
    const int row_lim = !EDGE ? (EPI == EPI_WGRAD ? 0x7fffffff : e_row_end)
                              : (col0 + (lane_e % (COLS / 8)) * 8 < p.n_cols) ? (EPI == EPI_WGRAD ? p.kc : e_row_end) : 0;
    // ROWW forward: the weights of this lane's row in every strip, fetched together up front
    float wrow_all[(ROWW && EPI == EPI_SWIGLU) ? TM : 1];
    if (ROWW && EPI == EPI_SWIGLU) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int64_t m = static_cast<int64_t>(e_row_begin) + wm_e * WM + i * 32 + lrow;
            wrow_all[(ROWW && EPI == EPI_SWIGLU) ? i : 0] = (m < e_row_end) ? p.row_scale[m] : 0.0f;
        }
    }
    // Weight gradient added to what the output already holds (a gradient buffer that several
    // backward passes accumulate into): the old values of a strip are fetched one strip ahead (two
    // register sets), and the sum is what an in-place bf16 `grad += dW` gives, two roundings.
    constexpr bool acc_out = ACCUM;
    u32x4 old2[ACCUM ? 2 : 1][ACCUM ? ITS : 1];
    auto load_old = [&](int i, int buf) {
        const int64_t m0 = static_cast<int64_t>(e_row_begin) + wm_e * WM + i * 32;
#pragma unroll
        for (int it = 0; it < ITS; it++) {
            const int q = it * 64 + lane_e;
            const int64_t o = (m0 + q / CPRW) * p.ldc + col0 + (q % CPRW) * 8;
            if (m0 + q / CPRW < row_lim)
                old2[ACCUM ? buf : 0][ACCUM ? it : 0] = *reinterpret_cast<const u32x4 *>(Cb + o);
        }
    };
    if (ACCUM) load_old(0, 0);
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int64_t m0 = static_cast<int64_t>(e_row_begin) + wm_e * WM + i * 32;  // first row of the strip
        if (ACCUM && i + 1 < TM) load_old(i + 1, (i + 1) & 1);
        u32x4 *old_out = old2[ACCUM ? (i & 1) : 0];
        if (EPI == EPI_SWIGLU) {
            const float wrow = wrow_all[(ROWW && EPI == EPI_SWIGLU) ? i : 0];   // ROWW: h = w[row] * silu(g) * u, one rounding
#pragma unroll
            for (int j = 0; j < TN; j += 2)
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    float hv[4];
#pragma unroll
                    for (int x = 0; x < 4; x++) {
                        const float gv = acc[i][j][rq * 4 + x], uv = acc[i][j + 1][rq * 4 + x];
                        hv[x] = (gv * fast_sigmoid(gv)) * uv;
                        if (ROWW) hv[x] *= wrow;
                    }
                    const int col = (j / 2) * 32 + rq * 8 + lcol;
                    strip_put(0, col, acc[i][j][rq * 4], acc[i][j][rq * 4 + 1], acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3]);
                    strip_put(1, col, acc[i][j + 1][rq * 4], acc[i][j + 1][rq * 4 + 1], acc[i][j + 1][rq * 4 + 2], acc[i][j + 1][rq * 4 + 3]);
                    strip_put(2, col, hv[0], hv[1], hv[2], hv[3]);
                }
        } else {
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int rq = 0; rq < 4; rq++)
                    strip_put(0, j * 32 + rq * 8 + lcol, acc[i][j][rq * 4], acc[i][j][rq * 4 + 1],
                              acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3]);
        }
        strip_sync();
        if (EPI == EPI_SWIGLU_BWD) {
            u32x4 gq[ITS], uq[ITS];
            // ROWW: lane l fetches the weight of strip row l % 32 along with the g/u loads; the
            // lanes that work on a row pick it up with a lane read
            float w_strip = 0.0f;
            if (ROWW && m0 + (lane_e & 31) < e_row_end) w_strip = p.row_scale[m0 + (lane_e & 31)];
#pragma unroll
            for (int it = 0; it < ITS; it++) {
                const int q = it * 64 + lane_e;
                const int64_t m = m0 + q / CPRW;
                if (m < row_lim) {
                    const int64_t o = m * p.ldc + col0 + (q % CPRW) * 8;
                    // g and u have no reader after this one: keep them out of the caches (-1 to -3 %)
                    gq[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.G + o));
                    uq[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.U + o));
                }
            }
#pragma unroll
            for (int it = 0; it < ITS; it++) {
                const int q = it * 64 + lane_e;
                const int64_t m = m0 + q / CPRW;
                float dot = 0.0f;   // ROWW: this lane's part of sum_i dh[m][i] * silu(g[m][i]) * u[m][i]
                const float wr = ROWW ? __shfl(w_strip, q / CPRW, 64) : 1.0f;
                if (m < row_lim) {
                    float dh[8], gv[8], uv[8], dg[8], du[8];
                    Elem<uint16_t>::unpack(strip_get(0, q / CPRW, q % CPRW), dh);
                    Elem<uint16_t>::unpack(gq[it], gv);
                    Elem<uint16_t>::unpack(uq[it], uv);
#pragma unroll
                    for (int x = 0; x < 8; x++) {
                        const float sg = fast_sigmoid(gv[x]);
                        const float sl = gv[x] * sg;
                        if (ROWW) {
                            // acc is the gradient of w * silu(g) * u: the routing weight's gradient
                            // is its product with silu(g) * u, the activation's gets the factor w
                            dot += dh[x] * (sl * uv[x]);
                            dh[x] *= wr;
                        }
                        du[x] = dh[x] * sl;
                        dg[x] = (dh[x] * uv[x]) * (sg * (1.0f + gv[x] * (1.0f - sg)));
                    }
                    const int64_t o = m * p.ldc + col0 + (q % CPRW) * 8;
                    u32x4 vg, vu;
#pragma unroll
                    for (int x = 0; x < 4; x++) {
                        vg[x] = pack2_bf16(dg[2 * x], dg[2 * x + 1]);
                        vu[x] = pack2_bf16(du[2 * x], du[2 * x + 1]);
                    }
                    *reinterpret_cast<u32x4 *>(p.C + o) = vg;
                    *reinterpret_cast<u32x4 *>(p.C1 + o) = vu;
                }
                if (ROWW) {
                    // the CPRW lanes of a row are neighbours: add them up in a fixed order and let
                    // the first one store the sum for this wavefront's column range
                    dot = lane_group_sum<CPRW>(dot);
                    if (q % CPRW == 0 && m < row_lim) p.row_dot[(col0 / COLS) * p.rows + m] = dot;
                }
            }
        } else {
#pragma unroll
            for (int it = 0; it < ITS; it++) {
                const int q = it * 64 + lane_e;
                const int64_t m = m0 + q / CPRW;
                if (m < row_lim) {
                    const int64_t o = m * p.ldc + col0 + (q % CPRW) * 8;
                    u32x4 v = strip_get(0, q / CPRW, q % CPRW);
                    if (EPI == EPI_WGRAD && acc_out) {
                        float fresh[8], old[8];
                        Elem<uint16_t>::unpack(v, fresh);
                        Elem<uint16_t>::unpack(old_out[ACCUM ? it : 0], old);
#pragma unroll
                        for (int x = 0; x < 4; x++)
                            v[x] = pack2_bf16(old[2 * x] + fresh[2 * x], old[2 * x + 1] + fresh[2 * x + 1]);
                    }
                    *reinterpret_cast<u32x4 *>(Cb + o) = v;
                    if (EPI == EPI_SWIGLU) {
                        *reinterpret_cast<u32x4 *>(p.C1 + o) = strip_get(1, q / CPRW, q % CPRW);
                        *reinterpret_cast<u32x4 *>(p.C2 + o) = strip_get(2, q / CPRW, q % CPRW);
                    }
                }
            }
        }
        strip_sync();  // the strip is rewritten by the next i
    }
    __syncthreads();  // the strips alias stage 1, which the next tile loads into
    }  // tile loop
}

// ---- host side ---------------------------------------------------------------------------------

// Two tile shapes: 256x256 (8 wavefronts of 128x64) for the training shapes, 128x128 (4 wavefronts
// of 64x64) when an extent is not a multiple of 256 or experts hold few rows each.

inline bool mult(int64_t v, int m) { return v > 0 && v % m == 0; }
// Operands are addressed as a 64-bit block-uniform base plus a 32-bit lane offset, so their size is
// only bounded by int64 arithmetic on element counts (2^40 here, far beyond device memory); a source
// whose rows are fetched through an index has index * pitch in the lane offset and must span
// < 2^31 elements.  Per-expert pitches are multiples of 8 elements (16-byte vectors need that).
inline bool fits_span(int64_t elems) { return elems >= 0 && elems < (1LL << 40); }
inline bool fits_gather(int64_t elems) { return elems >= 0 && elems < (1LL << 31); }
inline bool pitch_ok(int64_t stride) { return stride >= 0 && stride % 8 == 0; }

// Blocks of a launch: one resident set (a multiple of the 8 XCDs), or fewer when there are few
// tiles.  The 256x256 tile's 128 KB of LDS leave room for one block per CU, the 128x128 tile's
// 64 KB for two.
// Compute units of the current device (256 on an MI355X in its default partition mode), asked from
// the runtime once per device.
inline int device_cu_count() {
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < NUM_XCD)
            n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}
template <int BM> unsigned persistent_blocks(int64_t tiles) {
    const int64_t per_xcd_max = (device_cu_count() / NUM_XCD) * (BM == 256 ? 1 : 2);
    int64_t per_xcd = (tiles + NUM_XCD - 1) / NUM_XCD;
    if (per_xcd > per_xcd_max) per_xcd = per_xcd_max;
    if (per_xcd < 1) per_xcd = 1;
    return static_cast<unsigned>(per_xcd * NUM_XCD);
}

template <int BM> struct Waves {
    static constexpr int M = 2;                       // 256x256: 2 x 4 wavefronts of 128x64;
    static constexpr int N = (BM == 256) ? 4 : 2;    // 128x128: 2 x 2 wavefronts of 64x64
};

template <int BM, int BN, int AKIND, int BKIND, int EPI, int GATHER = GATHER_NONE, bool ROWW = false, bool KTAIL = false,
          bool REGLOAD = false>
int launch_rows(GemmParams &p, int64_t rows, hipStream_t st) {  // fwd / dgrad family
    constexpr int BN_OUT = (EPI == EPI_SWIGLU) ? BN / 2 : BN;
    if (p.n_experts > MAX_EXPERTS) return OM_ERR_SHAPE;   // the tile table lives in LDS
    p.m_tiles_max = static_cast<int>((rows + BM - 1) / BM + p.n_experts);
    const int64_t tiles = static_cast<int64_t>(p.m_tiles_max) * ((p.n_cols + BN_OUT - 1) / BN_OUT);
    if (tiles > 0x7fffffffLL) return OM_ERR_SHAPE;
    p.total_tiles = static_cast<int>(tiles);
    ggemm_kernel<BM, BN, Waves<BM>::M, Waves<BM>::N, AKIND, BKIND, EPI, GATHER, ROWW, false, KTAIL, REGLOAD>
        <<<dim3(persistent_blocks<BM>(tiles)), dim3(Waves<BM>::M * Waves<BM>::N * 64), 0, st>>>(p);
    return om_launch_status();
}

// The tile shape launch_rows_auto picks: 256x256 when the output columns are a whole number of such
// tiles, the contraction a whole number of step pairs, the experts hold enough rows to fill them, and there are enough of them for at least half
// the CUs (a tiny problem is spread over more CUs by the 128x128 tile).  The 128x128 tile takes any
// extents and contraction lengths that are multiples of 8: its last column tile and its last
// contraction step may be partial.
template <int EPI> bool uses_big_tile(int n_cols, int kc, int n_experts, int64_t rows) {
    constexpr int div = (EPI == EPI_SWIGLU) ? 2 : 1;
    if (n_cols % (256 / div) != 0 || kc % 128 != 0 || rows < static_cast<int64_t>(n_experts) * 192) return false;
    const int64_t tiles = ((rows + 255) / 256) * (n_cols / (256 / div));
    return tiles * 2 >= device_cu_count();
}

template <int AKIND, int BKIND, int EPI, int GATHER = GATHER_NONE, bool ROWW = false>
int launch_rows_auto(GemmParams &p, int64_t rows, hipStream_t st) {
    if (uses_big_tile<EPI>(p.n_cols, p.kc, p.n_experts, rows))
        return launch_rows<256, 256, AKIND, BKIND, EPI, GATHER, ROWW>(p, rows, st);
    if (p.n_cols % 8 != 0 || p.kc % 8 != 0) return OM_ERR_SHAPE;
    if (p.kc % 64 != 0) return launch_rows<128, 128, AKIND, BKIND, EPI, GATHER, ROWW, true>(p, rows, st);
    // Few rows per expert (fewer than 256 on average): the launch streams weights that are used once, and the
    // kernels that keep two steps of them in flight are 4-10 % faster; with more rows the direct-load kernels
    // are (4-9 % at 2000 rows per expert), so each regime gets its own.
    if (rows < static_cast<int64_t>(p.n_experts) * 256)
        return launch_rows<128, 128, AKIND, BKIND, EPI, GATHER, ROWW, false, true>(p, rows, st);
    return launch_rows<128, 128, AKIND, BKIND, EPI, GATHER, ROWW>(p, rows, st);
}

}  // namespace

extern "C" int om_grouped_gemm_fwd(const void *input, const void *weight, void *output,
                                   const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                   int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(N, 8) || !mult(K, 8)) return OM_ERR_SHAPE;
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
    if (!pitch_ok(p.strideB)) return OM_ERR_ALIGN;
    if (!fits_span(rows * K) || !fits_span(rows * N) || !fits_span(p.strideB * G)) return OM_ERR_SHAPE;
    p.rows = rows; p.n_experts = G; p.n_cols = N; p.kc = K; p.phases = 1;
    return launch_rows_auto<CONTIG, CONTIG, EPI_STORE>(p, rows, om_stream(stream));
}

extern "C" int om_grouped_gemm_dgrad(const void *output_grad, const void *weight, void *input_grad,
                                     const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                     int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(N, 8) || !mult(K, 8)) return OM_ERR_SHAPE;
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
    if (!pitch_ok(p.strideB)) return OM_ERR_ALIGN;
    if (!fits_span(rows * K) || !fits_span(rows * N) || !fits_span(p.strideB * G)) return OM_ERR_SHAPE;
    p.rows = rows; p.n_experts = G; p.n_cols = K; p.kc = N; p.phases = 1;
    return launch_rows_auto<CONTIG, STRIDED, EPI_STORE>(p, rows, om_stream(stream));
}

namespace {
// weight gradient; gather == GATHER_B: contraction row c of `input` is row index[c] of a
// [src_rows, K] matrix; gather == GATHER_WA: contraction row c of `output_grad` is row index[c] of a
// [src_rows, N] matrix (the token gather folded into the loads)
int wgrad_launch(const void *output_grad, const void *input, const int32_t *index, int gather,
                 int64_t src_rows, void *weight_grad, const int32_t *cum_token_counts, int64_t rows, int G,
                 int N, int K, int64_t w_stride, void *stream, bool accumulate = false) {
    if (rows < 0 || G < 1 || !mult(N, 8) || !mult(K, 8)) return OM_ERR_SHAPE;
    // rows == 0 (nothing routed to these experts): the activations may be empty tensors without
    // storage; the launch then only writes zeros
    if (!weight_grad || !cum_token_counts || (rows > 0 && (!output_grad || !input))) return OM_ERR_NULL;
    if (!om_aligned16(output_grad) || !om_aligned16(input) || !om_aligned16(weight_grad)) return OM_ERR_ALIGN;
    GemmParams p = {};
    p.A[0] = static_cast<const uint16_t *>(output_grad);  // [rows, N]: operand rows = n, c = row
    p.B[0] = static_cast<const uint16_t *>(input);        // [rows, K] (or [src_rows, K] through input_rows)
    p.C = static_cast<uint16_t *>(weight_grad);           // [G, N, K]
    p.cum = cum_token_counts;
    p.row_index = index;
    p.lda = N; p.ldb = K; p.ldc = K;
    p.strideC = w_stride ? w_stride : static_cast<int64_t>(N) * K;
    if (!pitch_ok(p.strideC)) return OM_ERR_ALIGN;
    if (!fits_span(rows * K) || !fits_span(rows * N) || !fits_span(p.strideC * G) ||
        !fits_gather(src_rows * (gather == GATHER_WA ? N : K)))
        return OM_ERR_SHAPE;
    p.rows = rows; p.n_experts = G; p.n_cols = K; p.kc = N; p.phases = 1;
    hipStream_t st = om_stream(stream);
    // 256x256 tiles unless they are too few to occupy half the CUs
    const bool big = N % 256 == 0 && K % 256 == 0 &&
                     static_cast<int64_t>(G) * (N / 256) * (K / 256) * 2 >= device_cu_count();
    p.tiles_e = big ? (N / 256) * (K / 256) : ((N + 127) / 128) * ((K + 127) / 128);
    const int64_t tiles = static_cast<int64_t>(p.tiles_e) * G;
    if (tiles > 0x7fffffffLL) return OM_ERR_SHAPE;
    p.total_tiles = static_cast<int>(tiles);
    const dim3 grid_big(persistent_blocks<256>(tiles)), block_big(Waves<256>::M * Waves<256>::N * 64);
    const dim3 grid_small(persistent_blocks<128>(tiles)), block_small(256);
    // ACCUM (C[g] = bf16(float(C[g]) + float(bf16(acc))) instead of C[g] = acc) is a template
    // parameter: the plain kernels carry none of it
#define OM_WGRAD(GATHER_KIND, ACC)                                                                               \
    do {                                                                                                         \
        if (big)                                                                                                 \
            ggemm_kernel<256, 256, Waves<256>::M, Waves<256>::N, STRIDED, STRIDED, EPI_WGRAD, GATHER_KIND, false, \
                         ACC><<<grid_big, block_big, 0, st>>>(p);                                                \
        else                                                                                                     \
            ggemm_kernel<128, 128, 2, 2, STRIDED, STRIDED, EPI_WGRAD, GATHER_KIND, false, ACC>                    \
                <<<grid_small, block_small, 0, st>>>(p);                                                         \
    } while (0)
    if (accumulate) {
        if (gather == GATHER_NONE) OM_WGRAD(GATHER_NONE, true);
        else if (gather == GATHER_B) OM_WGRAD(GATHER_B, true);
        else OM_WGRAD(GATHER_WA, true);
    } else {
        if (gather == GATHER_NONE) OM_WGRAD(GATHER_NONE, false);
        else if (gather == GATHER_B) OM_WGRAD(GATHER_B, false);
        else OM_WGRAD(GATHER_WA, false);
    }
#undef OM_WGRAD
    return om_launch_status();
}
}  // namespace

extern "C" int om_grouped_gemm_wgrad(const void *output_grad, const void *input, void *weight_grad,
                                     const int32_t *cum_token_counts, int64_t rows, int G, int N, int K,
                                     int64_t w_stride, void *stream) {
    return wgrad_launch(output_grad, input, nullptr, GATHER_NONE, 0, weight_grad, cum_token_counts, rows, G,
                        N, K, w_stride, stream);
}

extern "C" int om_grouped_gemm_wgrad_gathered(const void *output_grad, const void *input,
                                              const int32_t *input_rows, int64_t src_rows,
                                              void *weight_grad, const int32_t *cum_token_counts,
                                              int64_t rows, int G, int N, int K, int64_t w_stride,
                                              void *stream) {
    if (!input_rows) return OM_ERR_NULL;
    if (src_rows < 1) return OM_ERR_SHAPE;
    return wgrad_launch(output_grad, input, input_rows, GATHER_B, src_rows, weight_grad, cum_token_counts,
                        rows, G, N, K, w_stride, stream);
}

extern "C" int om_grouped_gemm_wgrad_gathered_out(const void *output_grad, const int32_t *output_grad_rows,
                                                  int64_t src_rows, const void *input, void *weight_grad,
                                                  const int32_t *cum_token_counts, int64_t rows, int G,
                                                  int N, int K, int64_t w_stride, void *stream) {
    if (!output_grad_rows) return OM_ERR_NULL;
    if (src_rows < 1) return OM_ERR_SHAPE;
    return wgrad_launch(output_grad, input, output_grad_rows, GATHER_WA, src_rows, weight_grad,
                        cum_token_counts, rows, G, N, K, w_stride, stream);
}

// The accumulating forms: weight_grad += dW in the gradient's dtype, inside the epilogue.
extern "C" int om_grouped_gemm_wgrad_accumulate(const void *output_grad, const void *input, void *weight_grad,
                                                const int32_t *cum_token_counts, int64_t rows, int G, int N,
                                                int K, int64_t w_stride, void *stream) {
    return wgrad_launch(output_grad, input, nullptr, GATHER_NONE, 0, weight_grad, cum_token_counts, rows, G,
                        N, K, w_stride, stream, true);
}

extern "C" int om_grouped_gemm_wgrad_gathered_accumulate(const void *output_grad, const void *input,
                                                         const int32_t *input_rows, int64_t src_rows,
                                                         void *weight_grad, const int32_t *cum_token_counts,
                                                         int64_t rows, int G, int N, int K, int64_t w_stride,
                                                         void *stream) {
    if (!input_rows) return OM_ERR_NULL;
    if (src_rows < 1) return OM_ERR_SHAPE;
    return wgrad_launch(output_grad, input, input_rows, GATHER_B, src_rows, weight_grad, cum_token_counts,
                        rows, G, N, K, w_stride, stream, true);
}

extern "C" int om_grouped_gemm_wgrad_gathered_out_accumulate(const void *output_grad,
                                                             const int32_t *output_grad_rows, int64_t src_rows,
                                                             const void *input, void *weight_grad,
                                                             const int32_t *cum_token_counts, int64_t rows,
                                                             int G, int N, int K, int64_t w_stride,
                                                             void *stream) {
    if (!output_grad_rows) return OM_ERR_NULL;
    if (src_rows < 1) return OM_ERR_SHAPE;
    return wgrad_launch(output_grad, input, output_grad_rows, GATHER_WA, src_rows, weight_grad,
                        cum_token_counts, rows, G, N, K, w_stride, stream, true);
}

namespace {
// `x_rows` != null: sorted row r of the activations is row x_rows[r] of x [src_rows, H]
// `row_weights` != null (needs x_rows): h = row_weights[r] * silu(g) * u
int gate_up_fwd_launch(const void *x, const int32_t *x_rows, int64_t src_rows, const void *w_gate,
                       const void *w_up, const float *row_weights, void *g, void *u, void *h,
                       const int32_t *cum_token_counts, int64_t rows, int G, int I, int H,
                       int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(I, 8) || !mult(H, 8)) return OM_ERR_SHAPE;
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
    p.row_index = x_rows;
    p.row_scale = row_weights;
    p.lda = H; p.ldb = H; p.ldc = I;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(I) * H;
    if (!pitch_ok(p.strideB)) return OM_ERR_ALIGN;
    if (!fits_span(rows * H) || !fits_span(rows * I) || !fits_span(p.strideB * G) || !fits_gather(src_rows * H))
        return OM_ERR_SHAPE;
    p.rows = rows; p.n_experts = G; p.n_cols = I; p.kc = H; p.phases = 1;
    if (row_weights) return launch_rows_auto<CONTIG, CONTIG, EPI_SWIGLU, GATHER_A, true>(p, rows, om_stream(stream));
    if (x_rows) return launch_rows_auto<CONTIG, CONTIG, EPI_SWIGLU, GATHER_A>(p, rows, om_stream(stream));
    return launch_rows_auto<CONTIG, CONTIG, EPI_SWIGLU>(p, rows, om_stream(stream));
}
}  // namespace

extern "C" int om_merged_mlp_gate_up_fwd(const void *x, const void *w_gate, const void *w_up, void *g,
                                         void *u, void *h, const int32_t *cum_token_counts,
                                         int64_t rows, int G, int I, int H, int64_t w_stride,
                                         void *stream) {
    return gate_up_fwd_launch(x, nullptr, 0, w_gate, w_up, nullptr, g, u, h, cum_token_counts, rows, G, I,
                              H, w_stride, stream);
}

extern "C" int om_merged_mlp_gate_up_fwd_gathered(const void *x, const int32_t *x_rows, int64_t src_rows,
                                                  const void *w_gate, const void *w_up, void *g, void *u,
                                                  void *h, const int32_t *cum_token_counts,
                                                  int64_t rows, int G, int I, int H, int64_t w_stride,
                                                  void *stream) {
    if (rows > 0 && !x_rows) return OM_ERR_NULL;
    if (src_rows < 1 && rows > 0) return OM_ERR_SHAPE;
    return gate_up_fwd_launch(x, x_rows, src_rows, w_gate, w_up, nullptr, g, u, h, cum_token_counts, rows,
                              G, I, H, w_stride, stream);
}

extern "C" int om_merged_mlp_gate_up_fwd_weighted(const void *x, const int32_t *x_rows, int64_t src_rows,
                                                  const void *w_gate, const void *w_up,
                                                  const float *row_weights, void *g, void *u, void *h,
                                                  const int32_t *cum_token_counts, int64_t rows, int G,
                                                  int I, int H, int64_t w_stride, void *stream) {
    if (rows > 0 && (!x_rows || !row_weights)) return OM_ERR_NULL;
    if (src_rows < 1 && rows > 0) return OM_ERR_SHAPE;
    return gate_up_fwd_launch(x, x_rows, src_rows, w_gate, w_up, row_weights, g, u, h, cum_token_counts,
                              rows, G, I, H, w_stride, stream);
}

namespace {
// columns of the intermediate size that one wavefront's epilogue covers (both tile shapes): the
// granularity of the row_dot partial sums
constexpr int ROW_DOT_COLS = 64;
static_assert(256 / Waves<256>::N == ROW_DOT_COLS && 128 / Waves<128>::N == ROW_DOT_COLS, "row_dot layout");

// `dy_rows` != null: sorted row r of dy is row dy_rows[r] of a [src_rows, H] matrix, the result is
// scaled by row_weights[r] and row_dot receives the partial sums of (dy W) * silu(g) * u
int down_dgrad_launch(const void *dy, const int32_t *dy_rows, int64_t src_rows, const void *w_down,
                      const void *g, const void *u, const float *row_weights, void *dg, void *du,
                      float *row_dot, const int32_t *cum_token_counts, int64_t rows, int G, int I, int H,
                      int64_t w_stride, void *stream) {
    if (rows < 0 || G < 1 || !mult(I, 8) || !mult(H, 8)) return OM_ERR_SHAPE;
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
    p.row_index = dy_rows;
    p.row_scale = row_weights;
    p.row_dot = row_dot;
    p.lda = H; p.ldb = I; p.ldc = I;
    p.strideB = w_stride ? w_stride : static_cast<int64_t>(H) * I;
    if (!pitch_ok(p.strideB)) return OM_ERR_ALIGN;
    if (!fits_span(rows * H) || !fits_span(rows * I) || !fits_span(p.strideB * G) || !fits_gather(src_rows * H))
        return OM_ERR_SHAPE;
    p.rows = rows; p.n_experts = G; p.n_cols = I; p.kc = H; p.phases = 1;
    if (dy_rows) return launch_rows_auto<CONTIG, STRIDED, EPI_SWIGLU_BWD, GATHER_A, true>(p, rows, om_stream(stream));
    return launch_rows_auto<CONTIG, STRIDED, EPI_SWIGLU_BWD>(p, rows, om_stream(stream));
}
}  // namespace

extern "C" int om_merged_mlp_down_dgrad(const void *dy, const void *w_down, const void *g, const void *u,
                                        void *dg, void *du, const int32_t *cum_token_counts,
                                        int64_t rows, int G, int I, int H, int64_t w_stride,
                                        void *stream) {
    return down_dgrad_launch(dy, nullptr, 0, w_down, g, u, nullptr, dg, du, nullptr, cum_token_counts, rows,
                             G, I, H, w_stride, stream);
}

extern "C" int om_merged_mlp_row_dot_parts(int I) {
    if (I < 8 || I % 8 != 0) return OM_ERR_SHAPE;
    return (I + ROW_DOT_COLS - 1) / ROW_DOT_COLS;
}

extern "C" int om_merged_mlp_down_dgrad_weighted(const void *dy, const int32_t *dy_rows, int64_t src_rows,
                                                 const void *w_down, const void *g, const void *u,
                                                 const float *row_weights, void *dg, void *du,
                                                 float *row_dot, const int32_t *cum_token_counts,
                                                 int64_t rows, int G, int I, int H, int64_t w_stride,
                                                 void *stream) {
    if (rows > 0 && (!dy_rows || !row_weights || !row_dot)) return OM_ERR_NULL;
    if (src_rows < 1 && rows > 0) return OM_ERR_SHAPE;
    return down_dgrad_launch(dy, dy_rows, src_rows, w_down, g, u, row_weights, dg, du, row_dot,
                             cum_token_counts, rows, G, I, H, w_stride, stream);
}

extern "C" int om_merged_mlp_gate_up_dgrad(const void *dg, const void *du, const void *w_gate,
                                           const void *w_up, void *dx, const int32_t *cum_token_counts,
                                           int64_t rows, int G, int I, int H, int64_t w_stride,
                                           void *stream) {
    if (rows < 0 || G < 1 || !mult(I, 8) || !mult(H, 8)) return OM_ERR_SHAPE;
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
    if (!pitch_ok(p.strideB)) return OM_ERR_ALIGN;
    if (!fits_span(rows * H) || !fits_span(rows * I) || !fits_span(p.strideB * G)) return OM_ERR_SHAPE;
    p.rows = rows; p.n_experts = G; p.n_cols = H; p.kc = I; p.phases = 2;
    return launch_rows_auto<CONTIG, STRIDED, EPI_STORE>(p, rows, om_stream(stream));
}
