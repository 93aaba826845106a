// Routers: one wavefront per token.
//  * softmax -> top-K (-> renormalise) of the OLMoE block, forward and backward;
//  * sigmoid -> bias-corrected group-limited top-K of the DeepSeek-V3 block, forward and backward.
// Selection order is total: (score descending, expert index ascending), so the result does not
// depend on lane scheduling.  Scores live in registers, expert i = lane + 64*j.
#include "common.h"

namespace {

#pragma clang fp contract(off)

constexpr int TOKENS_PER_BLOCK = 4;

template <typename T> __device__ __forceinline__ float load_logit(const T *p);
template <> __device__ __forceinline__ float load_logit<float>(const float *p) { return *p; }
template <> __device__ __forceinline__ float load_logit<uint16_t>(const uint16_t *p) { return bf16_bits_to_f32(*p); }

// (value, index) arg-max across the wavefront by an xor butterfly of lane permutes; ties go to
// the lower index.  Twelve dependent permutes: the slow path of wave_argmax below.
__device__ __forceinline__ void wave_argmax_butterfly(float &v, int &i) {
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, 64);
        const int oi = __shfl_xor(i, o, 64);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
}

// Maximum over the wavefront with data-parallel-primitive moves (no LDS traffic): within each row
// of 16 lanes by quad permutes and mirrors, then row 0 -> 1 and 2 -> 3, then rows 0-1 -> 2-3; lane
// 63 ends with the maximum and hands it to everyone through a scalar register.  A maximum does not
// depend on the order of the comparisons, so this is exact.
__device__ __forceinline__ float wave_max_dpp(float v) {
    int x = __float_as_int(v);
#define OM_DPP_MAX(ctrl, row_mask)                                                                   \
    x = __float_as_int(fmaxf(__int_as_float(x), __int_as_float(__builtin_amdgcn_update_dpp(         \
            x, x, ctrl, row_mask, 0xf, false))))
    OM_DPP_MAX(0xB1, 0xf);    // quad_perm [1,0,3,2]
    OM_DPP_MAX(0x4E, 0xf);    // quad_perm [2,3,0,1]
    OM_DPP_MAX(0x141, 0xf);   // row_half_mirror
    OM_DPP_MAX(0x140, 0xf);   // row_mirror: every lane of a row holds the row's maximum
    OM_DPP_MAX(0x142, 0xa);   // row_bcast15 into rows 1 and 3
    OM_DPP_MAX(0x143, 0xc);   // row_bcast31 into rows 2 and 3
#undef OM_DPP_MAX
    return __int_as_float(__builtin_amdgcn_readlane(x, 63));
}

// (value, index) arg-max across the wavefront; ties go to the lower index.  Fast path: the maximum
// by wave_max_dpp, a ballot of the lanes that hold it, and when exactly one lane does (no tie, no
// NaN) its index through a scalar lane read.  Everything else takes the butterfly, so the result
// is the butterfly's in every case.
__device__ __forceinline__ void wave_argmax(float &v, int &i) {
    const float m = wave_max_dpp(v);
    const unsigned long long vote = __ballot(v == m);
    if (__popcll(vote) == 1) {
        const int src = __ffsll(static_cast<long long>(vote)) - 1;
        i = __builtin_amdgcn_readlane(i, src);
        v = m;
    } else {
        wave_argmax_butterfly(v, i);
    }
}

// value of `x[e / 64]` held by lane e % 64, for a per-lane e (e < 0: undefined, caller masks)
template <int PER>
__device__ __forceinline__ float fetch_expert_value(const float (&x)[PER], int e) {
    float out = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const float v = __shfl(x[j], e & 63, 64);
        if ((e >> 6) == j) out = v;
    }
    return out;
}

// softmax probabilities of this token's row into p[PER]; returns nothing else.
template <int PER, typename T>
__device__ __forceinline__ void row_softmax(const T *row, int N, int lane, float (&p)[PER]) {
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        p[j] = (i < N) ? load_logit<T>(row + i) : -INFINITY;
        mx = fmaxf(mx, p[j]);
    }
    mx = wave_max_dpp(mx);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        p[j] = (i < N) ? expf(p[j] - mx) : 0.0f;
        sum += p[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < PER; j++) p[j] = p[j] / sum;
}

// K rounds of wave arg-max over s[PER] (entries with index >= N must be < every real score).
// Lane r keeps the r-th winner in (my_v, my_i).
template <int PER>
__device__ __forceinline__ void select_topk(float (&s)[PER], int N, int K, int lane, float &my_v,
                                            int &my_i) {
    my_v = 0.0f;
    my_i = 0;
    for (int r = 0; r < K; r++) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const int i = lane + 64 * j;
            if (i < N && (s[j] > bv)) { bv = s[j]; bi = i; }  // ascending i: first max wins
        }
        wave_argmax(bv, bi);
        if (lane == r) { my_v = bv; my_i = bi; }
#pragma unroll
        for (int j = 0; j < PER; j++)
            if (lane + 64 * j == bi) s[j] = -INFINITY;  // taken
    }
}

template <int PER, typename T, typename TW>
__global__ __launch_bounds__(256) void softmax_topk_kernel(const T *__restrict__ logits, int64_t Tn,
                                                           int N, int K, int renorm,
                                                           TW *__restrict__ weights_out,
                                                           int64_t *__restrict__ experts_out) {
    const int lane = threadIdx.x & 63;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * TOKENS_PER_BLOCK + (threadIdx.x >> 6);
    if (t >= Tn) return;
    float p[PER];
    row_softmax<PER, T>(logits + t * N, N, lane, p);
    float w; int e;
    select_topk<PER>(p, N, K, lane, w, e);
    if (renorm) {
        const float s = wave_sum(lane < K ? w : 0.0f);
        w = w / s;
    }
    if (lane < K) {
        Elem<TW>::store(weights_out + t * K + lane, w);
        experts_out[t * K + lane] = e;
    }
}

// dlogits_i = p_i * (dp_i - sum_j dp_j p_j), dp = scatter of dw over the selected experts, and
// with renormalisation dw_k = (dw'_k - sum_j dw'_j w_j / S) / S, S = sum_k w_k, w_k = p[e_k].
template <int PER, typename T, typename TW>
__global__ __launch_bounds__(256) void softmax_topk_bwd_kernel(const T *__restrict__ logits,
                                                               const int64_t *__restrict__ experts,
                                                               const TW *__restrict__ dweights,
                                                               int64_t Tn, int N, int K, int renorm,
                                                               T *__restrict__ dlogits) {
    const int lane = threadIdx.x & 63;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * TOKENS_PER_BLOCK + (threadIdx.x >> 6);
    if (t >= Tn) return;
    float p[PER];
    row_softmax<PER, T>(logits + t * N, N, lane, p);
    // lane k < K: its expert, the probability there and the incoming gradient
    const int e = (lane < K) ? static_cast<int>(experts[t * K + lane]) : -1;
    float dwk = (lane < K) ? Elem<TW>::load(dweights + t * K + lane) : 0.0f;
    float wk = fetch_expert_value<PER>(p, e);   // lane k < K: the probability of its expert
    if (lane >= K) wk = 0.0f;
    if (renorm) {
        const float S = wave_sum(wk);
        const float dot = wave_sum(dwk * wk);
        dwk = (dwk - dot / S) / S;
    }
    const float inner = wave_sum(dwk * wk);  // sum_j dp_j p_j
    float dp[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) dp[j] = 0.0f;
    for (int k = 0; k < K; k++) {
        const int ek = __shfl(e, k, 64);
        const float dk = __shfl(dwk, k, 64);
#pragma unroll
        for (int j = 0; j < PER; j++)
            if (lane + 64 * j == ek) dp[j] = dk;
    }
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        if (i < N) Elem<T>::store(dlogits + t * N + i, p[j] * (dp[j] - inner));
    }
}

// DeepSeek-V3 group-limited routing.  LDS holds the choice scores of the 4 tokens of the block
// so a lane can scan "its" group; everything else stays in registers.
template <int PER>
__global__ __launch_bounds__(256) void sigmoid_group_topk_kernel(
    const float *__restrict__ logits, const float *__restrict__ bias, int64_t Tn, int N, int n_group,
    int topk_group, int K, int renorm, float scale, int64_t *__restrict__ experts_out,
    float *__restrict__ weights_out) {
    __shared__ float choice_lds[TOKENS_PER_BLOCK][PER * 64];
    const int lane = threadIdx.x & 63;
    const int wv = threadIdx.x >> 6;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * TOKENS_PER_BLOCK + wv;
    if (t >= Tn) return;  // whole wavefront leaves together; no block-wide barrier below
    float score[PER], choice[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        if (i < N) {
            const float x = logits[t * N + i];
            score[j] = 1.0f / (1.0f + expf(-x));
            choice[j] = score[j] + bias[i];
            choice_lds[wv][i] = choice[j];
        } else {
            score[j] = 0.0f;
            choice[j] = -INFINITY;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // lane g < n_group: sum of the two largest choice values of group g
    const int gs = N / n_group;
    float gscore = -INFINITY;
    if (lane < n_group) {
        float a = -INFINITY, b = -INFINITY;
        for (int i = 0; i < gs; i++) {
            const float v = choice_lds[wv][lane * gs + i];
            if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
        }
        gscore = (gs >= 2) ? (a + b) : a;
    }
    // keep the topk_group best groups (score desc, group index asc)
    unsigned long long keep = 0ull;
    for (int r = 0; r < topk_group; r++) {
        float bv = gscore; int bi = (lane < n_group) ? lane : 0x7fffffff;
        wave_argmax(bv, bi);
        keep |= (1ull << bi);
        if (lane == bi) gscore = -INFINITY;
    }
    // masked_fill(~mask, 0.0): dropped groups compete with the value 0.0
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        if (i < N && !((keep >> (i / gs)) & 1ull)) choice[j] = 0.0f;
    }
    float cv; int e;
    select_topk<PER>(choice, N, K, lane, cv, e);
    // weight = sigmoid score (no bias) at the selected expert
    float w = fetch_expert_value<PER>(score, e);
    if (lane >= K) w = 0.0f;
    if (renorm) {
        const float S = wave_sum(lane < K ? w : 0.0f) + 1e-20f;
        w = w / S;
    }
    w = w * scale;
    if (lane < K) {
        experts_out[t * K + lane] = e;
        weights_out[t * K + lane] = w;
    }
}

// w'_k = scale * s_k / (S + 1e-20) (or scale * s_k); ds_k -> dlogit = ds * s * (1 - s).
template <int PER>
__global__ __launch_bounds__(256) void sigmoid_topk_bwd_kernel(const float *__restrict__ logits,
                                                               const int64_t *__restrict__ experts,
                                                               const float *__restrict__ dweights,
                                                               int64_t Tn, int N, int K, int renorm,
                                                               float scale, float *__restrict__ dlogits) {
    const int lane = threadIdx.x & 63;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * TOKENS_PER_BLOCK + (threadIdx.x >> 6);
    if (t >= Tn) return;
    const int e = (lane < K) ? static_cast<int>(experts[t * K + lane]) : -1;
    float sk = 0.0f;
    if (lane < K) sk = 1.0f / (1.0f + expf(-logits[t * N + e]));
    float d = (lane < K) ? dweights[t * K + lane] * scale : 0.0f;  // through "* scale"
    if (renorm) {
        const float S = wave_sum(sk) + 1e-20f;
        const float dot = wave_sum(d * sk);
        d = (d - dot / S) / S;
    }
    const float dl = d * (sk * (1.0f - sk));
    float out[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) out[j] = 0.0f;
    for (int k = 0; k < K; k++) {
        const int ek = __shfl(e, k, 64);
        const float dk = __shfl(dl, k, 64);
#pragma unroll
        for (int j = 0; j < PER; j++)
            if (lane + 64 * j == ek) out[j] += dk;
    }
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        if (i < N) dlogits[t * N + i] = out[j];
    }
}

// Router gate fused with the routing: logits = x @ Wg^T for 32 tokens per block on the matrix
// cores (bf16 operands whose products are exact in fp32, fp32 accumulation: the value of
// x.float() @ Wg.float().T up to the order of the sum), the contraction split over the block's
// wavefronts and reduced through LDS in a fixed order, then softmax / top-K of those tokens
// straight from LDS.  x is read from HBM exactly once (the pass is HBM-bound on it); Wg stays in L2.
// Operand fragments come straight from global memory in MFMA layout (lane = row, 8 consecutive
// h): the four loads that share a 128-byte line are issued together.
template <int NB, int WAVES, int UNR, int PER, typename TW, bool ROUTE>
__global__ __launch_bounds__(WAVES * 64) void gate_route_kernel(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ wg, int64_t Tn, int H, int N, int K,
    int renorm, float *__restrict__ logits_out, TW *__restrict__ weights_out,
    int64_t *__restrict__ experts_out) {
    constexpr int NP = NB * 32;  // expert count rounded up to the MFMA block
    __shared__ float part[WAVES][32][NP];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * 32;
    const int hw = H / WAVES;
    const int r32 = lane & 31, kofs = (lane >> 5) * 8;
    int64_t ta = t0 + r32;
    if (ta >= Tn) ta = Tn - 1;  // rows past the end: valid memory, result unused
    const uint16_t *ap = x + ta * H + wave * hw + kofs;
    const uint16_t *bp[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        int e = j * 32 + r32;
        if (e >= N) e = N - 1;
        bp[j] = wg + static_cast<int64_t>(e) * H + wave * hw + kofs;
    }
    f32x16 acc[NB];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = 0.0f;
    for (int h = 0; h < hw; h += 16 * UNR) {
        u32x4 a[UNR], b[NB][UNR];
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            a[u] = *reinterpret_cast<const u32x4 *>(ap + h + u * 16);
#pragma unroll
            for (int j = 0; j < NB; j++) b[j][u] = *reinterpret_cast<const u32x4 *>(bp[j] + h + u * 16);
        }
#pragma unroll
        for (int u = 0; u < UNR; u++)
#pragma unroll
            for (int j = 0; j < NB; j++)
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[u]),
                                                                 __builtin_bit_cast(bf16x8, b[j][u]),
                                                                 acc[j], 0, 0, 0);
    }
    // accumulator element r of lane l: token (r/4)*8 + (l/32)*4 + r%4, expert j*32 + l%32
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            part[wave][(r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)][j * 32 + r32] = acc[j][r];
    __syncthreads();
    for (int idx = threadIdx.x; idx < 32 * NP; idx += WAVES * 64) {
        const int row = idx / NP, col = idx % NP;
        float sum = part[0][row][col];
#pragma unroll
        for (int w = 1; w < WAVES; w++) sum += part[w][row][col];
        part[0][row][col] = sum;
        if (logits_out && t0 + row < Tn && col < N) logits_out[(t0 + row) * N + col] = sum;
    }
    if (!ROUTE) return;
    __syncthreads();
    for (int tk = wave; tk < 32; tk += WAVES) {
        const int64_t t = t0 + tk;
        if (t >= Tn) break;
        float p[PER];
        row_softmax<PER, float>(&part[0][tk][0], N, lane, p);
        float w; int e;
        select_topk<PER>(p, N, K, lane, w, e);
        if (renorm) {
            const float sk = wave_sum(lane < K ? w : 0.0f);
            w = w / sk;
        }
        if (lane < K) {
            Elem<TW>::store(weights_out + t * K + lane, w);
            experts_out[t * K + lane] = e;
        }
    }
}

template <bool ROUTE, typename TW>
int launch_gate(const void *x, const void *wg, int64_t T, int H, int N, int K, int renorm,
                float *logits_out, void *weights_out, int64_t *experts_out, hipStream_t st) {
    const unsigned nb = static_cast<unsigned>((T + 31) / 32);
    const uint16_t *xp = static_cast<const uint16_t *>(x), *wp = static_cast<const uint16_t *>(wg);
    TW *wo = static_cast<TW *>(weights_out);
#define OM_GATE(NB, WAVES, UNR, PER)                                                              \
    do {                                                                                          \
        if (H % (WAVES * 16 * UNR) != 0) return OM_ERR_SHAPE;                                     \
        gate_route_kernel<NB, WAVES, UNR, PER, TW, ROUTE><<<nb, WAVES * 64, 0, st>>>(             \
            xp, wp, T, H, N, K, renorm, logits_out, wo, experts_out);                             \
    } while (0)
    if (N <= 32) OM_GATE(1, 8, 4, 1);
    else if (N <= 64) OM_GATE(2, 8, 4, 1);
    else if (N <= 128) OM_GATE(4, 8, 2, 2);
    else OM_GATE(8, 4, 1, 4);
#undef OM_GATE
    return om_launch_status();
}

// Load-balancing statistics of one layer's router logits: for every expert the sum over tokens
// of its softmax probability and the number of tokens whose top-K contains it (the two factors of
// the auxiliary loss, reference optimus/models/olmoe/modeling_olmoe.py:29-85).  A block walks
// BAL_TOKENS tokens, one wavefront per token at a time, and leaves one partial row; a second
// kernel adds the rows in block order, so the result does not depend on scheduling.
constexpr int BAL_TOKENS = 64;
template <int PER, typename T>
__global__ __launch_bounds__(256) void balance_stats_kernel(const T *__restrict__ logits,
                                                            const float *__restrict__ token_weight,
                                                            int64_t Tn, int N, int K,
                                                            float *__restrict__ part_prob,
                                                            float *__restrict__ part_count) {
    __shared__ float lds_p[4][PER * 64];
    __shared__ float lds_c[4][PER * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float psum[PER];
    float cnt[PER];   // sums of token weights; whole numbers (exact) for 0/1 weights and without weights
#pragma unroll
    for (int j = 0; j < PER; j++) { psum[j] = 0.0f; cnt[j] = 0.0f; }
    const int64_t t_first = static_cast<int64_t>(blockIdx.x) * BAL_TOKENS;
    for (int i = wave; i < BAL_TOKENS; i += 4) {
        const int64_t t = t_first + i;
        if (t >= Tn) break;
        const float tw = token_weight ? token_weight[t] : 1.0f;   // the token's attention-mask entry
        float p[PER], s[PER];
        row_softmax<PER, T>(logits + t * N, N, lane, p);
#pragma unroll
        for (int j = 0; j < PER; j++) { psum[j] += token_weight ? tw * p[j] : p[j]; s[j] = p[j]; }
        float w; int e;
        select_topk<PER>(s, N, K, lane, w, e);
        for (int k = 0; k < K; k++) {
            const int ek = __shfl(e, k, 64);
#pragma unroll
            for (int j = 0; j < PER; j++)
                if (lane + 64 * j == ek) cnt[j] += tw;
        }
    }
#pragma unroll
    for (int j = 0; j < PER; j++) { lds_p[wave][lane + 64 * j] = psum[j]; lds_c[wave][lane + 64 * j] = cnt[j]; }
    __syncthreads();
    for (int i = threadIdx.x; i < N; i += 256) {
        part_prob[static_cast<int64_t>(blockIdx.x) * N + i] = (lds_p[0][i] + lds_p[1][i]) + (lds_p[2][i] + lds_p[3][i]);
        part_count[static_cast<int64_t>(blockIdx.x) * N + i] = (lds_c[0][i] + lds_c[1][i]) + (lds_c[2][i] + lds_c[3][i]);
    }
}

__global__ __launch_bounds__(256) void balance_reduce_kernel(const float *__restrict__ part_prob,
                                                             const float *__restrict__ part_count,
                                                             int n_blocks, int N,
                                                             float *__restrict__ prob_sum,
                                                             float *__restrict__ count) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    float ps = 0.0f;
    // a block's partial is a sum of at most BAL_TOKENS token weights (whole numbers for 0/1 weights
    // and without weights); adding the partials in double keeps whole-number counts exact at any
    // token count (a hot expert can exceed 2^24 tokens), one rounding to float at the end
    double c = 0.0;
    for (int b = 0; b < n_blocks; b++) {
        ps += part_prob[static_cast<int64_t>(b) * N + i];
        c += static_cast<double>(part_count[static_cast<int64_t>(b) * N + i]);
    }
    prob_sum[i] = ps;
    count[i] = static_cast<float>(c);
}

// dlogits[t,i] = p_i * (g_i - sum_j p_j g_j): the softmax backward of sum_i g_i * p[t,i].
template <int PER, typename T>
__global__ __launch_bounds__(256) void balance_bwd_kernel(const T *__restrict__ logits,
                                                          const float *__restrict__ g,
                                                          const float *__restrict__ token_weight,
                                                          int64_t Tn, int N, T *__restrict__ dlogits) {
    const int lane = threadIdx.x & 63;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * TOKENS_PER_BLOCK + (threadIdx.x >> 6);
    if (t >= Tn) return;
    float p[PER];
    row_softmax<PER, T>(logits + t * N, N, lane, p);
    float gv[PER], dot = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        gv[j] = (i < N) ? g[i] : 0.0f;
        dot += p[j] * gv[j];
    }
    dot = wave_sum(dot);
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int i = lane + 64 * j;
        if (i < N) Elem<T>::store(dlogits + t * N + i, (token_weight ? token_weight[t] : 1.0f) * (p[j] * (gv[j] - dot)));
    }
}

inline unsigned token_blocks(int64_t T) {
    return static_cast<unsigned>((T + TOKENS_PER_BLOCK - 1) / TOKENS_PER_BLOCK);
}
inline int per_lane(int N) { return N <= 64 ? 1 : N <= 128 ? 2 : N <= 256 ? 4 : 8; }

}  // namespace

#define OM_DISPATCH_PER(N, CALL)              \
    switch (per_lane(N)) {                    \
        case 1: { constexpr int PER = 1; CALL; } break; \
        case 2: { constexpr int PER = 2; CALL; } break; \
        case 4: { constexpr int PER = 4; CALL; } break; \
        default: { constexpr int PER = 8; CALL; } break; \
    }

extern "C" int om_route_softmax_topk(const void *logits, int logits_dtype, int64_t T, int N, int K,
                                     int norm_topk_prob, void *weights_out, int weights_dtype,
                                     int64_t *experts_out, void *stream) {
    if ((logits_dtype != OM_F32 && logits_dtype != OM_BF16) ||
        (weights_dtype != OM_F32 && weights_dtype != OM_BF16))
        return OM_ERR_DTYPE;
    if (T < 0 || N < 1 || N > 512 || K < 1 || K > N || K > 64 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!logits || !weights_out || !experts_out) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = token_blocks(T);
#define OM_RT(TL, TW)                                                                          \
    OM_DISPATCH_PER(N, (softmax_topk_kernel<PER, TL, TW><<<nb, 256, 0, st>>>(                  \
                           static_cast<const TL *>(logits), T, N, K, norm_topk_prob,           \
                           static_cast<TW *>(weights_out), experts_out)))
    if (logits_dtype == OM_F32 && weights_dtype == OM_F32) { OM_RT(float, float); }
    else if (logits_dtype == OM_F32) { OM_RT(float, uint16_t); }
    else if (weights_dtype == OM_F32) { OM_RT(uint16_t, float); }
    else { OM_RT(uint16_t, uint16_t); }
#undef OM_RT
    return om_launch_status();
}

extern "C" int om_route_softmax_topk_bwd(const void *logits, int logits_dtype, const int64_t *experts,
                                         const void *dweights, int weights_dtype, int64_t T, int N,
                                         int K, int norm_topk_prob, void *dlogits, void *stream) {
    if ((logits_dtype != OM_F32 && logits_dtype != OM_BF16) ||
        (weights_dtype != OM_F32 && weights_dtype != OM_BF16))
        return OM_ERR_DTYPE;
    if (T < 0 || N < 1 || N > 512 || K < 1 || K > N || K > 64 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!logits || !experts || !dweights || !dlogits) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = token_blocks(T);
#define OM_RB(TL, TW)                                                                          \
    OM_DISPATCH_PER(N, (softmax_topk_bwd_kernel<PER, TL, TW><<<nb, 256, 0, st>>>(              \
                           static_cast<const TL *>(logits), experts,                           \
                           static_cast<const TW *>(dweights), T, N, K, norm_topk_prob,         \
                           static_cast<TL *>(dlogits))))
    if (logits_dtype == OM_F32 && weights_dtype == OM_F32) { OM_RB(float, float); }
    else if (logits_dtype == OM_F32) { OM_RB(float, uint16_t); }
    else if (weights_dtype == OM_F32) { OM_RB(uint16_t, float); }
    else { OM_RB(uint16_t, uint16_t); }
#undef OM_RB
    return om_launch_status();
}

extern "C" int om_route_sigmoid_group_topk(const float *logits, const float *bias, int64_t T, int N,
                                           int n_group, int topk_group, int K, int norm_topk_prob,
                                           double routed_scaling_factor, int64_t *experts_out,
                                           float *weights_out, void *stream) {
    if (T < 0 || N < 1 || N > 512 || K < 1 || K > N || K > 64 || n_group < 1 || n_group > 64 ||
        N % n_group != 0 || topk_group < 1 || topk_group > n_group || T > 0x7fffffffLL)
        return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!logits || !bias || !experts_out || !weights_out) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = token_blocks(T);
    const float scale = static_cast<float>(routed_scaling_factor);
    OM_DISPATCH_PER(N, (sigmoid_group_topk_kernel<PER><<<nb, 256, 0, st>>>(
                           logits, bias, T, N, n_group, topk_group, K, norm_topk_prob, scale,
                           experts_out, weights_out)));
    return om_launch_status();
}

extern "C" int om_route_sigmoid_topk_bwd(const float *logits, const int64_t *experts,
                                         const float *dweights, int64_t T, int N, int K,
                                         int norm_topk_prob, double routed_scaling_factor,
                                         float *dlogits, void *stream) {
    if (T < 0 || N < 1 || N > 512 || K < 1 || K > N || K > 64 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!logits || !experts || !dweights || !dlogits) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = token_blocks(T);
    const float scale = static_cast<float>(routed_scaling_factor);
    OM_DISPATCH_PER(N, (sigmoid_topk_bwd_kernel<PER><<<nb, 256, 0, st>>>(
                           logits, experts, dweights, T, N, K, norm_topk_prob, scale, dlogits)));
    return om_launch_status();
}

extern "C" int om_router_gate_softmax_topk(const void *x, const void *gate_weight, int64_t T, int H,
                                           int N, int K, int norm_topk_prob, float *logits_out,
                                           void *weights_out, int weights_dtype, int64_t *experts_out,
                                           void *stream) {
    if (weights_dtype != OM_F32 && weights_dtype != OM_BF16) return OM_ERR_DTYPE;
    if (T < 0 || H < 1 || H % 8 != 0 || N < 1 || N > 256 || K < 1 || K > N || K > 64 ||
        T > 0x7fffffffLL)
        return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!x || !gate_weight || !weights_out || !experts_out) return OM_ERR_NULL;
    if (!om_aligned16(x) || !om_aligned16(gate_weight)) return OM_ERR_ALIGN;
    hipStream_t st = om_stream(stream);
    if (weights_dtype == OM_F32)
        return launch_gate<true, float>(x, gate_weight, T, H, N, K, norm_topk_prob, logits_out,
                                        weights_out, experts_out, st);
    return launch_gate<true, uint16_t>(x, gate_weight, T, H, N, K, norm_topk_prob, logits_out,
                                       weights_out, experts_out, st);
}

extern "C" int om_router_gate_logits(const void *x, const void *gate_weight, int64_t T, int H, int N,
                                     float *logits_out, void *stream) {
    if (T < 0 || H < 1 || H % 8 != 0 || N < 1 || N > 256 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!x || !gate_weight || !logits_out) return OM_ERR_NULL;
    if (!om_aligned16(x) || !om_aligned16(gate_weight)) return OM_ERR_ALIGN;
    return launch_gate<false, float>(x, gate_weight, T, H, N, 1, 0, logits_out, nullptr, nullptr,
                                     om_stream(stream));
}

extern "C" int64_t om_router_balance_workspace_bytes(int64_t T, int N) {
    if (T < 0 || N < 1) return 0;
    const int64_t blocks = (T + BAL_TOKENS - 1) / BAL_TOKENS;
    return blocks * N * 8;   // one float and one int per (block, expert)
}

extern "C" int om_router_balance_stats_masked(const void *logits, int logits_dtype,
                                              const float *token_weight, int64_t T, int N, int K,
                                              float *prob_sum, float *count, void *workspace,
                                              int64_t workspace_bytes, void *stream) {
    if (logits_dtype != OM_F32 && logits_dtype != OM_BF16) return OM_ERR_DTYPE;
    if (T < 1 || N < 1 || N > 512 || K < 1 || K > N || K > 64 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (!logits || !prob_sum || !count || !workspace) return OM_ERR_NULL;
    if (workspace_bytes < om_router_balance_workspace_bytes(T, N)) return OM_ERR_WORKSPACE;
    hipStream_t st = om_stream(stream);
    const int nb = static_cast<int>((T + BAL_TOKENS - 1) / BAL_TOKENS);
    float *pp = static_cast<float *>(workspace);
    float *pc = pp + static_cast<int64_t>(nb) * N;
    if (logits_dtype == OM_F32) {
        OM_DISPATCH_PER(N, (balance_stats_kernel<PER, float><<<nb, 256, 0, st>>>(
                               static_cast<const float *>(logits), token_weight, T, N, K, pp, pc)));
    } else {
        OM_DISPATCH_PER(N, (balance_stats_kernel<PER, uint16_t><<<nb, 256, 0, st>>>(
                               static_cast<const uint16_t *>(logits), token_weight, T, N, K, pp, pc)));
    }
    balance_reduce_kernel<<<(N + 255) / 256, 256, 0, st>>>(pp, pc, nb, N, prob_sum, count);
    return om_launch_status();
}

extern "C" int om_router_balance_stats(const void *logits, int logits_dtype, int64_t T, int N, int K,
                                       float *prob_sum, float *count, void *workspace,
                                       int64_t workspace_bytes, void *stream) {
    return om_router_balance_stats_masked(logits, logits_dtype, nullptr, T, N, K, prob_sum, count,
                                          workspace, workspace_bytes, stream);
}

extern "C" int om_router_balance_bwd_masked(const void *logits, int logits_dtype, const float *prob_grad,
                                            const float *token_weight, int64_t T, int N, void *dlogits,
                                            void *stream) {
    if (logits_dtype != OM_F32 && logits_dtype != OM_BF16) return OM_ERR_DTYPE;
    if (T < 0 || N < 1 || N > 512 || T > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!logits || !prob_grad || !dlogits) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = token_blocks(T);
    if (logits_dtype == OM_F32) {
        OM_DISPATCH_PER(N, (balance_bwd_kernel<PER, float><<<nb, 256, 0, st>>>(
                               static_cast<const float *>(logits), prob_grad, token_weight, T, N,
                               static_cast<float *>(dlogits))));
    } else {
        OM_DISPATCH_PER(N, (balance_bwd_kernel<PER, uint16_t><<<nb, 256, 0, st>>>(
                               static_cast<const uint16_t *>(logits), prob_grad, token_weight, T, N,
                               static_cast<uint16_t *>(dlogits))));
    }
    return om_launch_status();
}

extern "C" int om_router_balance_bwd(const void *logits, int logits_dtype, const float *prob_grad,
                                     int64_t T, int N, void *dlogits, void *stream) {
    return om_router_balance_bwd_masked(logits, logits_dtype, prob_grad, nullptr, T, N, dlogits, stream);
}
