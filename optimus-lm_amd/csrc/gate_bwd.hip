// Backward of the router's gate projection `router_logits = self.gate(hidden_states)` (reference
// optimus/models/common/moe.py:456, the gate nn.Linear of optimus/models/olmoe/modeling_olmoe.py):
// the weight gradient dW[n,h] = sum_t dlogits[t,n] * x[t,h] (first part of this file) and the input
// gradient dx[t,h] = sum_n dlogits[t,n] * W[n,h] (second part).
//
// The product is [N x T] x [T x H] with N = number of experts (tens to a few hundred), H the
// hidden size and T the tokens: a tiny output and a long contraction.  A library GEMM gives it a
// handful of tiles, i.e. a handful of CUs.  Here the token range is split over many blocks; every
// block contracts its tokens for one 128-column slice of H on bf16 MFMA with fp32 accumulation
// and writes an fp32 partial; a second kernel adds the partials in a fixed order (deterministic)
// and rounds once.  dlogits (fp32) is rounded to bf16 on the way into LDS, the precision a bf16
// gate's backward has anyway; bf16 x bf16 products are exact in fp32.
//
// Both operands are stored token-major ([t][n], [t][h]) while the MFMA wants, per lane, 8
// consecutive contraction indices (tokens) of one row.  The tiles are kept in LDS as they lie in
// memory and the fragments come from the transposing LDS read (ds_read_b64_tr_b16).  HBM-bound:
// x is read once (2 B per element), dlogits comes from L2 for all but the first column slice.
#include "common.h"

namespace {

typedef __attribute__((address_space(3))) s16x4 *lds_s16x4_ptr;
typedef __attribute__((ext_vector_type(8))) short s16x8;

constexpr int HT = 128;   // columns of H per block
constexpr int TC = 64;    // tokens per LDS stage

// Tile [TC token rows][R operand rows] of bf16, R*2-byte token rows, 16-byte chunk `ch` of token row
// `crow` stored at chunk position ch ^ ((crow & 3) << 2): the four token rows one transposing read
// touches fall into four different 64-byte bank windows.  Needs R >= 128 (16 chunks per row).
template <int R> __device__ __forceinline__ int tile_off(int crow, int ch) {
    return crow * (R * 2) + ((ch ^ ((crow & 3) << 2)) << 4);
}

// MFMA 32x32x16 operand fragment: lane l gets operand row m0 + l%32, tokens c0 + 8*(l/32) .. +7.
template <int R>
__device__ __forceinline__ bf16x8 read_frag(const char *tile, int c0, int m0, int lane) {
    const int i = lane & 15;
    const int r = i >> 2, q = i & 3;
    const int mb = ((lane >> 4) & 1) * 16;
    const int g2 = lane >> 5;
    const int m = m0 + mb + 4 * q;
    const int cr = c0 + 8 * g2 + r;
    const char *p = tile + tile_off<R>(cr, m >> 3) + (m & 7) * 2;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * R * 2));
    return __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

__device__ __forceinline__ uint32_t pack2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    f32x2 f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// grid (H / 128, splits); 256 threads.  NB accumulators per wavefront cover N = 32 NB rows of dW, of
// which the first n_real exist (the rest are zero columns of the dlogits tile); wavefront w owns
// the 32 columns [h0 + 32 w, h0 + 32 w + 32) of the block's slice and all rows of dW.
template <int NB>
__global__ __launch_bounds__(256) void gate_wgrad_kernel(const uint16_t *__restrict__ x,
                                                         const float *__restrict__ dlogits,
                                                         int64_t T, int H, int n_real,
                                                         int64_t tokens_per_split,
                                                         float *__restrict__ partial) {
    constexpr int N = NB * 32;
    constexpr int RD = N < 128 ? 128 : N;       // LDS row length of the dlogits tile (elements)
    constexpr int XL = TC * HT / 8 / 256;       // 16-byte x chunks per thread per stage
    constexpr int DL = TC * N / 4 / 256;        // float4 dlogits loads per thread per stage
    __shared__ __attribute__((aligned(16))) char xs[TC * HT * 2];
    __shared__ __attribute__((aligned(16))) char ds[TC * RD * 2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h0 = blockIdx.x * HT;
    const int64_t t_begin = static_cast<int64_t>(blockIdx.y) * tokens_per_split;
    int64_t t_end = t_begin + tokens_per_split;
    if (t_end > T) t_end = T;

    f32x16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][r] = 0.0f;

    u32x4 xq[XL];
    f32x4 dq[DL];
    auto fetch = [&](int64_t t0) {   // tokens past t_end contribute zeros
#pragma unroll
        for (int j = 0; j < XL; j++) {
            const int q = j * 256 + tid;
            const int64_t t = t0 + q / (HT / 8);
            xq[j] = u32x4{0, 0, 0, 0};
            const int hc = h0 + (q % (HT / 8)) * 8;     // the last column slice may be partial
            if (t < t_end && hc < H) xq[j] = *reinterpret_cast<const u32x4 *>(x + t * H + hc);
        }
#pragma unroll
        for (int j = 0; j < DL; j++) {
            const int q = j * 256 + tid;
            const int64_t t = t0 + q / (N / 4);
            const int col = (q % (N / 4)) * 4;
            dq[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (t < t_end && col < n_real) {
                const float *src = dlogits + t * n_real + col;
                if ((n_real & 3) == 0) {
                    dq[j] = *reinterpret_cast<const f32x4 *>(src);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (col + i < n_real) dq[j][i] = src[i];
                }
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int j = 0; j < XL; j++) {
            const int q = j * 256 + tid;
            *reinterpret_cast<u32x4 *>(xs + tile_off<HT>(q / (HT / 8), q % (HT / 8))) = xq[j];
        }
#pragma unroll
        for (int j = 0; j < DL; j++) {
            const int q = j * 256 + tid;
            const int crow = q / (N / 4), n = (q % (N / 4)) * 4;
            u32x2 v;
            v[0] = pack2(dq[j][0], dq[j][1]);
            v[1] = pack2(dq[j][2], dq[j][3]);
            *reinterpret_cast<u32x2 *>(ds + tile_off<RD>(crow, n >> 3) + (n & 7) * 2) = v;
        }
    };

    if (t_begin < t_end) fetch(t_begin);
    for (int64_t t0 = t_begin; t0 < t_end; t0 += TC) {
        __syncthreads();             // the previous stage has been read
        stash();
        __syncthreads();
        if (t0 + TC < t_end) fetch(t0 + TC);   // in flight under the MFMAs below
#pragma unroll
        for (int kk = 0; kk < TC / 16; kk++) {
            const bf16x8 fx = read_frag<HT>(xs, kk * 16, wave * 32, lane);
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const bf16x8 fd = read_frag<RD>(ds, kk * 16, b * 32, lane);
                // lane l then holds column h = l % 32 and rows n = 8*(r/4) + 4*(l/32) + r%4
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fd, fx, acc[b], 0, 0, 0);
            }
        }
    }
    const int h = h0 + wave * 32 + (lane & 31);
    float *out = partial + (static_cast<int64_t>(blockIdx.y) * n_real) * H + h;
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int n = b * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (n < n_real && h < H) out[static_cast<int64_t>(n) * H] = acc[b][r];
        }
}

// dW = sum over splits, in split order; 4 elements per thread.
template <typename T>
__global__ __launch_bounds__(256) void gate_wgrad_reduce_kernel(const float *__restrict__ partial,
                                                                int splits, int64_t nh, T *__restrict__ dw) {
    const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i >= nh) return;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < splits; k0 += 8) {   // eight loads in flight, added in split order
        f32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
            v[u] = (k0 + u < splits) ? *reinterpret_cast<const f32x4 *>(partial + (k0 + u) * nh + i)
                                     : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 8; u++) { s[0] += v[u][0]; s[1] += v[u][1]; s[2] += v[u][2]; s[3] += v[u][3]; }
    }
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<f32x4 *>(dw + i) = s;
    } else {
        u32x2 v;
        v[0] = pack2(s[0], s[1]);
        v[1] = pack2(s[2], s[3]);
        *reinterpret_cast<u32x2 *>(dw + i) = v;
    }
}

// Token ranges: enough blocks to fill the chip twice over, at least two stages each.
inline int gate_wgrad_splits(int64_t T, int H) {
    const int64_t stages = (T + TC - 1) / TC;
    const int slices = (H + HT - 1) / HT;
    int64_t want = (2 * 256 + slices - 1) / slices;   // ~2 blocks per CU
    if (want > stages / 2) want = stages / 2;
    if (want < 1) want = 1;
    if (want > 256) want = 256;
    return static_cast<int>(want);
}

inline bool gate_wgrad_shape_ok(int64_t T, int H, int N) {
    return T >= 0 && H > 0 && H % 8 == 0 && N >= 1 && N <= 256;   // 16-byte chunks of x
}

// ---- input gradient of the gate projection ---------------------------------------------------
// dx[t,h] = sum_n bf16(dlogits[t,n]) * W[n,h], optionally added to another gradient of the same
// tensor (the experts' input gradient): out = bf16(float(base) + float(bf16(sum))), the two
// roundings autograd's "matmul, then accumulate" has.  [T x N] x [N x H] with a short contraction:
// a block owns 128 tokens x 128 columns; W's [N x 128] slice sits in LDS as it lies in memory and is
// read through the transposing LDS read; a lane's dlogits fragment (8 consecutive n of one token)
// comes straight from global memory.  The results leave through per-wavefront LDS strips so that
// every store (and the read of `base`) covers whole 256-byte row segments.
constexpr int DG_HT = 128, DG_TOK = 128;
constexpr int DG_PITCH = DG_HT * 2 + 8;             // strip row pitch: conflict-free 8-byte accesses
constexpr int DG_STRIPS = 4 * 32 * DG_PITCH;        // four wavefronts x 32 token rows

inline size_t gate_dgrad_lds(int N) {
    const size_t w = static_cast<size_t>((N + 15) & ~15) * DG_HT * 2;
    return w > DG_STRIPS ? w : DG_STRIPS;
}

__global__ __launch_bounds__(256) void gate_dgrad_kernel(const float *__restrict__ dlogits,
                                                         const uint16_t *__restrict__ weight,
                                                         const uint16_t *base, uint16_t *out, int64_t T,
                                                         int H, int N) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h0 = blockIdx.x * DG_HT;
    const int64_t t0 = static_cast<int64_t>(blockIdx.y) * DG_TOK + wave * 32;
    const int n_pad = (N + 15) & ~15;
    for (int q = tid; q < n_pad * (DG_HT / 8); q += 256) {
        const int n = q / (DG_HT / 8), ch = q % (DG_HT / 8);
        u32x4 v = {0, 0, 0, 0};
        if (n < N && h0 + ch * 8 < H)
            v = *reinterpret_cast<const u32x4 *>(weight + static_cast<int64_t>(n) * H + h0 + ch * 8);
        *reinterpret_cast<u32x4 *>(lds + tile_off<DG_HT>(n, ch)) = v;
    }
    __syncthreads();
    f32x16 acc[DG_HT / 32];
#pragma unroll
    for (int b = 0; b < DG_HT / 32; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[b][r] = 0.0f;
    const int64_t t = t0 + (lane & 31);
    const float *drow = dlogits + t * N;
    for (int kk = 0; kk < n_pad; kk += 16) {
        const int nb = kk + 8 * (lane >> 5);
        float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (t < T) {
            if ((N & 3) == 0) {   // 16-byte aligned rows
#pragma unroll
                for (int half = 0; half < 2; half++)
                    if (nb + 4 * half < N) {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(drow + nb + 4 * half);
#pragma unroll
                        for (int i = 0; i < 4; i++) d[4 * half + i] = v[i];
                    }
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (nb + i < N) d[i] = drow[nb + i];
            }
        }
        u32x4 packed = {pack2(d[0], d[1]), pack2(d[2], d[3]), pack2(d[4], d[5]), pack2(d[6], d[7])};
        const bf16x8 fd = __builtin_bit_cast(bf16x8, packed);
#pragma unroll
        for (int b = 0; b < DG_HT / 32; b++) {
            const bf16x8 fw = read_frag<DG_HT>(lds, kk, b * 32, lane);
            // lane l then holds token l % 32 and columns 32 b + 8*(r/4) + 4*(l/32) + r%4
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw, fd, acc[b], 0, 0, 0);
        }
    }
    __syncthreads();   // the weight tile is dead; its memory becomes the strips
    char *strip = lds + wave * (32 * DG_PITCH);
#pragma unroll
    for (int b = 0; b < DG_HT / 32; b++)
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
            u32x2 v;
            v[0] = pack2(acc[b][rq * 4], acc[b][rq * 4 + 1]);
            v[1] = pack2(acc[b][rq * 4 + 2], acc[b][rq * 4 + 3]);
            const int col = b * 32 + rq * 8 + (lane >> 5) * 4;
            *reinterpret_cast<u32x2 *>(strip + (lane & 31) * DG_PITCH + col * 2) = v;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int it = 0; it < 32 * (DG_HT / 8) / 64; it++) {
        const int q = it * 64 + lane;
        const int row = q / (DG_HT / 8), ch = q % (DG_HT / 8);
        const int64_t tt = t0 + row;
        const int h = h0 + ch * 8;
        if (tt < T && h < H) {
            const char *sp = strip + row * DG_PITCH + ch * 16;
            const u32x2 lo = *reinterpret_cast<const u32x2 *>(sp);
            const u32x2 hi = *reinterpret_cast<const u32x2 *>(sp + 8);
            u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
            const int64_t o = tt * H + h;
            if (base) {
                float a[8], g[8];
                Elem<uint16_t>::unpack(__builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + o)), a);   // read once
                Elem<uint16_t>::unpack(v, g);
#pragma unroll
                for (int i = 0; i < 8; i++) a[i] = a[i] + g[i];
                v = Elem<uint16_t>::pack(a);
            }
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out + o));
        }
    }
}

}  // namespace

extern "C" int om_router_gate_dgrad(const float *dlogits, const void *gate_weight, const void *base,
                                    void *dx, int64_t T, int H, int N, void *stream) {
    if (T < 0 || H < 8 || H % 8 != 0 || N < 1 || N > 256) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!dlogits || !gate_weight || !dx) return OM_ERR_NULL;
    if (!om_aligned16(dlogits) || !om_aligned16(gate_weight) || !om_aligned16(dx) || !om_aligned16(base))
        return OM_ERR_ALIGN;
    const int64_t t_blocks = (T + DG_TOK - 1) / DG_TOK;
    if (t_blocks > 65535) {
        // the token blocks ride on the grid's second dimension: split long inputs into several launches
        const int64_t per = 65535LL * DG_TOK;
        for (int64_t done = 0; done < T; done += per) {
            const int64_t cnt = T - done < per ? T - done : per;
            const int rc = om_router_gate_dgrad(
                dlogits + done * N, gate_weight,
                base ? static_cast<const uint16_t *>(base) + done * H : nullptr,
                static_cast<uint16_t *>(dx) + done * H, cnt, H, N, stream);
            if (rc != OM_OK) return rc;
        }
        return OM_OK;
    }
    const dim3 grid((H + DG_HT - 1) / DG_HT, static_cast<unsigned>(t_blocks));
    gate_dgrad_kernel<<<grid, dim3(256), gate_dgrad_lds(N), om_stream(stream)>>>(
        dlogits, static_cast<const uint16_t *>(gate_weight), static_cast<const uint16_t *>(base),
        static_cast<uint16_t *>(dx), T, H, N);
    return om_launch_status();
}

extern "C" int64_t om_router_gate_wgrad_workspace_bytes(int64_t T, int H, int N) {
    if (!gate_wgrad_shape_ok(T, H, N)) return OM_ERR_SHAPE;
    return static_cast<int64_t>(gate_wgrad_splits(T, H)) * N * H * 4;
}

extern "C" int om_router_gate_wgrad(const void *x, const float *dlogits, int64_t T, int H, int N,
                                    void *dweight, int dweight_dtype, void *workspace,
                                    int64_t workspace_bytes, void *stream) {
    if (dweight_dtype != OM_BF16 && dweight_dtype != OM_F32) return OM_ERR_DTYPE;
    if (!gate_wgrad_shape_ok(T, H, N)) return OM_ERR_SHAPE;
    if (!dweight || !workspace) return OM_ERR_NULL;
    if (T > 0 && (!x || !dlogits)) return OM_ERR_NULL;
    if (!om_aligned16(x) || !om_aligned16(dlogits) || !om_aligned16(dweight) || !om_aligned16(workspace))
        return OM_ERR_ALIGN;
    const int splits = gate_wgrad_splits(T, H);
    const int64_t nh = static_cast<int64_t>(N) * H;
    if (workspace_bytes < splits * nh * 4) return OM_ERR_WORKSPACE;
    hipStream_t st = om_stream(stream);
    const int64_t stages = (T + TC - 1) / TC;
    const int64_t tokens_per_split = (stages + splits - 1) / splits * TC;
    const dim3 grid((H + HT - 1) / HT, splits);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    float *ws = static_cast<float *>(workspace);
    if (N <= 32)
        gate_wgrad_kernel<1><<<grid, dim3(256), 0, st>>>(xp, dlogits, T, H, N, tokens_per_split, ws);
    else if (N <= 64)
        gate_wgrad_kernel<2><<<grid, dim3(256), 0, st>>>(xp, dlogits, T, H, N, tokens_per_split, ws);
    else if (N <= 128)
        gate_wgrad_kernel<4><<<grid, dim3(256), 0, st>>>(xp, dlogits, T, H, N, tokens_per_split, ws);
    else
        gate_wgrad_kernel<8><<<grid, dim3(256), 0, st>>>(xp, dlogits, T, H, N, tokens_per_split, ws);
    const unsigned rblocks = static_cast<unsigned>((nh / 4 + 255) / 256);
    if (dweight_dtype == OM_F32)
        gate_wgrad_reduce_kernel<float><<<dim3(rblocks), dim3(256), 0, st>>>(ws, splits, nh, static_cast<float *>(dweight));
    else
        gate_wgrad_reduce_kernel<uint16_t><<<dim3(rblocks), dim3(256), 0, st>>>(ws, splits, nh, static_cast<uint16_t *>(dweight));
    return om_launch_status();
}
