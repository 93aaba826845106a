// Token permutation for the fast MoE block: a stable counting sort of the (token, k) pairs by
// local expert, producing exactly the arrays the reference builds with its two index kernels and
// two cumsums.  Three small launches:
//   count   — every block histograms its chunk of pairs per expert (wave ballots -> LDS);
//   scan    — one block (16 wavefront-wide scans at a time) turns the [block][expert] table into exclusive offsets in
//             (expert-major, block-minor) order = the stable order, and writes cum_token_counts;
//   scatter — every block re-reads its chunk and places each pair at offset + stable rank.
// Ranks come from wavefront ballots (lanes holding the same expert form a mask; rank = popcount of
// the mask below the lane), per-wave running offsets live in LDS: no atomics, so the result is
// deterministic.
// Also: the reference's two index operators with their own [expert][column] table layout, one
// wavefront per column.
#include "common.h"
#include <mutex>

namespace {

constexpr int SORT_THREADS = 256;
constexpr int SORT_WAVES = SORT_THREADS / 64;
constexpr int SORT_ITERS = 8;                                    // 64-pair steps per wavefront
constexpr int SORT_CHUNK = SORT_THREADS * SORT_ITERS;            // pairs per block
constexpr int SORT_MAX_NR = 1024;                                // local experts supported

template <typename TI>
__device__ __forceinline__ int local_key(const TI *selected_experts, int64_t j, int64_t n_pairs,
                                         int start, int end, int NR) {
    if (j >= n_pairs) return NR;
    const long long e = static_cast<long long>(selected_experts[j]);
    return (e >= start && e < end) ? static_cast<int>(e - start) : NR;
}

// Mask of the lanes of this wavefront that hold the same key (keys < 2^nbits).
__device__ __forceinline__ unsigned long long match_key(int key, int nbits) {
    unsigned long long m = ~0ull;
    for (int b = 0; b < nbits; b++) {
        const unsigned long long vote = __ballot((key >> b) & 1);
        m &= ((key >> b) & 1) ? vote : ~vote;
    }
    return m;
}

__device__ __forceinline__ unsigned long long lanemask_lt(int lane) { return (1ull << lane) - 1ull; }

// Per-wave histogram of the wave's SORT_ITERS*64 pairs into wave_hist[wave][0..NR).
template <typename TI>
__device__ __forceinline__ int wave_histogram(const TI *selected_experts, int64_t wave_base,
                                              int64_t n_pairs, int start, int end, int NR, int nbits,
                                              int lane, volatile int *hist) {
    int hits = 0;
    for (int it = 0; it < SORT_ITERS; it++) {
        const int64_t j = wave_base + it * 64 + lane;
        const int key = local_key(selected_experts, j, n_pairs, start, end, NR);
        const unsigned long long m = match_key(key, nbits);
        const bool leader = (__ffsll(static_cast<long long>(m)) - 1) == lane;
        if (leader && key < NR) hist[key] += __popcll(m);
        hits += __popcll(__ballot(key < NR));
        __builtin_amdgcn_wave_barrier();
    }
    return hits;
}

template <typename TI>
__global__ __launch_bounds__(SORT_THREADS) void sort_count_kernel(const TI *__restrict__ selected_experts,
                                                                  int64_t n_pairs, int start, int end,
                                                                  int NR, int nbits,
                                                                  int32_t *__restrict__ block_hist) {
    extern __shared__ int lds[];  // [SORT_WAVES][NR]
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < SORT_WAVES * NR; i += SORT_THREADS) lds[i] = 0;
    __syncthreads();
    const int64_t wave_base = static_cast<int64_t>(blockIdx.x) * SORT_CHUNK + wv * (SORT_ITERS * 64);
    wave_histogram(selected_experts, wave_base, n_pairs, start, end, NR, nbits, lane, lds + wv * NR);
    __syncthreads();
    for (int e = threadIdx.x; e < NR; e += SORT_THREADS) {
        int s = 0;
        for (int w = 0; w < SORT_WAVES; w++) s += lds[w * NR + e];
        block_hist[static_cast<int64_t>(blockIdx.x) * NR + e] = s;
    }
}

// Inclusive prefix sum over the 64 lanes of a wavefront.
__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
    for (int o = 1; o < 64; o <<= 1) {
        const int u = __shfl_up(v, o, 64);
        if (lane >= o) v += u;
    }
    return v;
}

// One block.  block_hist [NB][NR] -> in place: exclusive offset of (expert e, block b) in the
// stable order; hits_base [NB] = pairs kept by blocks before b; cum_token_counts [NR+1].
// Every phase is spread over the 16 wavefronts (lanes over blocks or over experts, wavefront
// scans), so nothing walks the table serially.
__global__ __launch_bounds__(1024) void sort_scan_kernel(int32_t *__restrict__ block_hist,
                                                          int32_t *__restrict__ hits_base, int NB,
                                                          int NR, int32_t *__restrict__ cum_token_counts,
                                                          int32_t *__restrict__ cum_expert_counts_ep,
                                                          int64_t T) {
    __shared__ int totals[SORT_MAX_NR + 1];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    // per-expert exclusive scan over blocks: one wavefront per expert, lanes over blocks
    for (int e = wv; e < NR; e += n_waves) {
        int run = 0;
        for (int b0 = 0; b0 < NB; b0 += 64) {
            const int b = b0 + lane;
            const int c = b < NB ? block_hist[static_cast<int64_t>(b) * NR + e] : 0;
            const int incl = wave_incl_scan(c, lane);
            if (b < NB) block_hist[static_cast<int64_t>(b) * NR + e] = run + incl - c;
            run += __shfl(incl, 63, 64);
        }
        if (lane == 0) totals[e] = run;
    }
    __syncthreads();
    if (wv == 0) {  // exclusive scan of the per-expert totals
        int run = 0;
        for (int e0 = 0; e0 < NR; e0 += 64) {
            const int e = e0 + lane;
            const int c = e < NR ? totals[e] : 0;
            const int incl = wave_incl_scan(c, lane);
            if (e < NR) {
                totals[e] = run + incl - c;
                cum_token_counts[e] = run + incl - c;
            }
            run += __shfl(incl, 63, 64);
        }
        if (lane == 0) {
            totals[NR] = run;
            cum_token_counts[NR] = run;
            cum_expert_counts_ep[T] = run;
        }
    }
    __syncthreads();
    // add the expert's base, and per block sum what its experts hold before it:
    // kept_before(b) = sum_e (off[b][e] - totals[e]) = sum_e of the within-expert offsets
    for (int b = wv; b < NB; b += n_waves) {
        int kept_before = 0;
        for (int e0 = 0; e0 < NR; e0 += 64) {
            const int e = e0 + lane;
            if (e < NR) {
                const int within = block_hist[static_cast<int64_t>(b) * NR + e];
                kept_before += within;
                block_hist[static_cast<int64_t>(b) * NR + e] = within + totals[e];
            }
        }
        kept_before = wave_sum_i(kept_before);
        if (lane == 0) hits_base[b] = kept_before;
    }
}

template <typename TI>
__global__ __launch_bounds__(SORT_THREADS) void sort_scatter_kernel(
    const TI *__restrict__ selected_experts, int64_t n_pairs, int K, int start, int end, int NR,
    int nbits, const int32_t *__restrict__ block_offsets, const int32_t *__restrict__ hits_base,
    int32_t *__restrict__ cum_expert_counts_ep, int32_t *__restrict__ input_indices,
    int32_t *__restrict__ output_indices, int32_t *__restrict__ selected_experts_indices) {
    extern __shared__ int lds[];  // [SORT_WAVES][NR] then [SORT_WAVES] wave hit counts
    int *wave_hits = lds + SORT_WAVES * NR;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < SORT_WAVES * NR; i += SORT_THREADS) lds[i] = 0;
    __syncthreads();
    const int64_t wave_base = static_cast<int64_t>(blockIdx.x) * SORT_CHUNK + wv * (SORT_ITERS * 64);
    const int hits = wave_histogram(selected_experts, wave_base, n_pairs, start, end, NR, nbits, lane,
                                    lds + wv * NR);
    if (lane == 0) wave_hits[wv] = hits;
    __syncthreads();
    // counts -> running offsets: off[w][e] = block offset + counts of the waves before w
    for (int e = threadIdx.x; e < NR; e += SORT_THREADS) {
        int run = block_offsets[static_cast<int64_t>(blockIdx.x) * NR + e];
        for (int w = 0; w < SORT_WAVES; w++) {
            const int c = lds[w * NR + e];
            lds[w * NR + e] = run;
            run += c;
        }
    }
    __syncthreads();
    int oi_base = hits_base[blockIdx.x];
    for (int w = 0; w < wv; w++) oi_base += wave_hits[w];
    volatile int *off = lds + wv * NR;
    // Entries past the number of kept pairs (an expert window keeps fewer than T*K) are given fixed
    // values, so that a caller who sizes its work by T*K instead of reading the count back can tell
    // them apart: output_indices -1 (no row), the other two 0 (a valid token / slot).
    const int total_kept = cum_expert_counts_ep[n_pairs / K];
    for (int it = 0; it < SORT_ITERS; it++) {
        const int64_t j = wave_base + it * 64 + lane;
        if (j < n_pairs && j >= total_kept) {
            output_indices[j] = -1;
            input_indices[j] = 0;
            selected_experts_indices[j] = 0;
        }
        const int key = local_key(selected_experts, j, n_pairs, start, end, NR);
        const unsigned long long m = match_key(key, nbits);
        const unsigned long long kept = __ballot(key < NR);
        const int oi = oi_base + __popcll(kept & lanemask_lt(lane));
        const bool valid = j < n_pairs;
        const int64_t t = valid ? j / K : 0;
        const int k = valid ? static_cast<int>(j - t * K) : 0;
        if (valid && k == 0) cum_expert_counts_ep[t] = oi;
        if (key < NR) {
            const int pos = off[key] + __popcll(m & lanemask_lt(lane));
            __builtin_amdgcn_wave_barrier();
            const bool leader = (__ffsll(static_cast<long long>(m)) - 1) == lane;
            if (leader) off[key] += __popcll(m);
            input_indices[pos] = static_cast<int32_t>(t);
            output_indices[oi] = pos;
            selected_experts_indices[oi] = k;
        } else {
            __builtin_amdgcn_wave_barrier();
        }
        oi_base += __popcll(kept);
        __builtin_amdgcn_wave_barrier();
    }
}

inline int key_bits(int NR) {  // keys 0..NR (NR = "not local")
    int b = 1;
    while ((1 << b) <= NR) b++;
    return b;
}

// ---- the reference's table layout [expert][column] ---------------------------------------------
// The pybind ops keep a table with one column per group of TB = T / TH consecutive tokens
// (partial_token_counts [NR][TH], then its flattened cumsum, then a same-shaped table of running
// increments).  Here one wavefront owns one column: its TB*K (token, k) pairs are walked in
// row-major order 64 at a time, equal experts are matched by ballots (match_key), and the
// column's per-expert running values live in the wavefront's slice of LDS.  Same results as the
// reference's one-work-item-per-column serial loops, entry for entry.
constexpr int COL_WAVES = 4;   // columns per block

template <typename TI>
__global__ __launch_bounds__(COL_WAVES * 64) void column_counts_kernel(
    const TI *__restrict__ selected_experts, int32_t *__restrict__ partial_token_counts,
    int32_t *__restrict__ expert_counts_ep, int start, int end, int NR, int nbits, int K, int64_t TB,
    int64_t TH) {
    extern __shared__ int lds[];   // [COL_WAVES][NR]
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * COL_WAVES + wv;
    if (col >= TH) return;   // whole wavefronts leave; no block-wide barrier below
    volatile int *hist = lds + wv * NR;
    for (int e = lane; e < NR; e += 64) hist[e] = 0;
    __builtin_amdgcn_wave_barrier();
    const int64_t j0 = col * TB * K, j1 = j0 + TB * K;
    for (int64_t base = j0; base < j1; base += 64) {
        const int key = local_key(selected_experts, base + lane, j1, start, end, NR);
        const unsigned long long m = match_key(key, nbits);
        if (key < NR && (__ffsll(static_cast<long long>(m)) - 1) == lane) hist[key] += __popcll(m);
        __builtin_amdgcn_wave_barrier();
    }
    for (int e = lane; e < NR; e += 64) {
        const int c = hist[e];
        if (c) partial_token_counts[static_cast<int64_t>(e) * TH + col] += c;   // the table is updated in place
    }
    // local hits per token: lanes over the column's tokens
    for (int64_t t = col * TB + lane; t < (col + 1) * TB; t += 64) {
        int hits = 0;
        for (int k = 0; k < K; k++) {
            const long long e = static_cast<long long>(selected_experts[t * K + k]);
            hits += (e >= start && e < end) ? 1 : 0;
        }
        expert_counts_ep[t] = hits;
    }
}

template <typename TI>
__global__ __launch_bounds__(COL_WAVES * 64) void column_scatter_kernel(
    const TI *__restrict__ selected_experts, const int32_t *__restrict__ partial_cum_token_counts,
    int32_t *__restrict__ input_increment_buffer, const int32_t *__restrict__ cum_expert_counts_ep,
    int32_t *__restrict__ selected_experts_indices, int32_t *__restrict__ input_indices,
    int32_t *__restrict__ output_indices, int start, int end, int NR, int nbits, int K, int64_t TB,
    int64_t TH) {
    extern __shared__ int lds[];   // [COL_WAVES][NR]: next free position of every expert in this column
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t col = static_cast<int64_t>(blockIdx.x) * COL_WAVES + wv;
    if (col >= TH) return;
    volatile int *off = lds + wv * NR;
    for (int e = lane; e < NR; e += 64) {
        const int64_t cell = static_cast<int64_t>(e) * TH + col;
        off[e] = partial_cum_token_counts[cell] + input_increment_buffer[cell];
    }
    __builtin_amdgcn_wave_barrier();
    const int64_t j0 = col * TB * K, j1 = j0 + TB * K;
    // kept pairs of the token that straddles into the current 64-pair step
    int64_t carry_token = -1;
    int carry_kept = 0;
    for (int64_t base = j0; base < j1; base += 64) {
        const int64_t j = base + lane;
        const bool valid = j < j1;
        const int key = local_key(selected_experts, j, j1, start, end, NR);
        const unsigned long long m = match_key(key, nbits);
        const unsigned long long kept = __ballot(key < NR);
        const int64_t t = valid ? j / K : -2;
        const int k = valid ? static_cast<int>(j - t * K) : 0;
        // lanes of this step that hold earlier pairs of the same token: [first, lane)
        const int64_t first64 = t * K - base;
        const int first = first64 > 0 ? static_cast<int>(first64) : 0;
        const unsigned long long same_before = lanemask_lt(lane) & ~lanemask_lt(first);
        if (key < NR) {
            const int oi = cum_expert_counts_ep[t] + __popcll(kept & same_before) +
                           (t == carry_token ? carry_kept : 0);
            const int pos = off[key] + __popcll(m & lanemask_lt(lane));
            input_indices[pos] = static_cast<int32_t>(t);
            output_indices[oi] = pos;
            selected_experts_indices[oi] = k;
        }
        __builtin_amdgcn_wave_barrier();
        if (key < NR && (__ffsll(static_cast<long long>(m)) - 1) == lane) off[key] += __popcll(m);
        // the step's last token may continue in the next step: hand its kept pairs on
        const int64_t t_last = __shfl(t, 63, 64);
        if (t_last >= 0) {
            const int here = __popcll(kept & __ballot(t == t_last));
            carry_kept = (t_last == carry_token ? carry_kept : 0) + here;
            carry_token = t_last;
        }
        __builtin_amdgcn_wave_barrier();
    }
    for (int e = lane; e < NR; e += 64) {   // leave the increments as the reference's loop leaves them
        const int64_t cell = static_cast<int64_t>(e) * TH + col;
        input_increment_buffer[cell] = off[e] - partial_cum_token_counts[cell];
    }
}

}  // namespace

extern "C" int64_t om_moe_sort_workspace_bytes(int64_t T, int K, int NR) {
    if (T < 0 || K < 1 || NR < 1) return 0;
    const int64_t n_pairs = T * K;
    const int64_t NB = (n_pairs + SORT_CHUNK - 1) / SORT_CHUNK;
    return (NB * NR + NB + 1) * static_cast<int64_t>(sizeof(int32_t));
}

namespace {

// Launches count, scan and scatter with `workspace` holding the [NB][NR] block table and the
// [NB] kept-pair bases.  Arguments are validated by the two entry points below.
int moe_sort_launch(const void *selected_experts, int index_dtype, int64_t T, int K,
                    int expert_start_idx, int expert_end_idx, int32_t *cum_token_counts,
                    int32_t *cum_expert_counts_ep, int32_t *input_indices, int32_t *output_indices,
                    int32_t *selected_experts_indices, int32_t *workspace, hipStream_t st) {
    const int NR = expert_end_idx - expert_start_idx;
    const int64_t n_pairs = T * K;
    const int64_t NB = (n_pairs + SORT_CHUNK - 1) / SORT_CHUNK;
    int32_t *block_hist = workspace;
    int32_t *hits_base = block_hist + NB * NR;
    const int nbits = key_bits(NR);
    const size_t lds_count = static_cast<size_t>(SORT_WAVES) * NR * sizeof(int);
    const size_t lds_scatter = lds_count + SORT_WAVES * sizeof(int);
    if (NB > 0) {
        if (index_dtype == OM_I64)
            sort_count_kernel<int64_t><<<static_cast<unsigned>(NB), SORT_THREADS, lds_count, st>>>(
                static_cast<const int64_t *>(selected_experts), n_pairs, expert_start_idx,
                expert_end_idx, NR, nbits, block_hist);
        else
            sort_count_kernel<int32_t><<<static_cast<unsigned>(NB), SORT_THREADS, lds_count, st>>>(
                static_cast<const int32_t *>(selected_experts), n_pairs, expert_start_idx,
                expert_end_idx, NR, nbits, block_hist);
    }
    sort_scan_kernel<<<1, 1024, 0, st>>>(block_hist, hits_base, static_cast<int>(NB), NR,
                                         cum_token_counts, cum_expert_counts_ep, T);
    if (NB > 0) {
        if (index_dtype == OM_I64)
            sort_scatter_kernel<int64_t><<<static_cast<unsigned>(NB), SORT_THREADS, lds_scatter, st>>>(
                static_cast<const int64_t *>(selected_experts), n_pairs, K, expert_start_idx,
                expert_end_idx, NR, nbits, block_hist, hits_base, cum_expert_counts_ep, input_indices,
                output_indices, selected_experts_indices);
        else
            sort_scatter_kernel<int32_t><<<static_cast<unsigned>(NB), SORT_THREADS, lds_scatter, st>>>(
                static_cast<const int32_t *>(selected_experts), n_pairs, K, expert_start_idx,
                expert_end_idx, NR, nbits, block_hist, hits_base, cum_expert_counts_ep, input_indices,
                output_indices, selected_experts_indices);
    }
    return om_launch_status();
}

int moe_sort_check(const void *selected_experts, int index_dtype, int64_t T, int K,
                   int expert_start_idx, int expert_end_idx, const int32_t *cum_token_counts,
                   const int32_t *cum_expert_counts_ep, const int32_t *input_indices,
                   const int32_t *output_indices, const int32_t *selected_experts_indices) {
    if (index_dtype != OM_I32 && index_dtype != OM_I64) return OM_ERR_DTYPE;
    const int NR = expert_end_idx - expert_start_idx;
    if (T < 0 || K < 1 || NR < 1 || NR > SORT_MAX_NR || expert_start_idx < 0) return OM_ERR_SHAPE;
    if (T * K > 0x7fffffffLL) return OM_ERR_SHAPE;
    if (!cum_token_counts || !cum_expert_counts_ep) return OM_ERR_NULL;
    if (T > 0 && (!selected_experts || !input_indices || !output_indices || !selected_experts_indices))
        return OM_ERR_NULL;
    return OM_OK;
}

}  // namespace

extern "C" int om_moe_sort(const void *selected_experts, int index_dtype, int64_t T, int K,
                           int expert_start_idx, int expert_end_idx, int32_t *cum_token_counts,
                           int32_t *cum_expert_counts_ep, int32_t *input_indices,
                           int32_t *output_indices, int32_t *selected_experts_indices,
                           void *workspace, int64_t workspace_bytes, void *stream) {
    const int rc = moe_sort_check(selected_experts, index_dtype, T, K, expert_start_idx, expert_end_idx,
                                  cum_token_counts, cum_expert_counts_ep, input_indices, output_indices,
                                  selected_experts_indices);
    if (rc != OM_OK) return rc;
    if (workspace_bytes < om_moe_sort_workspace_bytes(T, K, expert_end_idx - expert_start_idx))
        return OM_ERR_WORKSPACE;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 3u)) return OM_ERR_ALIGN;
    return moe_sort_launch(selected_experts, index_dtype, T, K, expert_start_idx, expert_end_idx,
                           cum_token_counts, cum_expert_counts_ep, input_indices, output_indices,
                           selected_experts_indices, static_cast<int32_t *>(workspace), om_stream(stream));
}

// ---- om_moe_sort for callers that cannot allocate ----------------------------------------------
// The block table lives in a file-scope device array instead of a caller's workspace.  The array's
// name is only a host-side handle: its device address is asked from the runtime once per device
// (with that device current) and kept; kernels and everything else in host code use that address.
constexpr int64_t SORT_SCRATCH_BYTES = 4ll << 20;
constexpr int SORT_MAX_DEVICES = 64;

static __device__ __align__(256) int32_t sort_scratch[SORT_SCRATCH_BYTES / sizeof(int32_t)];

namespace {

std::mutex sort_scratch_mutex;
int32_t *sort_scratch_ptr[SORT_MAX_DEVICES] = {};

// Device address of sort_scratch on the current device; nullptr if the runtime refuses.
int32_t *sort_scratch_on_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SORT_MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(sort_scratch_mutex);
    if (!sort_scratch_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(sort_scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return nullptr;
        }
        sort_scratch_ptr[dev] = static_cast<int32_t *>(p);
    }
    return sort_scratch_ptr[dev];
}

}  // namespace

extern "C" int64_t om_moe_sort_static_capacity_bytes(void) { return SORT_SCRATCH_BYTES; }

extern "C" int om_moe_sort_static(const void *selected_experts, int index_dtype, int64_t T, int K,
                                  int expert_start_idx, int expert_end_idx, int32_t *cum_token_counts,
                                  int32_t *cum_expert_counts_ep, int32_t *input_indices,
                                  int32_t *output_indices, int32_t *selected_experts_indices,
                                  void *stream) {
    const int rc = moe_sort_check(selected_experts, index_dtype, T, K, expert_start_idx, expert_end_idx,
                                  cum_token_counts, cum_expert_counts_ep, input_indices, output_indices,
                                  selected_experts_indices);
    if (rc != OM_OK) return rc;
    if (om_moe_sort_workspace_bytes(T, K, expert_end_idx - expert_start_idx) > SORT_SCRATCH_BYTES)
        return OM_ERR_WORKSPACE;
    int32_t *scratch = sort_scratch_on_current_device();
    if (!scratch) return OM_ERR_LAUNCH;
    // count writes every cell of the block table it later reads and scan writes every base, so
    // nothing left in the array by an earlier call needs clearing
    return moe_sort_launch(selected_experts, index_dtype, T, K, expert_start_idx, expert_end_idx,
                           cum_token_counts, cum_expert_counts_ep, input_indices, output_indices,
                           selected_experts_indices, scratch, om_stream(stream));
}

extern "C" int om_compute_partial_token_counts(const void *selected_experts, int index_dtype,
                                               int32_t *partial_token_counts,
                                               int32_t *expert_counts_ep, int expert_start_idx,
                                               int expert_end_idx, int64_t T, int K, int64_t TH,
                                               void *stream) {
    if (index_dtype != OM_I32 && index_dtype != OM_I64) return OM_ERR_DTYPE;
    const int NR = expert_end_idx - expert_start_idx;
    if (T < 0 || K < 1 || TH < 1 || T % TH != 0 || NR < 1 || NR > SORT_MAX_NR) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!selected_experts || !partial_token_counts || !expert_counts_ep) return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = static_cast<unsigned>((TH + COL_WAVES - 1) / COL_WAVES);
    const size_t lds = static_cast<size_t>(COL_WAVES) * NR * sizeof(int);
    const int nbits = key_bits(NR);
    if (index_dtype == OM_I64)
        column_counts_kernel<int64_t><<<nb, COL_WAVES * 64, lds, st>>>(
            static_cast<const int64_t *>(selected_experts), partial_token_counts, expert_counts_ep,
            expert_start_idx, expert_end_idx, NR, nbits, K, T / TH, TH);
    else
        column_counts_kernel<int32_t><<<nb, COL_WAVES * 64, lds, st>>>(
            static_cast<const int32_t *>(selected_experts), partial_token_counts, expert_counts_ep,
            expert_start_idx, expert_end_idx, NR, nbits, K, T / TH, TH);
    return om_launch_status();
}

extern "C" int om_compute_input_and_output_indices(
    const void *selected_experts, int index_dtype, const int32_t *partial_cum_token_counts,
    int32_t *input_increment_buffer, const int32_t *cum_expert_counts_ep,
    int32_t *selected_experts_indices, int32_t *input_indices, int32_t *output_indices,
    int expert_start_idx, int expert_end_idx, int64_t T, int K, int64_t TH, void *stream) {
    if (index_dtype != OM_I32 && index_dtype != OM_I64) return OM_ERR_DTYPE;
    const int NR = expert_end_idx - expert_start_idx;
    if (T < 0 || K < 1 || TH < 1 || T % TH != 0 || NR < 1 || NR > SORT_MAX_NR) return OM_ERR_SHAPE;
    if (T == 0) return OM_OK;
    if (!selected_experts || !partial_cum_token_counts || !input_increment_buffer ||
        !cum_expert_counts_ep || !selected_experts_indices || !input_indices || !output_indices)
        return OM_ERR_NULL;
    hipStream_t st = om_stream(stream);
    const unsigned nb = static_cast<unsigned>((TH + COL_WAVES - 1) / COL_WAVES);
    const size_t lds = static_cast<size_t>(COL_WAVES) * NR * sizeof(int);
    const int nbits = key_bits(NR);
    if (index_dtype == OM_I64)
        column_scatter_kernel<int64_t><<<nb, COL_WAVES * 64, lds, st>>>(
            static_cast<const int64_t *>(selected_experts), partial_cum_token_counts,
            input_increment_buffer, cum_expert_counts_ep, selected_experts_indices, input_indices,
            output_indices, expert_start_idx, expert_end_idx, NR, nbits, K, T / TH, TH);
    else
        column_scatter_kernel<int32_t><<<nb, COL_WAVES * 64, lds, st>>>(
            static_cast<const int32_t *>(selected_experts), partial_cum_token_counts,
            input_increment_buffer, cum_expert_counts_ep, selected_experts_indices, input_indices,
            output_indices, expert_start_idx, expert_end_idx, NR, nbits, K, T / TH, TH);
    return om_launch_status();
}
