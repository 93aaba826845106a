"""Token-permutation parity: om_moe_sort (and the reference-shaped K1/K3 ops) against the C
restatement of the SYCL index kernels.  Bar: bit-exact."""
import numpy as np
import pytest
import torch

from util import routed_experts

pytestmark = pytest.mark.gpu

CASES = [
    # T, N, K, start, end, skew, dtype
    (8, 8, 2, 0, 8, 0.0, torch.int64),
    (64, 8, 2, 0, 8, 0.0, torch.int32),
    (2048, 8, 2, 0, 8, 0.0, torch.int64),          # C1
    (512, 64, 8, 0, 64, 1.2, torch.int64),         # C4: skewed, empty experts likely
    (16384, 64, 8, 0, 64, 0.0, torch.int64),       # C3
    (8192, 256, 8, 64, 96, 0.0, torch.int64),      # C5: window of 32 of 256
    (1000 * 8, 16, 4, 4, 12, 2.0, torch.int64),    # window + skew
    (24, 64, 8, 0, 64, 3.0, torch.int64),          # tiny T, most experts empty
    (4104, 300, 3, 0, 300, 0.0, torch.int64),      # > 256 experts, pairs not a multiple of 64
    (40000, 128, 8, 0, 128, 0.5, torch.int64),     # 157 count blocks: the scan walks them 64 at a time
]


def _gpu_sort(se, start, end, cuda):
    from optimus.models.common.moe import build_token_permutation
    out = build_token_permutation(se.to(cuda), start, end)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in out]


@pytest.mark.parametrize("T,N,K,start,end,skew,dt", CASES)
def test_moe_sort_bit_exact(cuda, oracle_lib, T, N, K, start, end, skew, dt):
    se = routed_experts(T, N, K, seed=T + N + K, skew=skew)
    ref = oracle_lib.index_construction(se.numpy(), end - start, start, end)
    cum, cum_ep, ii, oi, si = _gpu_sort(se.to(dt), start, end, cuda)
    TR = ref["num_routed_tokens"]
    assert np.array_equal(cum, ref["cum_token_counts"])
    assert np.array_equal(cum_ep, ref["cum_expert_counts_ep"])
    assert np.array_equal(ii[:TR], ref["input_indices"])
    assert np.array_equal(oi[:TR], ref["output_indices"])
    assert np.array_equal(si[:TR], ref["selected_experts_indices"])


def test_no_token_routed_locally(cuda, oracle_lib):
    se = torch.zeros(64, 2, dtype=torch.int64)
    se[:, 1] = 1
    cum, cum_ep, ii, oi, si = _gpu_sort(se, 4, 8, cuda)
    assert cum.tolist() == [0] * 5 and cum_ep.max() == 0


def test_permutation_invariants_full_size(cuda):
    """C3 size: output_indices is a permutation, input_indices inverts it, experts non-decreasing."""
    T, N, K = 16384, 64, 8
    se = routed_experts(T, N, K, seed=3)
    cum, cum_ep, ii, oi, si = _gpu_sort(se, 0, N, cuda)
    assert cum[-1] == T * K and np.array_equal(np.sort(oi), np.arange(T * K))
    j = np.arange(T * K)
    assert np.array_equal(ii[oi], j // K) and np.array_equal(si, j % K)
    e_sorted = se.numpy().reshape(-1)[np.argsort(oi, kind="stable")]
    assert np.all(np.diff(e_sorted) >= 0)
    assert np.array_equal(np.bincount(se.numpy().reshape(-1), minlength=N), np.diff(cum))


@pytest.mark.parametrize("T,N,K,start,end,TB", [
    (2048, 8, 2, 0, 8, 8), (4096, 64, 8, 16, 48, 8),     # the reference's blocking: 8 tokens per column
    (1536, 16, 3, 0, 16, 32),      # 96 pairs per column: two 64-pair steps, a token straddles them
    (640, 300, 5, 20, 290, 64),    # 320 pairs per column, five steps, more than 256 local experts
    (77, 8, 2, 2, 6, 1),           # one token per column
    (512, 64, 8, 0, 64, 512),      # a single column holds every token
])
def test_reference_shaped_index_ops(cuda, oracle_lib, T, N, K, start, end, TB):
    """pcl_xpu_customops.compute_partial_token_counts / compute_input_and_output_indices with the
    reference's own call sequence (moe.py:492-554), torch.cumsum as K2; the table has one column per
    TB consecutive tokens (the reference fixes TB = 8, the operators take any T / TH)."""
    import pcl_xpu_customops as ops
    se = routed_experts(T, N, K, seed=11, skew=0.7).to(cuda)
    NR, TH = end - start, T // TB
    ref = oracle_lib.index_construction(se.cpu().numpy(), NR, start, end, tokens_per_thread=TB)
    i32 = dict(dtype=torch.int32, device=cuda)
    partial = torch.zeros((NR, TH), **i32)
    partial_cum = torch.zeros(NR * TH + 1, **i32)
    counts_ep = torch.zeros(T, **i32)
    cum_ep = torch.zeros(T + 1, **i32)
    incr = torch.zeros((NR, TH), **i32)
    ret = ops.compute_partial_token_counts(se, partial, counts_ep, start, end)
    assert ret is partial
    torch.cumsum(partial.flatten(), dim=0, out=partial_cum[1:])
    torch.cumsum(counts_ep, dim=0, out=cum_ep[1:])
    TR = int(partial_cum[-1].item())
    si = torch.empty(TR, **i32); ii = torch.empty(TR, **i32); oi = torch.empty(TR, **i32)
    ops.compute_input_and_output_indices(se, partial_cum, incr, cum_ep, si, ii, oi, start, end)
    torch.cuda.synchronize()
    assert np.array_equal(partial.cpu().numpy(), ref["partial_token_counts"])
    assert np.array_equal(counts_ep.cpu().numpy(), ref["expert_counts_ep"])
    assert np.array_equal(ii.cpu().numpy(), ref["input_indices"])
    assert np.array_equal(oi.cpu().numpy(), ref["output_indices"])
    assert np.array_equal(si.cpu().numpy(), ref["selected_experts_indices"])
    # the increments end as the per-column counts, like the reference's read-modify-write leaves them
    assert np.array_equal(incr.cpu().numpy(), ref["partial_token_counts"])


@pytest.mark.parametrize("seed", list(range(16)))
def test_moe_sort_random_shapes(cuda, oracle_lib, seed):
    """Seeded sweep over token counts (one to a few hundred count blocks), expert counts up to the
    kernel's limit, top-k and expert windows, bit-exact against the restatement of the reference's
    K1 -> cumsum -> K3."""
    rng = np.random.RandomState(7 + seed)
    N = int(rng.choice([2, 8, 60, 64, 65, 128, 256, 700, 1024]))
    K = int(rng.choice([1, 2, min(8, N)]))
    T = int(rng.choice([1, 9, 255, 257, 4096, 30000, 70000]))
    start = int(rng.choice([0, N // 3]))
    end = int(rng.choice([N, max(start + 1, N - N // 5)]))
    dt = [torch.int64, torch.int32][seed % 2]
    se = routed_experts(T, N, K, seed=seed, skew=float(rng.choice([0.0, 0.8, 2.5])))
    # the restatement keeps the reference's tokens-per-thread blocking (T a multiple of it); its
    # result does not depend on the blocking (tests/test_oracle_moe.py), so 1 serves any T
    ref = oracle_lib.index_construction(se.numpy(), end - start, start, end,
                                        tokens_per_thread=8 if T % 8 == 0 else 1)
    cum, cum_ep, ii, oi, si = _gpu_sort(se.to(dt), start, end, cuda)
    TR = ref["num_routed_tokens"]
    tag = (T, N, K, start, end)
    assert np.array_equal(cum, ref["cum_token_counts"]), tag
    assert np.array_equal(cum_ep, ref["cum_expert_counts_ep"]), tag
    assert np.array_equal(ii[:TR], ref["input_indices"]), tag
    assert np.array_equal(oi[:TR], ref["output_indices"]), tag
    assert np.array_equal(si[:TR], ref["selected_experts_indices"]), tag
