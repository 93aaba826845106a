"""Row movers (K4 / K6 / index_add) through pcl_xpu_customops against the C restatement of the
SYCL kernels.  Bar: bit-exact, except routing_weights_grad (a dot product whose summation order
differs: wavefront tree vs serial) which is held to 2e-3 relative."""
import numpy as np
import pytest
import torch

from util import bits, from_bits, routed_experts

pytestmark = pytest.mark.gpu


def _setup(T, N, K, E, start, end, dtype, oracle_lib, seed=0):
    se = routed_experts(T, N, K, seed=seed + 1)
    idx = oracle_lib.index_construction(se.numpy(), end - start, start, end)
    g = torch.Generator().manual_seed(seed)
    TR = idx["num_routed_tokens"]
    x = torch.randn(T, E, generator=g).to(dtype)
    y = torch.randn(TR, E, generator=g).to(dtype)
    w = torch.rand(T, K, generator=g)
    return se, idx, x, y, w


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,N,K,E,start,end", [(64, 8, 2, 256, 0, 8), (512, 64, 8, 2048, 0, 64),
                                              (256, 32, 4, 136, 8, 24), (128, 8, 2, 100, 0, 8)])
def test_gather_reduce_combine(cuda, oracle_lib, dtype, T, N, K, E, start, end):
    import pcl_xpu_customops as ops
    se, idx, x, y, w = _setup(T, N, K, E, start, end, dtype, oracle_lib)
    TR = idx["num_routed_tokens"]
    d = lambda a: torch.from_numpy(a).to(cuda)
    ii, oi, si, ce = d(idx["input_indices"]), d(idx["output_indices"]), d(idx["selected_experts_indices"]), d(idx["cum_expert_counts_ep"])
    # K4 forward
    out = torch.empty(TR, E, dtype=dtype, device=cuda)
    assert ops.index_gather(x.to(cuda), ii, out) is out
    assert np.array_equal(bits(out), oracle_lib.index_gather(bits(x), idx["input_indices"]))
    # K4 backward
    hg = torch.empty(T, E, dtype=dtype, device=cuda)
    ops.shuffle_sub_matrix_reduce(y.to(cuda), ce, oi, hg)
    assert np.array_equal(bits(hg), oracle_lib.shuffle_sub_matrix_reduce(bits(y), idx["cum_expert_counts_ep"], idx["output_indices"], T))
    # K6 forward: weights in the activation dtype, and fp32 weights with bf16 activations
    for wdt in ([dtype] if dtype == torch.float32 else [torch.bfloat16, torch.float32]):
        ww = w.to(wdt)
        fin = torch.empty(T, E, dtype=dtype, device=cuda)
        ops.reduce_ggemm_output(y.to(cuda), ww.to(cuda), ce, si, oi, fin, False)
        ref = oracle_lib.reduce_ggemm_output(bits(y), bits(ww), idx["cum_expert_counts_ep"], idx["selected_experts_indices"], idx["output_indices"])
        assert np.array_equal(bits(fin), ref)
        # K6 backward
        dout = torch.randn(T, E, generator=torch.Generator().manual_seed(3)).to(dtype)
        dy = torch.empty(TR, E, dtype=dtype, device=cuda)
        dw = torch.zeros(T, K, dtype=wdt, device=cuda)
        ops.reduce_ggemm_output_backward(dout.to(cuda), y.to(cuda), ww.to(cuda), ce, si, ii, oi, dy, dw)
        rdy, rdw = oracle_lib.reduce_ggemm_output_backward(bits(dout), bits(y), bits(ww), idx["selected_experts_indices"], idx["input_indices"], idx["output_indices"])
        assert np.array_equal(bits(dy), rdy)
        a, b = dw.float().cpu(), from_bits(rdw, wdt).float()
        tol = 2e-2 if wdt == torch.bfloat16 else 2e-3
        assert float((a - b).abs().max()) <= tol * float(b.abs().max())
        # not-local entries stay zero
        local = ((se >= start) & (se < end))
        assert float(a[~local].abs().max() if (~local).any() else 0.0) == 0.0
    # skip_weights_scaling
    fin = torch.empty(T, E, dtype=dtype, device=cuda)
    ops.reduce_ggemm_output(y.to(cuda), w.to(dtype).to(cuda), ce, si, oi, fin, True)
    assert np.array_equal(bits(fin), oracle_lib.shuffle_sub_matrix_reduce(bits(y), idx["cum_expert_counts_ep"], idx["output_indices"], T))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_index_add_and_autograd_function(cuda, oracle_lib, dtype):
    from optimus.custom_ops import IndexAddOpFunction
    g = torch.Generator().manual_seed(0)
    C, E, S = 96, 72, 40
    inp = torch.randn(C, E, generator=g).to(dtype)
    base = torch.randn(S, E, generator=g).to(dtype)
    idx = torch.randperm(S, generator=g)[:C % S].tolist() + list(range(S)) + torch.randperm(S, generator=g)[: C - S - C % S].tolist()
    idx = torch.tensor(idx[:C], dtype=torch.int32)
    uniq = torch.randperm(S, generator=g)[:32].to(torch.int32)   # distinct: bit-exact case
    out = base.clone().to(cuda)
    import pcl_xpu_customops as ops
    ops.index_add_op(inp[:32].contiguous().to(cuda), out, uniq.to(cuda))
    ref = bits(base).copy()
    oracle_lib.index_add(bits(inp[:32].contiguous()), ref, uniq.numpy())
    assert np.array_equal(bits(out), ref)
    # duplicates: sums are order-dependent in the last bit; compare in fp32 with tolerance
    out = base.clone().to(cuda)
    ops.index_add_op(inp.to(cuda), out, idx.to(cuda))
    want = base.float().index_add(0, idx.long(), inp.float())
    tol = 1e-5 if dtype == torch.float32 else 6e-2
    assert float((out.float().cpu() - want).abs().max()) <= tol
    # autograd wrapper: gradient wrt expert_output is a gather of grad_output
    eo = inp[:32].contiguous().to(cuda).requires_grad_(True)
    fo = base.clone().to(cuda)
    res = IndexAddOpFunction.apply(eo, fo, uniq.to(cuda))
    gout = torch.randn(S, E, generator=g).to(dtype).to(cuda)
    res.backward(gout)
    assert torch.equal(eo.grad, gout[uniq.long().to(cuda)])


@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                          (torch.float32, torch.float32)])
@pytest.mark.parametrize("T,N,K,E,start,end", [(64, 8, 2, 256, 0, 8), (512, 64, 8, 2048, 0, 64),
                                              (256, 32, 4, 136, 8, 24), (128, 8, 2, 100, 0, 8)])
def test_combine_with_residual_equals_two_steps(cuda, oracle_lib, dtype, wdtype, T, N, K, E, start, end):
    """reduce_ggemm_output_residual = reduce_ggemm_output (already bit-exact against the restatement
    of the SYCL kernel) followed by the tensor addition the callers perform: the same bits, for an
    expert window (tokens without a local expert get residual + 0) and row lengths that are not a
    multiple of the vector width."""
    import pcl_xpu_customops as ops
    se, idx, x, y, w = _setup(T, N, K, E, start, end, dtype, oracle_lib, seed=5)
    d = lambda a: torch.from_numpy(a).to(cuda)
    oi, si, ce = d(idx["output_indices"]), d(idx["selected_experts_indices"]), d(idx["cum_expert_counts_ep"])
    yd, wd, res = y.to(cuda), w.to(wdtype).to(cuda), x.to(cuda)
    two = torch.empty(T, E, dtype=dtype, device=cuda)
    ops.reduce_ggemm_output(yd, wd, ce, si, oi, two, False)
    two = res + two
    one = torch.empty(T, E, dtype=dtype, device=cuda)
    ops.reduce_ggemm_output_residual(yd, wd, ce, si, oi, res, one)
    assert np.array_equal(bits(one), bits(two))
