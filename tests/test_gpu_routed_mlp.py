"""RoutedMLPFunction: gather, expert MLP and combine in one function, with the routing weight
applied in the gate+up epilogue and the combine's backward folded into the down projection's
backward GEMMs (om_moe_row_weights, om_merged_mlp_gate_up_fwd_weighted, om_sum_ggemm_output,
om_grouped_gemm_wgrad_gathered_out, om_merged_mlp_down_dgrad_weighted, om_moe_row_weights_grad).

The weight commutes with the linear down projection, so the mathematics is that of the reference's
sequence PrepareInputForGroupGemmFunction -> MergedMLP -> GroupGemmOutputReductionFunction
(optimus/models/common/moe.py:217-405); bf16 roundings fall in different places.  The checks:
against a float32 statement of the layer (tolerances of the separate functions' own tests), and
against the separate functions (never further from float32 than they are, by more than a margin).
"""
import pytest
import torch

from util import assert_bf16_parity, max_abs, mean_rel, routed_experts

pytestmark = pytest.mark.gpu


def _case(T, K, N, start, end, I, H, skew, cuda, weights_dtype=torch.float32, seed=0):
    from optimus.models.common.moe import build_token_permutation
    G = end - start
    g = torch.Generator().manual_seed(T + I + seed)
    se = routed_experts(T, N, K, seed=T + K + seed, skew=skew).to(cuda)
    cum, cum_ep, ii, oi, sel = build_token_permutation(se, start, end)
    rows = int(cum[-1].item())
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    rw = torch.rand(T, K, generator=g) + 0.05
    rw = (rw / rw.sum(-1, keepdim=True)).to(weights_dtype)
    ws = [(torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16),
          (torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16),
          (torch.randn(G, H, I, generator=g) * 0.05).to(torch.bfloat16)]
    dout = torch.randn(T, H, generator=g).to(torch.bfloat16)
    res = torch.randn(T, H, generator=g).to(torch.bfloat16)
    return dict(se=se, cum=cum, cum_ep=cum_ep, ii=ii[:rows], oi=oi[:rows], sel=sel[:rows], rows=rows, x=x,
                rw=rw, ws=ws, dout=dout, res=res, start=start, end=end)


def _run(c, cuda, routed, residual=False):
    from optimus.models.common.moe import (GatheredMergedMLPFunction, GroupGemmOutputReductionFunction,
                                           GroupGemmOutputReductionResidualFunction, RoutedMLPFunction)
    x = c["x"].to(cuda).requires_grad_(True)
    rw = c["rw"].to(cuda).requires_grad_(True)
    ws = [w.to(cuda).requires_grad_(True) for w in c["ws"]]
    res = c["res"].to(cuda).requires_grad_(True) if residual else None
    if routed:
        out = RoutedMLPFunction.apply(x, rw, c["ii"], c["cum_ep"], c["oi"], c["sel"], c["cum"], res, True, *ws)
    else:
        y = GatheredMergedMLPFunction.apply(x, c["ii"], c["cum_ep"], c["oi"], *ws, c["cum"])
        if residual:
            out = GroupGemmOutputReductionResidualFunction.apply(y, rw, c["cum_ep"], c["sel"], c["ii"],
                                                                 c["oi"], res)
        else:
            out = GroupGemmOutputReductionFunction.apply(y, rw, c["cum_ep"], c["sel"], c["ii"], c["oi"])
    out.backward(c["dout"].to(cuda))
    grads = [x.grad, rw.grad] + [w.grad for w in ws] + ([res.grad] if residual else [])
    return [out.detach().float().cpu()] + [t.float().cpu() for t in grads]


def _reference(c, residual=False):
    """float32 on the CPU, token by token over the experts of the window."""
    # clones: .float() of a float32 tensor is the tensor itself
    x = c["x"].detach().clone().float().requires_grad_(True)
    rw = c["rw"].detach().clone().float().requires_grad_(True)
    ws = [w.detach().clone().float().requires_grad_(True) for w in c["ws"]]
    res = c["res"].detach().clone().float().requires_grad_(True) if residual else None
    se = c["se"].cpu()
    out = torch.zeros_like(x)
    if residual:
        out = out + res
    for e in range(c["start"], c["end"]):
        tok, slot = torch.nonzero(se == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        xe = x[tok]
        ye = (torch.nn.functional.silu(xe @ ws[0][e - c["start"]].t()) * (xe @ ws[1][e - c["start"]].t())) \
            @ ws[2][e - c["start"]].t()
        out = out.index_add(0, tok, ye * rw[tok, slot].unsqueeze(1))
    out.backward(c["dout"].float())
    grads = [x.grad, rw.grad] + [w.grad for w in ws] + ([res.grad] if residual else [])
    return [out.detach()] + grads


# (excess over one ideal bf16 rounding, cap); measured: out 1.0-2.0 x, gradients 1.55-2.7 x
ROUTED_BARS = {"out": (2.3, 3.2e-3), "grad": (3.1, 4.4e-3)}
NAMES = ("out", "dx", "d_routing_weights", "dw_gate", "dw_up", "dw_down", "d_residual")


@pytest.mark.parametrize("T,K,N,start,end,I,H,skew,wdt", [
    (2048, 8, 64, 0, 64, 512, 512, 0.0, torch.float32),     # 256x256 tiles
    (512, 2, 8, 0, 8, 128, 384, 0.0, torch.bfloat16),       # 128x128 tiles, bf16 routing weights
    (1500, 4, 16, 4, 12, 256, 256, 1.5, torch.float32),     # expert window: some pairs are not routed
    (70, 8, 64, 0, 64, 128, 128, 3.0, torch.float32),       # most experts empty, a few rows each
    (512, 8, 64, 0, 64, 1024, 2048, 1.2, torch.bfloat16),   # the skewed small batch: a few rows per expert
    (300, 4, 32, 8, 24, 256, 512, 2.0, torch.float32),      # the same with an expert window
])
@pytest.mark.parametrize("residual", [False, True])
def test_routed_mlp_against_float32_and_separate_functions(cuda, T, K, N, start, end, I, H, skew, wdt, residual):
    c = _case(T, K, N, start, end, I, H, skew, cuda, weights_dtype=wdt)
    ref = _reference(c, residual)
    sep = _run(c, cuda, routed=False, residual=residual)
    fus = _run(c, cuda, routed=True, residual=residual)
    assert len(ref) == len(sep) == len(fus) == (7 if residual else 6)
    for name, r, s, f in zip(NAMES, ref, sep, fus):
        assert bool(torch.isfinite(f).all()), name
        scale = max(1.0, float(r.abs().max()))
        e_sep = mean_rel(s, r)
        # the same bars as the separate functions' tests (excess over one ideal bf16 rounding) ...
        e_fus = mean_rel(f, r)
        if name != "d_residual":
            assert_bf16_parity(f, r, *ROUTED_BARS["out" if name == "out" else "grad"],
                               tag=f"routed_mlp[{T},{K},{N},{I},{H},{residual}] {name}")
        assert max_abs(f, r) <= 3e-2 * scale, (name, max_abs(f, r), scale)
        # ... and no worse than the separate functions by more than a margin
        assert e_fus <= 1.25 * e_sep + 5e-4, (name, e_fus, e_sep)
    if residual:
        assert torch.equal(fus[6], c["dout"].float())   # the gradient passes to the residual unchanged
    # pairs outside the expert window get exactly zero
    routed = (c["se"].cpu() >= start) & (c["se"].cpu() < end)
    assert float(fus[2][~routed].abs().sum()) == 0.0


def test_routed_mlp_full_size_against_separate_functions(cuda):
    """OLMoE-1B-7B layer shape (16384 tokens, top-8 of 64, H 2048, I 1024): the two forms agree to
    bf16 accuracy in the output and every gradient."""
    c = _case(16384, 8, 64, 0, 64, 1024, 2048, 0.0, cuda)
    sep = _run(c, cuda, routed=False)
    fus = _run(c, cuda, routed=True)
    for name, s, f in zip(NAMES, sep, fus):
        assert bool(torch.isfinite(f).all()), name
        assert mean_rel(f, s) <= 8e-3, (name, mean_rel(f, s))
        assert max_abs(f, s) <= 4e-2 * max(1.0, float(s.abs().max())), name


def test_routed_mlp_is_deterministic(cuda):
    c = _case(1024, 4, 16, 0, 16, 256, 256, 0.5, cuda)
    a = _run(c, cuda, routed=True)
    b = _run(c, cuda, routed=True)
    for name, p, q in zip(NAMES, a, b):
        assert torch.equal(p, q), name


def test_routed_mlp_unit_weights_reduce_to_the_unweighted_functions(cuda):
    """With every routing weight equal to 1 the weighted epilogues multiply by 1.0 exactly: h, the
    experts' output and the sum are then the bits of the separate functions, and so are the
    gradients that do not pass through the weights' own gradient."""
    c = _case(1024, 2, 8, 0, 8, 256, 256, 0.0, cuda)
    c["rw"] = torch.ones_like(c["rw"])
    sep = _run(c, cuda, routed=False)
    fus = _run(c, cuda, routed=True)
    for i in (0, 1, 3, 4, 5):
        assert torch.equal(sep[i], fus[i]), NAMES[i]
    assert mean_rel(fus[2], sep[2]) <= 6e-3


@pytest.mark.parametrize("residual", [False, True])
def test_routed_mlp_with_no_routed_rows(cuda, residual):
    from optimus.models.common.moe import RoutedMLPFunction, build_token_permutation
    T, K, H, I, G = 64, 2, 128, 128, 2
    se = torch.zeros(T, K, dtype=torch.int64, device=cuda)
    se[:, 1] = 1
    cum, cum_ep, ii, oi, sel = build_token_permutation(se, 4, 6)   # window [4, 6): nothing routed
    assert int(cum[-1].item()) == 0
    x = torch.randn(T, H, device=cuda).to(torch.bfloat16).requires_grad_(True)
    rw = torch.rand(T, K, device=cuda).requires_grad_(True)
    res = torch.randn(T, H, device=cuda).to(torch.bfloat16).requires_grad_(True) if residual else None
    ws = [torch.randn(G, I, H, device=cuda).to(torch.bfloat16).requires_grad_(True),
          torch.randn(G, I, H, device=cuda).to(torch.bfloat16).requires_grad_(True),
          torch.randn(G, H, I, device=cuda).to(torch.bfloat16).requires_grad_(True)]
    out = RoutedMLPFunction.apply(x, rw, ii[:0], cum_ep, oi[:0], sel[:0], cum, res, True, *ws)
    assert out.shape == (T, H)
    if residual:
        assert torch.equal(out, res.detach())
    else:
        assert float(out.detach().abs().max()) == 0.0
    out.sum().backward()
    assert float(x.grad.abs().max()) == 0.0 and float(rw.grad.abs().max()) == 0.0
    for w in ws:
        assert float(w.grad.abs().max()) == 0.0


@pytest.mark.parametrize("merged", [True, False])
def test_block_switch_for_routing_weight_fusion(cuda, merged):
    """The OLMoE block with the fusion on (default) and off: both within the layer tolerance of
    each other in the output and every gradient, including the gate's (which receives the routing
    weights' gradient)."""
    import synthetic_configs as sc
    from test_gpu_moe_layer import _olmoe_block
    inp = sc.moe_inputs("C4")
    c = inp["cfg"]
    res = []
    for fuse in (True, False):
        blk = _olmoe_block(inp, cuda, merged=merged)
        assert blk.fuse_routing_weights is True
        blk.fuse_routing_weights = fuse
        xi = inp["x"].to(cuda).view(1, c["T"], c["H"]).requires_grad_(True)
        o, _ = blk(xi)
        o.backward(inp["dout"].to(cuda).view_as(o))
        res.append([o, xi.grad] + [p.grad for p in blk.parameters()])
    assert len(res[0]) == len(res[1]) >= 5
    differs = False
    for a, b in zip(*res):
        assert mean_rel(a.float().cpu(), b.float().cpu()) <= 1e-2
        differs = differs or not torch.equal(a, b)
    assert differs   # the switch really selects another code path


@pytest.mark.parametrize("seed", list(range(12)))
def test_routed_mlp_random_shapes(cuda, seed):
    """Seeded sweep over token counts, top-k, expert windows and sizes.  With unit routing weights
    the folded form must give the separate functions' bits (this pins the two gathered backward
    GEMMs and the row bookkeeping); with random weights it must stay within bf16 accuracy of them
    and give exact zeros for pairs outside the expert window."""
    import numpy as np
    rng = np.random.RandomState(4321 + seed)
    N = int(rng.choice([4, 8, 16, 64]))
    K = int(rng.choice([1, 2, min(4, N)]))
    T = int(rng.choice([5, 64, 300, 1024, 5000]))
    H = int(rng.choice([128, 256, 384, 512]))
    I = int(rng.choice([128, 256, 384]))
    start = int(rng.choice([0, N // 4]))
    end = int(rng.choice([N, max(start + 1, N - N // 4)]))
    wdt = [torch.float32, torch.bfloat16][seed % 2]
    c = _case(T, K, N, start, end, I, H, float(rng.choice([0.0, 1.0])), cuda, weights_dtype=wdt, seed=seed)
    tag = (T, K, N, start, end, I, H, c["rows"])
    residual = bool(seed % 3 == 0)
    sep = _run(c, cuda, routed=False, residual=residual)
    fus = _run(c, cuda, routed=True, residual=residual)
    routed = (c["se"].cpu() >= start) & (c["se"].cpu() < end)
    assert float(fus[2][~routed].abs().sum()) == 0.0, tag
    for name, s, f in zip(NAMES, sep, fus):
        assert bool(torch.isfinite(f).all()), (name, tag)
        # a routing weight's gradient is one dot product with cancellation: a relative measure over
        # a handful of them says nothing
        if name == "d_routing_weights" and c["rows"] < 64:
            continue
        if float(s.abs().mean()) > 0:
            assert mean_rel(f, s) <= 1.5e-2, (name, tag, mean_rel(f, s))
    c["rw"] = torch.ones_like(c["rw"])
    sep1 = _run(c, cuda, routed=False, residual=residual)
    fus1 = _run(c, cuda, routed=True, residual=residual)
    for i in (0, 1, 3, 4, 5):
        assert torch.equal(sep1[i], fus1[i]), (NAMES[i], tag)
