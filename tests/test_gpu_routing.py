"""Router parity through the module-level autograd Functions (-> C-ABI om_route_*).

Bar: expert indices bit-exact on fixtures whose top-(K+1) scores are separated by more than 4 fp32
ulp (so a last-ulp difference between two exp() implementations cannot reorder a row); weights
within 1 bf16 ulp / 1e-6 relative in fp32; gradients against autograd of the torch restatement."""
import numpy as np
import pytest
import torch

from oracle import routing as R

pytestmark = pytest.mark.gpu


def _valid_logits(T, N, K, seed, scale=1.0, bias=None):
    while True:
        g = torch.Generator().manual_seed(seed)
        logits = torch.randn(T, N, generator=g) * scale
        if bias is not None:
            logits = logits + bias
        if R.min_topk_gap_ulps(torch.softmax(logits, 1), K) > 4.0:
            return logits
        seed += 1000


@pytest.mark.parametrize("T,N,K,renorm,ldt,wdt", [
    (2048, 8, 2, True, torch.float32, torch.float32),      # C1
    (16384, 64, 8, False, torch.float32, torch.bfloat16),  # C3: fp32 logits
    (512, 64, 8, False, torch.float32, torch.bfloat16),    # C4 shape
    (300, 100, 5, True, torch.float32, torch.float32),     # N not a multiple of 64
    (257, 256, 8, True, torch.float32, torch.float32),
    (64, 384, 6, False, torch.float32, torch.float32),
])
def test_softmax_topk_forward(cuda, T, N, K, renorm, ldt, wdt):
    from optimus.models.common.moe import SoftmaxTopkRouterFunction as F
    logits = _valid_logits(T, N, K, seed=T + N)
    w_ref, e_ref, _ = R.olmoe_router(logits, K, renorm, wdt)
    w, e = F.apply(logits.to(ldt).to(cuda), K, renorm, wdt)
    assert e.dtype == torch.int64 and torch.equal(e.cpu(), e_ref)
    if wdt == torch.bfloat16:
        # at most one bf16 ulp apart
        a = w.cpu().view(torch.int16).int(); b = w_ref.view(torch.int16).int()
        assert int((a - b).abs().max()) <= 1
    else:
        assert float(((w.cpu() - w_ref).abs() / w_ref).max()) <= 2e-6


@pytest.mark.parametrize("seed", list(range(16)))
def test_softmax_topk_random_shapes(cuda, seed):
    """Seeded sweep over expert counts (one to eight experts per lane), top-k up to 64, odd token
    counts, logit scales (sharp and flat distributions), both weight dtypes."""
    from optimus.models.common.moe import SoftmaxTopkRouterFunction as F
    rng = np.random.RandomState(31 + seed)
    N = int(rng.choice([2, 3, 8, 60, 64, 65, 128, 200, 256, 512]))
    K = int(rng.choice([1, 2, min(8, N), min(64, N)]))
    T = int(rng.choice([1, 7, 100, 1023, 5000]))
    renorm = bool(seed % 2)
    wdt = [torch.float32, torch.bfloat16][(seed // 2) % 2]
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, N, generator=g) * float(rng.choice([0.3, 1.0, 4.0]))
    # rows whose top-(K+1) probabilities are more than 4 ulp apart: there a last-ulp difference in
    # exp() cannot change the choice, and the result must be the restatement's
    probs = torch.softmax(logits, 1)
    top = torch.sort(probs, dim=1, descending=True).values[:, :min(K + 1, N)]
    ok = ((top[:, :-1] - top[:, 1:]) > 4 * top[:, :-1] * 2.0 ** -23).all(dim=1) if N > 1 else torch.ones(T, dtype=torch.bool)
    w_ref, e_ref, _ = R.olmoe_router(logits, K, renorm, wdt)
    w, e = F.apply(logits.to(cuda), K, renorm, wdt)
    tag = (T, N, K, renorm, wdt)
    assert int(ok.sum()) >= T // 2, tag
    assert torch.equal(e.cpu()[ok], e_ref[ok]), tag
    if wdt == torch.bfloat16:
        a = w.cpu()[ok].view(torch.int16).int(); b = w_ref[ok].view(torch.int16).int()
        assert int((a - b).abs().max()) <= 1, tag
    else:
        assert float(((w.cpu()[ok] - w_ref[ok]).abs() / w_ref[ok].clamp_min(1e-30)).max()) <= 4e-6, tag
    # every row, tie or not: K distinct experts, none of them worse than an unselected one
    sel = probs.gather(1, e.cpu())
    rest = probs.scatter(1, e.cpu(), -1.0)
    assert bool((sel.min(1).values >= rest.max(1).values * (1 - 1e-6)).all()), tag
    srt = torch.sort(e.cpu(), 1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all()), tag


def test_softmax_topk_bf16_logits_and_ties(cuda):
    """bf16 logits tie often; the rule is (probability desc, expert index asc) = stable sort."""
    from optimus.models.common.moe import SoftmaxTopkRouterFunction as F
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(4096, 64, generator=g).to(torch.bfloat16)
    logits[:64] = 0.0            # all equal: experts 0..K-1 in order
    logits[64:128] = logits[64:128].clamp(max=2.0)
    logits[64:128, 10:20] = 3.0  # ten-way tie above the rest: 10..17
    w, e = F.apply(logits.to(cuda), 8, False, torch.float32)
    e = e.cpu()
    assert torch.equal(e[:64], torch.arange(8).expand(64, 8))
    assert torch.equal(e[64:128], torch.arange(10, 18).expand(64, 8))
    # rows whose fp32 probabilities have no near-ties must match the oracle exactly
    probs = torch.softmax(logits.float(), 1)
    top = torch.sort(probs, dim=1, descending=True).values[:, :9]
    ok = ((top[:, :-1] - top[:, 1:]) > 4 * top[:, :-1] * 2.0 ** -23).all(dim=1)
    _, e_ref, _ = R.olmoe_router(logits, 8, False, torch.float32)
    assert int(ok.sum()) > 1000 and torch.equal(e[ok], e_ref[ok])
    # every row: a valid top-K set (K-th selected prob >= best unselected prob, up to 4 ulp)
    sel = probs.gather(1, e)
    rest = probs.scatter(1, e, -1.0)
    assert bool((sel.min(1).values >= rest.max(1).values * (1 - 1e-6)).all())
    assert bool((torch.sort(e, 1).values[:, 1:] != torch.sort(e, 1).values[:, :-1]).all())


@pytest.mark.parametrize("N,K,renorm,ldt", [(8, 2, True, torch.float32), (64, 8, False, torch.float32),
                                           (64, 8, True, torch.bfloat16), (256, 8, True, torch.float32)])
def test_softmax_topk_backward(cuda, N, K, renorm, ldt):
    from optimus.models.common.moe import SoftmaxTopkRouterFunction as F
    T = 512
    logits = _valid_logits(T, N, K, seed=N).to(ldt)
    g = torch.Generator().manual_seed(1)
    dw = torch.randn(T, K, generator=g)
    x = logits.to(cuda).requires_grad_(True)
    w, e = F.apply(x, K, renorm, torch.float32)
    w.backward(dw.to(cuda))
    xr = logits.float().requires_grad_(True)
    wr, er, _ = R.olmoe_router(xr, K, renorm, torch.float32)
    wr.backward(dw)
    tol = 1e-5 if ldt == torch.float32 else 1e-2
    err = (x.grad.float().cpu() - xr.grad).abs().max() / xr.grad.abs().max()
    assert float(err) <= tol, float(err)


def _dsv3_case(T, N, n_group, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(T, N, generator=g) * 0.5, torch.randn(N, generator=g) * 0.1


@pytest.mark.parametrize("T,N,n_group,topk_group,K,renorm", [
    (8192, 256, 8, 4, 8, True),      # C5
    (512, 16, 4, 2, 2, True),        # tiny brute-force shape
    (512, 64, 8, 3, 6, False),
    (100, 256, 1, 1, 8, True),       # one group = plain top-K
])
def test_sigmoid_group_topk(cuda, T, N, n_group, topk_group, K, renorm):
    from optimus.models.deepseek_v3.modeling_deepseek_v3 import SigmoidGroupTopkRouterFunction as F
    logits, bias = _dsv3_case(T, N, n_group, seed=N + K)
    scores = logits.sigmoid()
    e_ref, choice = R.dsv3_topk_indices(scores, bias, n_group, topk_group, K)
    w_ref = scores.gather(1, e_ref)
    if renorm:
        w_ref = w_ref / (w_ref.sum(-1, keepdim=True) + 1e-20)
    w_ref = w_ref * 2.5
    x = logits.to(cuda).requires_grad_(True)
    e, w = F.apply(x, bias.to(cuda), n_group, topk_group, K, renorm, 2.5)
    # rows where group scores and choice scores are well separated must match exactly
    gs = R._topk_stable((scores + bias).view(T, n_group, -1), 2)[0].sum(-1)
    gtop = torch.sort(gs, dim=1, descending=True).values
    gap_g = (gtop[:, topk_group - 1] - gtop[:, topk_group]) if topk_group < n_group else torch.ones(T)
    ctop = torch.sort(choice, dim=1, descending=True).values[:, :K + 1]
    gap_c = (ctop[:, :-1] - ctop[:, 1:]).min(1).values
    ok = (gap_g > 1e-5) & (gap_c > 1e-5)
    assert int(ok.sum()) > 0.9 * T
    assert torch.equal(e.cpu()[ok], e_ref[ok])          # same order: choice desc
    assert float((w.detach().cpu()[ok] - w_ref[ok]).abs().max()) <= 1e-5
    if renorm:
        assert float((w.detach().sum(1).cpu() - 2.5).abs().max()) <= 1e-5
    # gradient through gather -> renorm -> scale -> sigmoid
    dw = torch.randn(T, K, generator=torch.Generator().manual_seed(2))
    w.backward(dw.to(cuda))
    lr = logits.clone().requires_grad_(True)
    sr = lr.sigmoid()
    wr = sr.gather(1, e.cpu())
    if renorm:
        wr = wr / (wr.sum(-1, keepdim=True) + 1e-20)
    (wr * 2.5).backward(dw)
    assert float((x.grad.cpu() - lr.grad).abs().max()) <= 1e-5 * max(1.0, float(lr.grad.abs().max()))


# ---- gate projection fused with the routing (om_router_gate_logits / om_router_gate_softmax_topk) --
def _gate_inputs(T, H, N, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, H, generator=g) * 0.02).to(torch.bfloat16)
    return x, w


@pytest.mark.parametrize("T,H,N", [(1000, 2048, 64), (64, 512, 8), (33, 1024, 128), (300, 7168, 256),
                                   (4096, 2048, 60), (200, 2304, 8), (77, 192, 60),   # hidden sizes the one-pass kernel does not take
                                   # more than 64 experts: the kernel that shares the weight tile
                                   # through LDS and splits H (odd step counts, padded expert rows,
                                   # a partial last 128-token block, one and several slices)
                                   (8192, 7168, 256), (1000, 1024, 130), (129, 320, 96), (5, 64, 200),
                                   # hidden sizes that are multiples of 8 only: a last step with fewer than 64 columns
                                   (300, 72, 8), (129, 328, 96), (1000, 1000, 130), (5, 8, 200), (2048, 200, 64)])
def test_gate_logits_match_fp32_matmul(cuda, T, H, N):
    """fp32 logits from bf16 operands: the products are exact, only the order of the fp32 sum differs
    from the CPU matmul of the up-cast operands."""
    from optimus.models.common.moe import fp32_logits
    x, w = _gate_inputs(T, H, N, seed=T + N)
    got = fp32_logits(x.to(cuda), w.to(cuda)).cpu()
    ref = x.float() @ w.float().t()
    exact = (x.double() @ w.double().t())
    assert got.dtype == torch.float32 and got.shape == (T, N)
    # both are fp32 sums of the same exact products: compare their distance to the fp64 value
    err_got = float((got.double() - exact).abs().max()); err_ref = float((ref.double() - exact).abs().max())
    assert err_got <= max(4 * err_ref, 2e-6), (err_got, err_ref)


@pytest.mark.parametrize("T,H,N,K,renorm,wdt", [
    (16384, 2048, 64, 8, False, torch.bfloat16),    # C3
    (1000, 2048, 64, 8, True, torch.float32),       # ragged token count
    (512, 1024, 128, 6, True, torch.float32),
    (96, 512, 8, 2, True, torch.bfloat16),
])
def test_gate_softmax_topk_equals_two_step_on_its_own_logits(cuda, T, H, N, K, renorm, wdt):
    """The routing half of the fused kernel is the same code as om_route_softmax_topk: on the logits
    the kernel itself returns, experts and weights must be identical bit for bit, and the experts
    equal the CPU oracle's on rows without near-ties."""
    from optimus.models.common.moe import GateSoftmaxTopkFunction, SoftmaxTopkRouterFunction
    x, w = _gate_inputs(T, H, N, seed=7 * T + N)
    wts, exp, logits, x_out = GateSoftmaxTopkFunction.apply(x.to(cuda), w.to(cuda), K, renorm, wdt)
    assert x_out.data_ptr() != 0 and torch.equal(x_out.cpu(), x)      # the pass-through of the hidden states
    w2, e2 = SoftmaxTopkRouterFunction.apply(logits.contiguous(), K, renorm, wdt)
    assert torch.equal(exp, e2) and torch.equal(wts.view(torch.int16 if wdt == torch.bfloat16 else torch.int32),
                                                w2.view(torch.int16 if wdt == torch.bfloat16 else torch.int32))
    lg = logits.cpu()
    w_ref, e_ref, _ = R.olmoe_router(lg, K, renorm, wdt)
    probs = torch.softmax(lg, 1)
    top = torch.sort(probs, dim=1, descending=True).values[:, :K + 1]
    ok = ((top[:, :-1] - top[:, 1:]) > 4 * top[:, :-1] * 2.0 ** -23).all(dim=1)
    assert int(ok.sum()) >= 0.99 * T and torch.equal(exp.cpu()[ok], e_ref[ok])


def test_gate_softmax_topk_backward(cuda):
    """dx and dW of the fused router against autograd of the fp32 restatement (the gradient of the
    logits is rounded to bf16 before the two GEMMs, as a bf16 router's backward does)."""
    from optimus.models.common.moe import GateSoftmaxTopkFunction
    T, H, N, K = 2048, 1024, 64, 8
    x, w = _gate_inputs(T, H, N, seed=5)
    g = torch.Generator().manual_seed(6)
    dw_out = torch.randn(T, K, generator=g)
    dlogit_out = torch.randn(T, N, generator=g) * 0.1
    xg = x.to(cuda).requires_grad_(True); wg = w.to(cuda).requires_grad_(True)
    dx_other = torch.randn(T, H, generator=g).to(torch.bfloat16)     # a gradient arriving through the pass-through
    wts, exp, logits, x_out = GateSoftmaxTopkFunction.apply(xg, wg, K, True, torch.float32)
    (wts * dw_out.to(cuda)).sum().backward(retain_graph=True)
    gx1, gw1 = xg.grad.clone(), wg.grad.clone()
    xg.grad = None; wg.grad = None
    ((wts * dw_out.to(cuda)).sum() + (logits * dlogit_out.to(cuda)).sum()).backward(retain_graph=True)
    # reference in fp32 on the CPU with the kernel's own expert choice
    xr = x.float().requires_grad_(True); wr = w.float().requires_grad_(True)
    lr = xr @ wr.t()
    pr = torch.softmax(lr, 1).gather(1, exp.cpu())
    pr = pr / pr.sum(1, keepdim=True)
    ((pr * dw_out).sum() + (lr * dlogit_out).sum()).backward()
    rel = lambda a, b: float((a.float().cpu() - b).abs().mean() / b.abs().mean())
    assert rel(xg.grad, xr.grad) < 1e-2 and rel(wg.grad, wr.grad) < 1e-2
    assert not torch.equal(gx1, xg.grad)     # the logits' own gradient takes part
    # a gradient through the pass-through output is added inside the kernel with autograd's two
    # roundings: bf16(float(other) + float(gate dx)) bit for bit
    gate_dx = xg.grad.clone()
    xg.grad = None; wg.grad = None
    ((wts * dw_out.to(cuda)).sum() + (logits * dlogit_out.to(cuda)).sum()
     + (x_out.float() * dx_other.to(cuda).float()).sum()).backward()
    want = (dx_other.to(cuda).float() + gate_dx.float()).to(torch.bfloat16)
    assert torch.equal(xg.grad, want)


@pytest.mark.parametrize("T,H,N,wdt", [(16384, 2048, 64, torch.bfloat16), (1, 128, 32, torch.float32),
                                       (100, 256, 64, torch.float32), (5000, 1024, 128, torch.bfloat16),
                                       (777, 7168, 256, torch.float32), (64, 2048, 64, torch.float32),
                                       # expert counts that are no multiple of 32 or of 4
                                       (300, 256, 8, torch.bfloat16), (1000, 384, 60, torch.float32),
                                       (500, 128, 130, torch.float32), (257, 512, 7, torch.float32),
                                       # hidden sizes that end in a partial 128-column slice
                                       (700, 192, 8, torch.bfloat16), (2048, 320, 64, torch.float32),
                                       (333, 72, 5, torch.float32)])
def test_gate_weight_grad_matches_fp32_matmul(cuda, T, H, N, wdt):
    """om_router_gate_wgrad against the product it replaces: dlogits rounded to bf16, multiplied in
    fp32.  The bf16 x bf16 products are exact in fp32, so only the order of the fp32 sum differs
    (float64 reference; bound = a few fp32 roundings of the absolute sum), plus one final rounding
    for a bf16 weight.  Token counts that are not multiples of the 64-token stage or of the split."""
    from optimus.models.common.moe import _gate_weight_grad
    g = torch.Generator().manual_seed(T + N)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    dl = torch.randn(T, N, generator=g) * 0.3
    w = torch.empty(N, H, dtype=wdt)
    out = _gate_weight_grad(x.to(cuda), w.to(cuda), dl.to(cuda))
    assert out.dtype == wdt and out.shape == (N, H)
    d16 = dl.to(torch.bfloat16).double()
    ref = d16.t() @ x.double()
    bound = 1e-6 * (d16.abs().t() @ x.double().abs()) + 1e-30
    err = (out.double().cpu() - ref).abs()
    if wdt == torch.bfloat16:
        bound = bound + ref.abs() * 2.0 ** -8      # one bf16 rounding
    assert bool((err <= bound).all()), float((err / bound).max())
    # deterministic: same bits on a second run
    out2 = _gate_weight_grad(x.to(cuda), w.to(cuda), dl.to(cuda))
    assert torch.equal(out, out2)


# ---- auxiliary load-balancing loss (om_router_balance_stats / _bwd) ---------------------------------
@pytest.mark.parametrize("L,T,N,K", [(3, 4096, 64, 8), (2, 1000, 100, 5), (1, 77, 256, 8), (4, 512, 8, 2)])
def test_balance_losses_match_the_reference_expressions(cuda, L, T, N, K):
    from optimus.models.common.ral_functions import (layer_level_load_balancing_loss_func,
                                                     load_balancing_loss_func,
                                                     single_input_load_balancing_loss_func)
    layers = tuple(_valid_logits(T, N, K, seed=31 * l + T) for l in range(L))
    dev = tuple(l.to(cuda) for l in layers)
    got = float(load_balancing_loss_func(dev, N, K)); want = float(R.load_balancing_loss(layers, N, K))
    assert abs(got - want) <= 2e-5 * want
    got = float(layer_level_load_balancing_loss_func(dev, N, K))
    want = float(R.layer_level_load_balancing_loss(layers, N, K))
    assert abs(got - want) <= 2e-5 * want
    got = float(single_input_load_balancing_loss_func(dev[0], N, K))
    want = float(R.load_balancing_loss(layers[:1], N, K))
    assert abs(got - want) <= 2e-5 * want
    assert load_balancing_loss_func(None, N, K) == 0 and load_balancing_loss_func(dev[0], N, K) == 0


def test_balance_loss_gradient_and_bf16_logits(cuda):
    from optimus.models.common.ral_functions import load_balancing_loss_func
    L, T, N, K = 2, 2048, 64, 8
    layers = [_valid_logits(T, N, K, seed=77 + l) for l in range(L)]
    ref = [l.clone().requires_grad_(True) for l in layers]
    R.load_balancing_loss(tuple(ref), N, K).backward()
    dev = [l.to(cuda).requires_grad_(True) for l in layers]
    load_balancing_loss_func(tuple(dev), N, K).backward()
    for a, b in zip(dev, ref):
        assert float((a.grad.cpu() - b.grad).abs().max()) <= 1e-5 * float(b.grad.abs().max())
    # bf16 logits: probabilities are kept in fp32 here, rounded to bf16 in the reference
    b16 = tuple(l.to(torch.bfloat16) for l in layers)
    got = float(load_balancing_loss_func(tuple(l.to(cuda) for l in b16), N, K))
    want = float(R.load_balancing_loss(tuple(l.float() for l in b16), N, K))
    assert abs(got - want) <= 1e-3 * want


@pytest.mark.parametrize("T,H,N,with_other", [(16384, 2048, 64, True), (1, 128, 32, False), (100, 264, 60, True),
                                              (5000, 1024, 128, False), (777, 7168, 256, True), (130, 2304, 7, True),
                                              (64, 8, 5, False)])
def test_gate_input_grad_matches_fp32_matmul(cuda, T, H, N, with_other):
    """om_router_gate_dgrad against the product it replaces, mm(bf16(dlogits), W): exact products,
    fp32 sums in another order, one bf16 rounding; with `other` the second rounding of the
    accumulation.  Partial token blocks, partial column blocks, expert counts that need padding."""
    from optimus.models.common.moe import _gate_input_grad
    g = torch.Generator().manual_seed(3 * T + N)
    w = (torch.randn(N, H, generator=g) * 0.05).to(torch.bfloat16)
    dl = torch.randn(T, N, generator=g) * 0.3
    other = torch.randn(T, H, generator=g).to(torch.bfloat16) if with_other else None
    got = _gate_input_grad(w.to(cuda), dl.to(cuda), None if other is None else other.to(cuda))
    assert got.dtype == torch.bfloat16 and got.shape == (T, H)
    d16 = dl.to(torch.bfloat16).double()
    exact = d16 @ w.double()
    bound = 1e-6 * (d16.abs() @ w.double().abs()) + exact.abs() * 2.0 ** -8 + 1e-30     # order of the sum + one rounding
    if other is None:
        err = (got.double().cpu() - exact).abs()
        assert bool((err <= bound).all()), float((err / bound).max())
    else:
        total = other.double() + exact
        err = (got.double().cpu() - total).abs()
        bound = bound + total.abs() * 2.0 ** -8
        assert bool((err <= bound).all()), float((err / bound).max())
        # exactly the two roundings: round the kernel's own product, add, round
        alone = _gate_input_grad(w.to(cuda), dl.to(cuda))
        assert torch.equal(got, (other.to(cuda).float() + alone.float()).to(torch.bfloat16))
    assert torch.equal(got, _gate_input_grad(w.to(cuda), dl.to(cuda), None if other is None else other.to(cuda)))


def test_gate_shapes_without_a_kernel_raise(cuda):
    """No library fallback behind the gate: a bf16 gate whose shape the kernels do not take raises."""
    from optimus._native import NativeLibraryError
    from optimus.models.common.moe import _gate_backward, fp32_logits
    x = torch.zeros(16, 100, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(NativeLibraryError):
        fp32_logits(x, torch.zeros(8, 100, dtype=torch.bfloat16, device=cuda))            # H % 64
    x = torch.zeros(16, 128, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(NativeLibraryError):
        fp32_logits(x, torch.zeros(300, 128, dtype=torch.bfloat16, device=cuda))          # more than 256 experts
    x = torch.zeros(16, 196, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(NativeLibraryError):
        _gate_backward(x, torch.zeros(8, 196, dtype=torch.bfloat16, device=cuda),
                       torch.zeros(16, 8, device=cuda), (False, True))                      # weight gradient: H % 8
    x = torch.zeros(16, 192, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(TypeError):
        fp32_logits(x, torch.zeros(8, 192, dtype=torch.float32, device=cuda))              # mixed dtypes


@pytest.mark.parametrize("L,B,S,N,K,dtype", [(3, 4, 1024, 64, 8, torch.float32), (2, 5, 200, 100, 5, torch.float32),
                                             (1, 1, 77, 256, 8, torch.float32), (2, 2, 48, 16, 2, torch.bfloat16),
                                             (4, 2, 256, 8, 2, torch.float32)])
def test_masked_balance_loss_matches_the_reference_expression(cuda, L, B, S, N, K, dtype):
    """load_balancing_loss_func with an attention mask (modeling_olmoe.py:58-83): value against the
    oracle's restatement of the masked branch, gradient against autograd through it; masked tokens get
    exactly zero gradient; an all-ones mask gives the unmasked loss."""
    from optimus.models.common.ral_functions import load_balancing_loss_func
    T = B * S
    def layer_logits(seed):
        if dtype == torch.float32:
            return _valid_logits(T, N, K, seed=seed)
        while True:    # the ROUNDED logits must order every token's top-(K+1) without ties
            lg = (torch.randn(T, N, generator=torch.Generator().manual_seed(seed)) * 4.0).to(dtype).float()
            if R.min_topk_gap_ulps(torch.softmax(lg, 1), K) > 4.0:
                return lg
            seed += 1000
    layers = tuple(layer_logits(17 * l + T + N) for l in range(L))
    g = torch.Generator().manual_seed(L + N)
    mask = (torch.rand(B, S, generator=g) > 0.3).long()
    mask[0, 0] = 1
    dev = tuple(l.to(dtype).to(cuda).requires_grad_(True) for l in layers)
    got = load_balancing_loss_func(dev, N, K, attention_mask=mask.to(cuda))
    got.backward()
    ref_in = tuple(l.to(dtype).float().requires_grad_(True) for l in layers)
    want = R.load_balancing_loss(ref_in, N, K, attention_mask=mask.float())
    want.backward()
    tol = 2e-5 if dtype == torch.float32 else 2e-3
    assert abs(float(got.detach()) - float(want.detach())) <= tol * float(want.detach())
    keep = mask.reshape(-1).bool()
    for a, b in zip(dev, ref_in):
        ga = a.grad.float().cpu()
        assert float(ga[~keep].abs().max()) == 0.0 if bool((~keep).any()) else True
        err = float((ga - b.grad).abs().max())
        assert err <= (1e-3 if dtype == torch.float32 else 2e-2) * float(b.grad.abs().max()) + 1e-12, err
    ones = load_balancing_loss_func(tuple(d.detach() for d in dev), N, K, attention_mask=torch.ones(B, S, device=cuda))
    plain = load_balancing_loss_func(tuple(d.detach() for d in dev), N, K)
    assert abs(float(ones) - float(plain)) <= 1e-6 * float(plain)


@pytest.mark.parametrize("T,H,N", [(2048, 256, 8), (1, 7, 3), (777, 100, 130), (5000, 2048, 64)])
def test_float32_gate_kernels_match_float64_products(cuda, T, H, N):
    """The float32 module's gate (om_router_gate_logits_f32 and its two backward products) against
    float64 products of the same float32 values: only the order of the float32 sums differs, so the
    bound is a few float32 roundings of the absolute sum (the weight gradient, summed in double,
    one rounding of the result)."""
    from optimus.models.common.moe import GateLogitsF32Function
    g = torch.Generator().manual_seed(T + H + N)
    x = torch.randn(T, H, generator=g)
    w = torch.randn(N, H, generator=g) * 0.1
    dl = torch.randn(T, N, generator=g)
    xd, wd = x.to(cuda).requires_grad_(True), w.to(cuda).requires_grad_(True)
    logits = GateLogitsF32Function.apply(xd, wd)
    logits.backward(dl.to(cuda))
    eps = 2.0 ** -23
    cases = (("logits", logits, x.double() @ w.double().t(), x.double().abs() @ w.double().abs().t(), 8.0),
             ("dx", xd.grad, dl.double() @ w.double(), dl.double().abs() @ w.double().abs(), 8.0),
             ("dw", wd.grad, dl.double().t() @ x.double(), dl.double().abs().t() @ x.double().abs(), 1.0))
    for name, got, ref, absum, k in cases:
        err = (got.detach().double().cpu() - ref).abs()
        bound = k * eps * absum + 1e-30
        assert bool((err <= bound).all()), (name, float((err / bound).max()))
