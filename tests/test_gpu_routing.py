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
