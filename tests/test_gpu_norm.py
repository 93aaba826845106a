"""RMSNorm kernels (om_rmsnorm_fwd / om_rmsnorm_bwd) through the reference-shaped modules.

Bars: fp32 within 2e-6 relative of the CPU restatement; bf16 identical except where the last ulp of
rsqrt / of the fp32 sum of squares moves the first of the two bf16 roundings (the product with a
weight above 1 can then land two bf16 steps away; under 1 % of the elements differ at all); the residual sum h bit-exact; gradients against autograd of the
restatement run in fp32."""
import pytest
import torch

from oracle.moe_layer import rmsnorm

pytestmark = pytest.mark.gpu


def _inputs(rows, E, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, E, generator=g) * 2).to(dtype)
    res = torch.randn(rows, E, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(E, generator=g)).to(dtype)
    return x, res, w


def _close_bf16(a, b, frac=0.01):
    ai = a.view(torch.int16).int(); bi = b.view(torch.int16).int()
    d = (ai - bi).abs()
    assert int(d.max()) <= 2 and float((d > 0).float().mean()) <= frac, (int(d.max()), float((d > 0).float().mean()))


@pytest.mark.parametrize("rows,E", [(1000, 2048), (64, 7168), (5, 256), (300, 4104)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fused", [False, True])
def test_forward(cuda, rows, E, dtype, fused):
    from optimus.models.olmoe.modeling_olmoe import OlmoeParallelRMSNorm
    x, res, w = _inputs(rows, E, dtype, seed=rows + E)
    m = OlmoeParallelRMSNorm(E, eps=1e-5).to(dtype).to(cuda)
    with torch.no_grad():
        m.weight.copy_(w)
    if fused:
        y, h = m.forward_with_residual(x.to(cuda), res.to(cuda))
        y_ref, h_ref = rmsnorm(x, w, 1e-5, residual=res)
        assert torch.equal(h.cpu(), h_ref)
    else:
        y = m(x.to(cuda))
        y_ref, _ = rmsnorm(x, w, 1e-5)
    if dtype == torch.float32:
        torch.testing.assert_close(y.cpu(), y_ref, rtol=2e-6, atol=1e-7)
    else:
        _close_bf16(y.cpu(), y_ref)


@pytest.mark.parametrize("rows,E,dtype", [(777, 2048, torch.bfloat16), (130, 7168, torch.bfloat16),
                                          (257, 512, torch.float32)])
def test_backward(cuda, rows, E, dtype):
    from optimus.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3ParallelRMSNorm
    x, res, w = _inputs(rows, E, dtype, seed=3 * rows + E)
    g = torch.Generator().manual_seed(9)
    gy = torch.randn(rows, E, generator=g).to(dtype); gh = torch.randn(rows, E, generator=g).to(dtype)
    m = DeepseekV3ParallelRMSNorm(E, eps=1e-6).to(dtype).to(cuda)
    with torch.no_grad():
        m.weight.copy_(w)
    xg = x.to(cuda).requires_grad_(True); rg = res.to(cuda).requires_grad_(True)
    y, h = m.forward_with_residual(xg, rg)
    (y.float() * gy.to(cuda).float()).sum().add((h.float() * gh.to(cuda).float()).sum()).backward()
    xr = x.float().requires_grad_(True); rr = res.float().requires_grad_(True); wr = w.float().requires_grad_(True)
    yr, hr = rmsnorm(xr, wr, 1e-6, residual=rr)
    ((yr * gy.float()).sum() + (hr * gh.float()).sum()).backward()
    rel = lambda a, b: float((a.float().cpu() - b).abs().mean() / b.abs().mean())
    tol = 2e-6 if dtype == torch.float32 else 6e-3
    assert rel(xg.grad, xr.grad) <= tol and rel(rg.grad, rr.grad) <= tol
    assert rel(m.weight.grad, wr.grad) <= (1e-5 if dtype == torch.float32 else 6e-3)
    assert torch.equal(xg.grad, rg.grad)
