"""Pins the RMSNorm restatement (oracle/moe_layer.py rmsnorm) with an independent library routine
(torch.nn.functional.rms_norm, fp32), closed forms and invariants."""
import torch

from oracle.moe_layer import rmsnorm


def test_matches_library_rms_norm_in_fp32():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(37, 256, generator=g) * 3
    w = torch.randn(256, generator=g)
    y, h = rmsnorm(x, w, 1e-5)
    ref = torch.nn.functional.rms_norm(x, (256,), weight=w, eps=1e-5)
    assert torch.equal(h, x)
    torch.testing.assert_close(y, ref, rtol=2e-6, atol=1e-7)


def test_closed_form_constant_row_and_roundings():
    E, c = 64, 3.0
    x = torch.full((2, E), c, dtype=torch.bfloat16)
    w = torch.full((E,), 0.3, dtype=torch.bfloat16)
    y, _ = rmsnorm(x, w, 1e-5)
    r = 1.0 / (c * c + 1e-5) ** 0.5
    xn = torch.tensor(c * r).to(torch.bfloat16)                    # first rounding
    want = (w[0].float() * xn.float()).to(torch.bfloat16)          # second rounding
    assert y.dtype == torch.bfloat16 and torch.equal(y, want.expand(2, E))


def test_scale_invariance_and_residual():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 128, generator=g); res = torch.randn(5, 128, generator=g)
    w = torch.ones(128)
    y1, _ = rmsnorm(x, w, 0.0)
    y2, _ = rmsnorm(x * 7.5, w, 0.0)
    torch.testing.assert_close(y1, y2, rtol=1e-5, atol=1e-6)
    assert torch.allclose(y1.pow(2).mean(-1), torch.ones(5), atol=1e-5)
    y3, h3 = rmsnorm(x, w, 1e-5, residual=res)
    y4, _ = rmsnorm(x + res, w, 1e-5)
    assert torch.equal(y3, y4) and torch.equal(h3, x + res)
