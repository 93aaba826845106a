"""Pins the gradient-norm / clip restatement (oracle/adamw_oracle.c orc_grad_norm_clip_*,
orc_scale_grads_*) against the library calls the reference itself makes on the gradient views
(torch.nn.utils.get_total_norm, clip_grads_with_norm_; optimus/optimizers.py:136-160), run on
CPU.  Several seeds and ragged parameter sizes, so that dropping any one of the roundings to the
gradient dtype (per-parameter norm, total, the sum with 1e-6, the reciprocal, the product) or
evaluating max_norm/x as a division shows up as a different coefficient or different gradients."""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle.adamw import grad_norm_and_clip_torch
from util import bits, from_bits

SIZES = [1, 7, 64, 1000, 4096, 33, 129, 8191, 2, 515, 70000, 12, 3001]


def _flat(dtype, seed, scale):
    g = torch.Generator().manual_seed(seed)
    n = sum(SIZES)
    return (torch.randn(n, generator=g) * scale).to(dtype)


def _views(flat):
    out, pos = [], 0
    for s in SIZES:
        out.append(flat[pos:pos + s])
        pos += s
    return out


def _starts():
    return np.cumsum([0] + SIZES[:-1])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("scale", [1e-3, 3e-2, 1.0])      # total norm below, near and above 1
def test_norm_coef_and_scaled_grads_match_the_library_calls(dtype, seed, scale):
    flat = _flat(dtype, seed, scale)
    ref = flat.clone()
    total_ref = grad_norm_and_clip_torch(_views(ref), clip=True)
    assert total_ref.dtype == dtype

    arr = bits(flat).copy()
    seg, total, coef = clib.grad_norm_clip(arr, _starts(), SIZES, 1.0)
    if dtype == torch.bfloat16:
        assert total == float(total_ref)                   # both are bf16 values
        per = [float(torch.linalg.vector_norm(v)) for v in _views(flat)]
        assert list(seg) == per
    else:
        assert abs(total - float(total_ref)) <= 1e-6 * float(total_ref)
    clib.scale_grads(arr, coef)
    got = from_bits(arr, dtype)
    if dtype == torch.bfloat16:
        assert torch.equal(got, ref)
    else:
        # fp32: the summation order leaves the last bits of the norm, hence of the coefficient, open
        torch.testing.assert_close(got, ref, rtol=2e-6, atol=0)
    if float(total_ref) <= 0.99:
        assert coef == 1.0 and torch.equal(got, flat)      # clamp: nothing is scaled
    elif float(total_ref) > 1.01:
        assert coef < 1.0


def test_no_clip_leaves_gradients_alone():
    flat = _flat(torch.bfloat16, 0, 1.0)
    ref = flat.clone()
    total = grad_norm_and_clip_torch(_views(ref), clip=False)
    assert torch.equal(ref, flat) and float(total) > 1.0


def test_coefficient_is_not_a_plain_fp32_division():
    """The bf16 roundings matter: for a bf16 total norm the coefficient is itself a bf16 value and
    differs from 1/(total+1e-6) taken in fp32 for most totals."""
    flat = _flat(torch.bfloat16, 3, 1.0)
    _, total, coef = clib.grad_norm_clip(bits(flat).copy(), _starts(), SIZES, 1.0)
    as_bf16 = float(torch.tensor(coef).to(torch.bfloat16))
    assert coef == as_bf16
    assert coef != np.float32(1.0) / np.float32(total + 1e-6)


def test_closed_form_single_parameter():
    """One parameter holding k copies of a: norm = |a|·sqrt(k) exactly representable."""
    a, k = 0.5, 64                                         # norm = 4.0
    arr = np.full(k, a, dtype=np.float32)
    seg, total, coef = clib.grad_norm_clip(arr, [0], [k], 1.0)
    assert seg[0] == 4.0 and total == 4.0
    assert coef == np.float32(1.0) / np.float32(np.float32(4.0) + np.float32(1e-6))
