"""Pins the restatement of the sharded optimizer's clip decision and step
(oracle/adamw_oracle.c orc_shard_clip_multiplier, oracle/adamw.py sharded_clip_and_step_torch;
reference optimus/optimizers.py:398-479) on the CPU:
  * the scalar C function against the torch expressions the reference evaluates, op by op, over
    values below, near and above 1 (a dropped rounding, a division instead of reciprocal-times, or
    the unrounded coefficient in the multiply each changes a result somewhere in these sweeps);
  * the step of S ranks against the unsharded step: AdamW is element-wise, so with the same
    multiplier the shards' results are the slices of the whole buffer's;
  * the all-reduced norm against the norm of the whole gradient (equal up to the bf16 rounding of
    the S shard norms)."""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle.adamw import adamw_step_torch, sharded_clip_and_step_torch
from util import bits

HP = dict(lr=4e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)


def _values():
    g = torch.Generator().manual_seed(3)
    v = torch.cat([torch.linspace(0.2, 3.0, 257), torch.rand(300, generator=g) * 0.2 + 0.9,
                   torch.tensor([1.0, 0.99999, 1.00001, 1e-4, 1e3, 0.0])])
    return v


def test_mode0_bf16_is_the_expression_on_a_bf16_tensor():
    for v in _values().to(torch.bfloat16):
        coef = 1.0 / (v + 1e-6)                                # optimizers.py:430 on a 0-dim bf16 tensor
        assert coef.dtype == torch.bfloat16
        want = float(coef) if bool(coef < 1.0) else 1.0
        norm, mult = clib.shard_clip_multiplier(float(v), 0, True)
        assert norm == float(v) and mult == want, (float(v), mult, want)


def test_mode0_f32_and_mode1_are_plain_fp32():
    """fp32 branches against IEEE single-precision arithmetic as numpy does it (sqrt, add, divide and
    multiply each correctly rounded), and against the torch expressions: those agree to one unit in
    the last place of the norm, because torch's CPU sqrt (a vector-library routine) is not always
    correctly rounded, while the device sqrt the reference runs is."""
    one, tiny = np.float32(1.0), np.float32(1e-6)
    for v in _values():
        coef = 1.0 / (v + 1e-6)
        want = float(coef) if bool(coef < 1.0) else 1.0
        norm, mult = clib.shard_clip_multiplier(float(v), 0, False)
        assert norm == float(v) and mult == want
        sq = torch.pow(v, 2) + torch.pow(v * 0.5, 2)           # two ranks' squared norms, summed
        gn = np.sqrt(np.float32(float(sq)))
        c = one / (gn + tiny) * one
        norm, mult = clib.shard_clip_multiplier(float(sq), 1, False)
        assert norm == float(gn) and mult == (float(c) if c < one else 1.0)
        assert abs(float(torch.sqrt(sq)) - norm) <= 2.0 ** -23 * norm
        # bf16 gradients: the multiply casts the fp32 coefficient to bf16
        norm, mult = clib.shard_clip_multiplier(float(sq), 1, True)
        assert norm == float(gn)
        assert mult == (float(torch.tensor(float(c)).to(torch.bfloat16)) if c < one else 1.0)


def test_the_cast_of_the_coefficient_changes_gradients():
    """The rounding of the coefficient to bf16 is visible: for a typical coefficient a fifth of the
    scaled gradients differ from those scaled by the fp32 value."""
    g = torch.randn(20000, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    coef = torch.tensor(0.33371234)
    a = g.clone().mul_(coef.to(torch.bfloat16))
    b = (g.float() * coef).to(torch.bfloat16)
    assert 0.02 < float((a != b).float().mean()) < 0.9


def _job(S, shard, scale, seed):
    g = torch.Generator().manual_seed(seed)
    n = S * shard
    grad = (torch.randn(n, generator=g) * scale).to(torch.bfloat16)
    param = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16)
    return grad, param


@pytest.mark.parametrize("S,scale", [(1, 1.0), (4, 1.0), (4, 1e-4), (3, 2e-3)])
def test_sharded_step_is_the_unsharded_step_in_slices(S, scale):
    shard = 1536
    grad, param = _job(S, shard, scale, 7)
    gs = [t.clone() for t in grad.split(shard)]
    ps = [t.clone() for t in param.split(shard)]
    ws = [p.float() for p in ps]
    ms = [torch.zeros(shard) for _ in range(S)]
    vs = [torch.zeros(shard) for _ in range(S)]
    norm = sharded_clip_and_step_torch(gs, ps, ws, ms, vs, 4, HP["lr"], HP["betas"], HP["eps"],
                                       HP["weight_decay"], clip=True, process_group=True)
    assert norm.dtype == torch.float32
    # the all-reduced norm is the whole gradient's norm up to the bf16 rounding of S shard norms
    whole = float(torch.linalg.vector_norm(grad.double()))
    assert abs(float(norm) - whole) <= 2.0 ** -8 * whole
    # the same multiplier applied to the whole buffer, then one unsharded update
    coef = 1.0 / (norm + 1e-6)
    mult = float(coef.to(torch.bfloat16)) if bool(coef < 1.0) else 1.0
    _, mult_c = clib.shard_clip_multiplier(float(norm) ** 2, 1, True)
    assert mult_c == mult
    sq = sum(float(torch.nn.utils.get_total_norm(t).float()) ** 2 for t in grad.split(shard))
    G = grad.clone()
    if mult < 1.0:
        G.mul_(torch.tensor(mult, dtype=torch.bfloat16))
    P = param.clone(); W = param.float(); M = torch.zeros(S * shard); V = torch.zeros(S * shard)
    adamw_step_torch(P, G, W, M, V, 4, HP["lr"], HP["betas"], HP["eps"], HP["weight_decay"])
    assert torch.equal(torch.cat(gs), G) and torch.equal(torch.cat(ps), P)
    assert torch.equal(torch.cat(ws), W) and torch.equal(torch.cat(ms), M) and torch.equal(torch.cat(vs), V)
    if scale == 1.0:
        assert mult < 1.0 and not torch.equal(G, grad)
    else:
        assert mult == 1.0 and torch.equal(G, grad)
    assert abs(sq - float(norm) ** 2) <= 1e-5 * sq


def test_single_process_branch_returns_the_shard_norm_in_the_gradient_dtype():
    grad, param = _job(1, 2048, 1.0, 9)
    gs, ps = [grad.clone()], [param.clone()]
    ws, ms, vs = [param.float()], [torch.zeros(2048)], [torch.zeros(2048)]
    norm = sharded_clip_and_step_torch(gs, ps, ws, ms, vs, 0, HP["lr"], HP["betas"], HP["eps"],
                                       HP["weight_decay"], clip=True, process_group=False)
    assert norm.dtype == torch.bfloat16
    seg, total, _ = clib.grad_norm_clip(bits(grad).copy(), [0], [2048], 1.0)
    assert float(norm) == total == float(seg[0])
    _, mult = clib.shard_clip_multiplier(total, 0, True)
    assert mult < 1.0
    want = grad.clone().mul_(torch.tensor(mult, dtype=torch.bfloat16))
    assert torch.equal(gs[0], want)
