"""Gradient norm / clip kernels and the clip folded into the AdamW kernel, through the C-ABI
(om_grad_sumsq, om_grad_norm_clip_coef, om_adamw_step_clipped) and through
MixedPrecisionAdamW.step (reference optimus/optimizers.py:136-160 followed by :162-205).

Bars: per-parameter norms, total norm and clip coefficient equal the scalar C restatement (bf16:
identical values — both sides round the same fp32 quantity, summed in a different order, to 8
bits; fp32: 1e-6 relative); given the same coefficient, the scaled gradients and the AdamW state
are bit-identical to "scale the gradients, then run the update" on the CPU."""
import numpy as np
import pytest
import torch

from util import bits

pytestmark = pytest.mark.gpu

HP = dict(lr=4e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
SIZES = [1, 7, 64, 1000, 4096, 33, 0, 129, 8191, 2, 515, 70000, 12, 3001, 200001]


def _starts(sizes):
    return [int(x) for x in np.cumsum([0] + list(sizes[:-1]))]


def _grad(n, dtype, seed, scale):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("chunk", [1 << 16, 1000, 37])
@pytest.mark.parametrize("scale", [1e-3, 1.0])
def test_norms_and_coefficient_vs_oracle(cuda, oracle_lib, dtype, chunk, scale):
    from optimus.optimizers import GradNormPlan
    flat = _grad(sum(SIZES), dtype, 5, scale)
    plan = GradNormPlan(_starts(SIZES), SIZES, cuda, chunk=chunk)
    total, coef = plan.run(flat.to(cuda))
    torch.cuda.synchronize()
    seg_o, total_o, coef_o = oracle_lib.grad_norm_clip(bits(flat).copy(), _starts(SIZES), SIZES, 1.0)
    seg = plan.seg_norms.cpu().numpy()
    if dtype == torch.bfloat16:
        assert np.array_equal(seg, seg_o)
        assert float(total) == total_o and float(coef) == coef_o
    else:
        np.testing.assert_allclose(seg, seg_o, rtol=1e-6, atol=0)
        assert abs(float(total) - total_o) <= 1e-6 * total_o
        assert abs(float(coef) - coef_o) <= 2e-6 * coef_o
    assert seg[SIZES.index(0)] == 0.0                       # the empty parameter
    assert (float(coef) == 1.0) == (total_o + 1e-6 <= 1.0)


def test_sumsq_beyond_2_pow_32_elements(cuda):
    """int64 indexing: one parameter of 2^32 + 4099 bf16 elements, all 2^-12; the sum of squares
    is exact in fp32 at every level, so the norm is a closed form."""
    from optimus.optimizers import GradNormPlan
    n = (1 << 32) + 4099
    flat = torch.full((n,), 2.0 ** -12, dtype=torch.bfloat16, device=cuda)
    plan = GradNormPlan([0], [n], cuda)
    total, coef = plan.run(flat)
    want = torch.tensor(np.sqrt(n) * 2.0 ** -12, dtype=torch.float32).to(torch.bfloat16)
    assert float(total) == float(want)
    # every chunk partial is exact
    part = plan.partials.cpu()
    assert float(part[0]) == 65536 * 2.0 ** -24 and float(part[-1]) == (n % 65536) * 2.0 ** -24
    del flat


def _state(n, seed=1002):
    import synthetic_configs as sc
    return sc.adamw_chunk(n, seed=seed)


@pytest.mark.parametrize("n", [5, 4096 + 3, (1 << 20) + 1])
@pytest.mark.parametrize("store", [True, False])
def test_clipped_step_bf16_bit_exact(cuda, oracle_lib, n, store):
    from optimus.optimizers import adamw_step_
    st = _state(n)
    coef = float(torch.tensor(0.3712).to(torch.bfloat16))
    d = {k: v.clone().to(cuda) for k, v in st.items()}
    scale = torch.tensor([coef], dtype=torch.float32, device=cuda)
    adamw_step_(d["param"], d["grad"], d["master"], d["exp_avg"], d["exp_avg_sq"], 100, HP["lr"],
                HP["beta1"], HP["beta2"], HP["eps"], HP["weight_decay"], grad_scale=scale,
                store_scaled_grad=store)
    torch.cuda.synchronize()
    p = bits(st["param"]).copy(); g = bits(st["grad"]).copy()
    w = st["master"].numpy().copy(); m = st["exp_avg"].numpy().copy(); v = st["exp_avg_sq"].numpy().copy()
    oracle_lib.scale_grads(g, coef)
    oracle_lib.adamw_step_bf16(p, g, w, m, v, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"],
                               HP["weight_decay"], 100)
    assert np.array_equal(d["master"].cpu().numpy().view(np.uint32), w.view(np.uint32))
    assert np.array_equal(d["exp_avg"].cpu().numpy().view(np.uint32), m.view(np.uint32))
    assert np.array_equal(d["exp_avg_sq"].cpu().numpy().view(np.uint32), v.view(np.uint32))
    assert np.array_equal(bits(d["param"]), p)
    assert np.array_equal(bits(d["grad"]), g if store else bits(st["grad"]))


@pytest.mark.parametrize("store", [True, False])
def test_clipped_step_fp32_bit_exact(cuda, oracle_lib, store):
    from optimus.optimizers import adamw_step_
    n = 100003
    st = _state(n)
    coef = 0.4321
    g0 = st["grad"].float()
    w = st["master"].clone().to(cuda); g = g0.clone().to(cuda)
    m = st["exp_avg"].clone().to(cuda); v = st["exp_avg_sq"].clone().to(cuda)
    scale = torch.tensor([coef], dtype=torch.float32, device=cuda)
    adamw_step_(w, g, w, m, v, 100, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"], HP["weight_decay"],
                grad_scale=scale, store_scaled_grad=store)
    torch.cuda.synchronize()
    go = g0.numpy().copy(); wo = st["master"].numpy().copy()
    mo = st["exp_avg"].numpy().copy(); vo = st["exp_avg_sq"].numpy().copy()
    oracle_lib.scale_grads(go, float(np.float32(coef)))
    oracle_lib.adamw_step_f32(wo, go, mo, vo, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"],
                              HP["weight_decay"], 100)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), wo.view(np.uint32))
    assert np.array_equal(m.cpu().numpy().view(np.uint32), mo.view(np.uint32))
    assert np.array_equal(v.cpu().numpy().view(np.uint32), vo.view(np.uint32))
    assert np.array_equal(g.cpu().numpy(), go if store else g0.numpy())


class _Net(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.a = torch.nn.Linear(67, 129, bias=True)
        self.b = torch.nn.Linear(129, 31, bias=False)
        self.c = torch.nn.Parameter(torch.zeros(5))


@pytest.mark.parametrize("warmup_steps,grad_scale", [(0, 1.0), (0, 1e-3), (10, 1.0)])
def test_optimizer_step_clips_like_the_reference_sequence(cuda, oracle_lib, warmup_steps, grad_scale):
    """Whole MixedPrecisionAdamW.step(): norm over the parameters' gradient views, clip to 1.0 after
    warm-up, update.  Checked against the CPU sequence norm -> scale -> update on the same bits."""
    from optimus.optimizers import MixedPrecisionAdamW
    torch.manual_seed(11)
    net = _Net().to(torch.bfloat16).to(cuda)
    opt = MixedPrecisionAdamW(net.parameters(), net, lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]),
                              eps=HP["eps"], weight_decay=HP["weight_decay"], warmup_steps=warmup_steps,
                              dtype=torch.bfloat16, device=cuda)
    n = opt.flat_param_size
    grad = _grad(n, torch.bfloat16, 21, grad_scale)
    opt.flat_grad.copy_(grad)
    master0 = opt.flat_fp32_master_param.cpu().clone()
    param0 = opt.flat_param.cpu().clone()
    norm = opt.step()
    torch.cuda.synchronize()

    sizes = opt.param_sizes
    g = bits(grad).copy()
    _, total_o, coef_o = oracle_lib.grad_norm_clip(g, opt.param_start_inds, sizes, 1.0)
    assert norm.dtype == torch.bfloat16 and float(norm) == total_o
    clips = warmup_steps == 0
    if clips:
        oracle_lib.scale_grads(g, coef_o)
    p = bits(param0).copy(); w = master0.numpy().copy()
    m = np.zeros(n, np.float32); v = np.zeros(n, np.float32)
    oracle_lib.adamw_step_bf16(p, g, w, m, v, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"],
                               HP["weight_decay"], 1)
    assert np.array_equal(opt.flat_fp32_master_param.cpu().numpy().view(np.uint32), w.view(np.uint32))
    assert np.array_equal(bits(opt.flat_param), p)
    assert np.array_equal(bits(opt.flat_grad), g)           # clipped in place, like the reference
    if clips and grad_scale == 1.0:
        assert coef_o < 1.0 and not np.array_equal(g, bits(grad))
    # the model's parameters are still views of the flat buffer
    first = next(iter(net.parameters()))
    assert first.data_ptr() == opt.flat_param.data_ptr()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_returned_norm_is_not_overwritten_by_the_next_step(cuda, dtype):
    """step() hands back a tensor of its own (the reference returns get_total_norm's fresh result,
    optimizers.py:136-158): a training loop that keeps the norms of several steps must not see the
    first one change when the second step runs."""
    from optimus.optimizers import MixedPrecisionAdamW
    torch.manual_seed(5)
    net = _Net().to(dtype).to(cuda)
    opt = MixedPrecisionAdamW(net.parameters(), net, lr=1e-3, dtype=dtype, device=cuda, warmup_steps=10**9)
    opt.flat_grad.copy_(_grad(opt.flat_param_size, dtype, 1, 1.0))
    first = opt.step()
    kept = float(first)
    opt.flat_grad.copy_(_grad(opt.flat_param_size, dtype, 2, 3.0))
    second = opt.step()
    torch.cuda.synchronize()
    assert float(first) == kept and abs(float(second) - 3.0 * kept) < 0.1 * kept
    assert first.data_ptr() != second.data_ptr() and first.dtype == dtype


@pytest.mark.parametrize("clip", [True, False])
def test_parameters_outside_the_optimizer_count_in_norm_and_clip(cuda, clip):
    """A model with parameters the optimizer was not given: the reference takes the norm and clips
    over model.parameters() (optimizers.py:143-158), so their gradients count and are scaled too.
    Checked against the same library calls on CPU copies."""
    from optimus.optimizers import MixedPrecisionAdamW
    torch.manual_seed(3)
    net = _Net().to(torch.bfloat16).to(cuda)
    owned = [net.a.weight, net.a.bias]
    opt = MixedPrecisionAdamW(owned, net, lr=1e-3, dtype=torch.bfloat16, device=cuda,
                              warmup_steps=0 if clip else 10**9)
    g = torch.Generator().manual_seed(8)
    for p in net.parameters():
        val = torch.randn(p.shape, generator=g).to(torch.bfloat16).to(cuda)
        if p.grad is None:
            p.grad = val
        else:
            p.grad.copy_(val)
    cpu = [p.grad.detach().cpu().clone() for p in net.parameters()]
    want = torch.nn.utils.get_total_norm(cpu)
    if clip:
        holders = [torch.nn.Parameter(torch.empty_like(t)) for t in cpu]
        for h, t in zip(holders, cpu):
            h.grad = t
        torch.nn.utils.clip_grads_with_norm_(holders, 1.0, want)
    norm = opt.step()
    torch.cuda.synchronize()
    assert float(norm) == float(want)
    for p, t in zip(net.parameters(), cpu):
        assert torch.equal(p.grad.cpu(), t), "gradient after step() differs from the library sequence"
    assert float(want) > 1.0
