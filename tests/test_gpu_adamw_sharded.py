"""ShardedMixedPrecisionAdamW (reference optimus/optimizers.py:227-522) through the C-ABI: the
device-side clip decision (om_shard_clip_multiplier) and the whole step, for one process and for a
job of several ranks.

One GPU is all there is, so the ranks of a job are threads of this process that meet in an
in-process stand-in for the process group (`Rendezvous`): every collective is a barrier, a sum or
copy in rank order, and a barrier.  Everything the optimizer does itself runs as in a real job.

Bars: norm, multiplier, clipped gradients, master weights, moments and parameters bit-identical to the
scalar C restatement run rank by rank on the CPU."""
import threading

import numpy as np
import pytest
import torch

from util import bits

pytestmark = pytest.mark.gpu

HP = dict(lr=4e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


class _Net(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.a = torch.nn.Linear(67, 129, bias=True)
        self.b = torch.nn.Linear(129, 31, bias=False)
        self.c = torch.nn.Parameter(torch.zeros(5))


def _make(cuda, dtype, seed=11, **kw):
    from optimus.optimizers import ShardedMixedPrecisionAdamW
    torch.manual_seed(seed)
    net = _Net().to(dtype).to(cuda)
    opt = ShardedMixedPrecisionAdamW(net.parameters(), net, lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]),
                                     eps=HP["eps"], weight_decay=HP["weight_decay"], dtype=dtype,
                                     device=cuda, **kw)
    return net, opt


def _grad(n, dtype, seed, scale):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g) * scale).to(dtype)


def test_torch_multiplies_by_the_coefficient_cast_to_the_gradient_dtype(cuda):
    """The fact the multiplier's rounding rests on, shown with the library call the reference makes
    (optimizers.py:432) on this device: a bf16 tensor times a 0-dim float32 DEVICE tensor uses the
    coefficient rounded to bf16; the same 0-dim tensor on the CPU would be taken as an exact scalar."""
    g = _grad(1 << 18, torch.bfloat16, 1, 1.0).to(cuda)
    coef = torch.tensor(0.33371234, dtype=torch.float32, device=cuda)
    got = g.clone().mul_(coef)
    rounded = (g.float() * coef.to(torch.bfloat16).float()).to(torch.bfloat16)
    exact = (g.float() * coef).to(torch.bfloat16)
    assert torch.equal(got, rounded) and not torch.equal(got, exact)
    assert torch.equal(g.clone().mul_(coef.cpu()), exact)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_clip_multiplier_kernel_vs_oracle(cuda, oracle_lib, mode, dtype):
    from optimus import _native as n
    g = torch.Generator().manual_seed(3)
    vals = torch.cat([torch.linspace(0.2, 3.0, 129), torch.rand(100, generator=g) * 0.2 + 0.9,
                      torch.tensor([1.0, 0.99999, 1.00001, 1e-4, 1e3, 0.0])])
    if mode == 0 and dtype == torch.bfloat16:
        vals = vals.to(torch.bfloat16).float()           # a shard norm is a value of the gradient dtype
    dev = vals.to(cuda)
    out = torch.zeros(vals.numel(), 2, device=cuda)
    code = n.OM_BF16 if dtype == torch.bfloat16 else n.OM_F32
    for i in range(vals.numel()):
        n.check(n.lib().om_shard_clip_multiplier(n.ptr(dev) + 4 * i, mode, code, 1.0, n.ptr(out) + 8 * i,
                                                 n.ptr(out) + 8 * i + 4, n.stream()), "om_shard_clip_multiplier")
    out = out.cpu()
    for i, v in enumerate(vals.tolist()):
        norm, mult = oracle_lib.shard_clip_multiplier(v, mode, dtype == torch.bfloat16)
        assert float(out[i, 0]) == norm and float(out[i, 1]) == mult, (v, out[i].tolist(), norm, mult)
    assert (out[:, 1] < 1.0).any() and (out[:, 1] == 1.0).any()


def _oracle_rank_step(oracle_lib, grad_bits, param_bits, master, m, v, mult, step):
    if mult is not None:
        oracle_lib.scale_grads(grad_bits, mult)
    oracle_lib.adamw_step_bf16(param_bits, grad_bits, master, m, v, HP["lr"], HP["beta1"], HP["beta2"],
                               HP["eps"], HP["weight_decay"], step)


@pytest.mark.parametrize("warmup_steps,grad_scale", [(0, 1.0), (0, 1e-4), (10, 1.0)])
def test_single_process_step_vs_oracle(cuda, oracle_lib, warmup_steps, grad_scale):
    """No process group, one shard: the norm is the shard's norm in the gradient dtype and the
    coefficient is evaluated in that dtype (optimizers.py:404-405, :430-432)."""
    net, opt = _make(cuda, torch.bfloat16, warmup_steps=warmup_steps)
    n, size = opt.flat_buffer_size, opt.flat_param_size
    assert opt.shard_size == n == -(-size // 512) * 512 and opt.opt_key == "shard"
    assert not opt.flat_param[size:].any()                                   # padding starts as zeros
    first = next(iter(net.parameters()))
    assert first.data_ptr() == opt.flat_param.data_ptr() and first.grad.data_ptr() == opt.flat_grad.data_ptr()
    grad = torch.zeros(n, dtype=torch.bfloat16)
    grad[:size] = _grad(size, torch.bfloat16, 21, grad_scale)
    opt.flat_grad.copy_(grad)
    p = bits(opt.flat_param).copy(); w = opt.flat_fp32_master_param_shard.cpu().numpy().copy()
    m = np.zeros(n, np.float32); v = np.zeros(n, np.float32)
    norm = opt.step()
    torch.cuda.synchronize()

    g = bits(grad).copy()
    _, total, _ = oracle_lib.grad_norm_clip(g, [0], [n], 1.0)
    norm_o, mult = oracle_lib.shard_clip_multiplier(total, 0, True)
    assert norm.dtype == torch.bfloat16 and float(norm) == norm_o == total
    clips = warmup_steps == 0
    _oracle_rank_step(oracle_lib, g, p, w, m, v, mult if clips else None, 1)
    assert np.array_equal(bits(opt.flat_grad), g)
    assert np.array_equal(bits(opt.flat_param), p)
    assert np.array_equal(opt.flat_fp32_master_param_shard.cpu().numpy().view(np.uint32), w.view(np.uint32))
    assert np.array_equal(opt.flat_exp_avg_shard.cpu().numpy().view(np.uint32), m.view(np.uint32))
    assert np.array_equal(opt.flat_exp_avg_sq_shard.cpu().numpy().view(np.uint32), v.view(np.uint32))
    assert (mult < 1.0) == (grad_scale == 1.0)
    if clips and grad_scale == 1.0:
        assert not np.array_equal(g, bits(grad))
    else:
        assert np.array_equal(g, bits(grad))
    assert opt.step_id == 1


def test_single_process_float32_mode(cuda, oracle_lib):
    net, opt = _make(cuda, torch.float32)
    n, size = opt.flat_buffer_size, opt.flat_param_size
    assert opt.flat_fp32_master_param_shard.data_ptr() == opt.flat_param_shard.data_ptr()
    grad = torch.zeros(n)
    grad[:size] = _grad(size, torch.float32, 5, 1.0)
    opt.flat_grad.copy_(grad)
    w = opt.flat_param.cpu().numpy().copy()
    m = np.zeros(n, np.float32); v = np.zeros(n, np.float32)
    norm = opt.step()
    torch.cuda.synchronize()
    g = grad.numpy().copy()
    _, total, _ = oracle_lib.grad_norm_clip(g, [0], [n], 1.0)
    assert norm.dtype == torch.float32 and abs(float(norm) - total) <= 1e-6 * total
    _, mult = oracle_lib.shard_clip_multiplier(float(norm), 0, False)
    assert mult < 1.0
    oracle_lib.scale_grads(g, mult)
    oracle_lib.adamw_step_f32(w, g, m, v, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"], HP["weight_decay"], 1)
    assert np.array_equal(opt.flat_grad.cpu().numpy().view(np.uint32), g.view(np.uint32))
    assert np.array_equal(opt.flat_param.cpu().numpy().view(np.uint32), w.view(np.uint32))


class Rendezvous:
    """In-process stand-in for a process group of `world` ranks (threads).  Sums run in float32 in
    rank order and are rounded once to the tensor's dtype."""

    def __init__(self, world):
        self.world = world
        self.slots = [None] * world
        self.barrier = threading.Barrier(world, timeout=60)

    def member(self, rank):
        return _Member(self, rank)


class _Member:
    def __init__(self, job, rank):
        self.job, self.rank = job, rank
        self.calls = []

    def active(self):
        return True

    def _meet(self, tensor):
        self.job.slots[self.rank] = tensor
        self.job.barrier.wait()

    def _sum(self, pick):
        acc = None
        for r in range(self.job.world):
            t = pick(self.job.slots[r]).float()
            acc = t if acc is None else acc + t
        return acc

    def reduce_scatter(self, shard, full, group):
        self.calls.append("reduce_scatter")
        n = shard.numel()
        self._meet(full)
        acc = self._sum(lambda t: t[self.rank * n:(self.rank + 1) * n]).to(shard.dtype)
        self.job.barrier.wait()
        shard.copy_(acc)

    def all_reduce(self, tensor, group=None):
        self.calls.append("all_reduce")
        self._meet(tensor)
        acc = self._sum(lambda t: t).to(tensor.dtype)
        self.job.barrier.wait()
        tensor.copy_(acc)
        self.job.barrier.wait()

    def all_gather(self, full, shard, group):
        self.calls.append("all_gather")
        n = shard.numel()
        self._meet(shard)
        for r in range(self.job.world):
            if r != self.rank:
                full[r * n:(r + 1) * n].copy_(self.job.slots[r])
        self.job.barrier.wait()


def _run_job(opts):
    out, errs = [None] * len(opts), []

    def work(r):
        try:
            out[r] = opts[r].step()
        except BaseException as e:           # a broken barrier in the others follows; report the first
            errs.append(e)
            opts[r].exchange.job.barrier.abort()

    threads = [threading.Thread(target=work, args=(r,)) for r in range(len(opts))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not any(t.is_alive() for t in threads)
    if errs:
        raise errs[0]
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("world", [2, 4])
@pytest.mark.parametrize("flags", [{}, {"opt_use_allreduce_for_param_gather": True},
                                   {"opt_use_allreduce_for_grad_acc": True, "opt_use_chunked_allreduce": True}])
@pytest.mark.parametrize("grad_scale", [1.0, 1e-4])
def test_job_of_several_ranks_vs_oracle(cuda, oracle_lib, world, flags, grad_scale):
    """Every rank holds the same parameters and its own local gradient; two steps (the second with
    non-zero moments and new gradients)."""
    job = Rendezvous(world)
    opts = []
    for r in range(world):
        _, opt = _make(cuda, torch.bfloat16, num_shards=world, shard_id=r, **flags)
        opt.exchange = job.member(r)
        opts.append(opt)
    shard, n, size = opts[0].shard_size, opts[0].flat_buffer_size, opts[0].flat_param_size
    assert n == world * shard and shard % 512 == 0 and n - size < world * 512
    p = bits(opts[0].flat_param).copy()
    w = [opts[r].flat_fp32_master_param_shard.cpu().numpy().copy() for r in range(world)]
    for r in range(world):
        assert np.array_equal(w[r], opts[0].flat_param[r * shard:(r + 1) * shard].float().cpu().numpy())
    m = [np.zeros(shard, np.float32) for _ in range(world)]
    v = [np.zeros(shard, np.float32) for _ in range(world)]

    for step in (1, 2):
        local = []
        for r in range(world):
            g = torch.zeros(n, dtype=torch.bfloat16)
            g[:size] = _grad(size, torch.bfloat16, 100 * step + r, grad_scale)
            local.append(g)
            opts[r].flat_grad.copy_(g)
        norms = _run_job(opts)

        acc = local[0].float()
        for g in local[1:]:
            acc = acc + g.float()
        mean = acc.to(torch.bfloat16).div_(world)            # world is a power of two: exact in any form
        gb = [bits(mean[r * shard:(r + 1) * shard]).copy() for r in range(world)]
        total_sq = np.float32(0)
        for r in range(world):
            _, t, _ = oracle_lib.grad_norm_clip(gb[r], [0], [shard], 1.0)
            total_sq = np.float32(total_sq + np.float32(t) * np.float32(t)) if r else np.float32(t) * np.float32(t)
        norm_o, mult = oracle_lib.shard_clip_multiplier(float(total_sq), 1, True)
        assert (mult < 1.0) == (grad_scale == 1.0)
        for r in range(world):
            pr = p[r * shard:(r + 1) * shard]
            _oracle_rank_step(oracle_lib, gb[r], pr, w[r], m[r], v[r], mult, step)
        for r in range(world):
            o = opts[r]
            assert norms[r].dtype == torch.float32 and float(norms[r]) == norm_o
            assert np.array_equal(bits(o.flat_grad_shard), gb[r]), (step, r)
            assert np.array_equal(o.flat_fp32_master_param_shard.cpu().numpy().view(np.uint32), w[r].view(np.uint32))
            assert np.array_equal(o.flat_exp_avg_shard.cpu().numpy().view(np.uint32), m[r].view(np.uint32))
            assert np.array_equal(o.flat_exp_avg_sq_shard.cpu().numpy().view(np.uint32), v[r].view(np.uint32))
            assert np.array_equal(bits(o.flat_param), p), (step, r)        # every rank holds all parameters
    kinds = set(opts[0].exchange.calls)
    if flags.get("opt_use_allreduce_for_grad_acc"):
        assert kinds == {"all_reduce", "all_gather"}
    elif flags.get("opt_use_allreduce_for_param_gather"):
        assert kinds == {"reduce_scatter", "all_reduce"}
    else:
        assert kinds == {"reduce_scatter", "all_reduce", "all_gather"}


@pytest.mark.parametrize("chunked", [False, True])
def test_unsharded_optimizer_averages_gradients_over_the_ranks(cuda, oracle_lib, chunked):
    """MixedPrecisionAdamW with num_shards > 1 and a process group (reference optimizers.py:120-133):
    the whole flat gradient is all-reduced and divided by the number of ranks, then every rank
    takes the same norm, clip and update; two ranks as threads."""
    from optimus.optimizers import MixedPrecisionAdamW
    world = 2
    job = Rendezvous(world)
    opts = []
    for r in range(world):
        torch.manual_seed(11)
        net = _Net().to(torch.bfloat16).to(cuda)
        opt = MixedPrecisionAdamW(net.parameters(), net, lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]),
                                  eps=HP["eps"], weight_decay=HP["weight_decay"], dtype=torch.bfloat16,
                                  device=cuda, num_shards=world, shard_id=r,
                                  opt_use_chunked_allreduce=chunked)
        opt.exchange = job.member(r)
        opts.append(opt)
    n = opts[0].flat_param_size
    local = [_grad(n, torch.bfloat16, 300 + r, 1.0) for r in range(world)]
    for r in range(world):
        opts[r].flat_grad.copy_(local[r])
    p = bits(opts[0].flat_param).copy(); w = opts[0].flat_fp32_master_param.cpu().numpy().copy()
    m = np.zeros(n, np.float32); v = np.zeros(n, np.float32)
    norms = _run_job(opts)

    mean = (local[0].float() + local[1].float()).to(torch.bfloat16).div_(world)
    g = bits(mean).copy()
    _, total, coef = oracle_lib.grad_norm_clip(g, opts[0].param_start_inds, opts[0].param_sizes, 1.0)
    assert coef < 1.0
    oracle_lib.scale_grads(g, coef)
    oracle_lib.adamw_step_bf16(p, g, w, m, v, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"], HP["weight_decay"], 1)
    for r in range(world):
        assert float(norms[r]) == total
        assert np.array_equal(bits(opts[r].flat_grad), g)
        assert np.array_equal(bits(opts[r].flat_param), p)
        assert np.array_equal(opts[r].flat_fp32_master_param.cpu().numpy().view(np.uint32), w.view(np.uint32))
        assert opts[r].exchange.calls == ["all_reduce"]


def test_state_dict_keys_and_round_trip(cuda):
    _, a = _make(cuda, torch.bfloat16, num_shards=4, shard_id=2)
    a.flat_grad.copy_(_grad(a.flat_buffer_size, torch.bfloat16, 2, 1e-3))
    a.step()
    state = a.state_dict()
    assert set(state) == {"flat_exp_avg_shard", "flat_exp_avg_sq_shard", "flat_fp32_master_param_shard", "step_id"}
    assert state["flat_exp_avg_shard"].numel() == a.shard_size and state["step_id"] == 1
    _, b = _make(cuda, torch.bfloat16, seed=12, num_shards=4, shard_id=2)
    b.load_state_dict({k: (t.clone() if torch.is_tensor(t) else t) for k, t in state.items()})
    assert b.step_id == 1 and torch.equal(b.flat_fp32_master_param_shard, a.flat_fp32_master_param_shard)
    assert torch.equal(b.flat_exp_avg_sq_shard, a.flat_exp_avg_sq_shard)
    _, c = _make(cuda, torch.bfloat16, disable_optimizer_state_checkpointing=True)
    assert set(c.state_dict()) == {"step_id"}
    # without a process group a rank of a larger job updates its own shard only
    lo = 2 * a.shard_size
    _, fresh = _make(cuda, torch.bfloat16, num_shards=4, shard_id=2)
    assert torch.equal(a.flat_param[:lo], fresh.flat_param[:lo])
    assert not torch.equal(a.flat_param_shard, fresh.flat_param_shard)


def test_constructor_rejects_what_the_path_does_not_cover(cuda):
    from optimus.optimizers import ShardedMixedPrecisionAdamW
    net = _Net().to(torch.bfloat16).to(cuda)
    with pytest.raises(AssertionError):
        ShardedMixedPrecisionAdamW(net.parameters(), net, dtype=torch.bfloat16, device=None)
    with pytest.raises(AssertionError):
        ShardedMixedPrecisionAdamW(net.parameters(), net, dtype=torch.bfloat16, device=cuda, expert_parallelism=2)
    with pytest.raises(ValueError):
        ShardedMixedPrecisionAdamW(net.parameters(), net, dtype=torch.bfloat16, device=cuda, shard_divisible_by=3)
    with pytest.raises(ValueError):
        ShardedMixedPrecisionAdamW(net.parameters(), net, dtype=torch.bfloat16, device=cuda, num_shards=2, shard_id=2)
