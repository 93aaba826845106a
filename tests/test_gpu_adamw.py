"""AdamW kernel parity (through optimus.optimizers -> C-ABI om_adamw_step).

Bar: fp32 master / exp_avg / exp_avg_sq bit-identical to the scalar C restatement of the
reference op sequence (each op rounded on its own); master within 1e-6 relative of the fp64
recurrence; bf16 params exactly bf16(master)."""
import numpy as np
import pytest
import torch

from util import bits, from_bits

pytestmark = pytest.mark.gpu

HP = dict(lr=4e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


def _state(n, seed=1002):
    import synthetic_configs as sc
    return sc.adamw_chunk(n, seed=seed)


def _run_gpu(st, step, hp, dev, steps=1):
    from optimus.optimizers import adamw_step_
    d = {k: v.clone().to(dev) for k, v in st.items()}
    for i in range(steps):
        adamw_step_(d["param"], d["grad"], d["master"], d["exp_avg"], d["exp_avg_sq"], step + i,
                    hp["lr"], hp["beta1"], hp["beta2"], hp["eps"], hp["weight_decay"])
    torch.cuda.synchronize()
    return {k: v.cpu() for k, v in d.items()}


def _run_oracle(st, step, hp, clib, steps=1):
    p = bits(st["param"]).copy(); g = bits(st["grad"]).copy()
    w = st["master"].numpy().copy(); m = st["exp_avg"].numpy().copy(); v = st["exp_avg_sq"].numpy().copy()
    for i in range(steps):
        clib.adamw_step_bf16(p, g, w, m, v, hp["lr"], hp["beta1"], hp["beta2"], hp["eps"],
                             hp["weight_decay"], step + i)
    return p, w, m, v


@pytest.mark.parametrize("n", [1, 7, 8, 2048 * 3 + 5, (1 << 20) + 3])
@pytest.mark.parametrize("wd", [0.1, 0.0])
def test_bf16_bit_exact_vs_oracle(cuda, oracle_lib, n, wd):
    hp = dict(HP, weight_decay=wd)
    st = _state(n)
    out = _run_gpu(st, 100, hp, cuda)
    p, w, m, v = _run_oracle(st, 100, hp, oracle_lib)
    assert np.array_equal(out["master"].numpy().view(np.uint32), w.view(np.uint32))
    assert np.array_equal(out["exp_avg"].numpy().view(np.uint32), m.view(np.uint32))
    assert np.array_equal(out["exp_avg_sq"].numpy().view(np.uint32), v.view(np.uint32))
    assert np.array_equal(bits(out["param"]), p)
    # params are exactly the RNE bf16 rounding of the master weights
    assert torch.equal(out["param"], out["master"].to(torch.bfloat16))


def test_multi_step_and_fp64_distance(cuda, oracle_lib):
    n = 1 << 18
    st = _state(n)
    out = _run_gpu(st, 98, HP, cuda, steps=5)
    p, w, m, v = _run_oracle(st, 98, HP, oracle_lib, steps=5)
    assert np.array_equal(out["master"].numpy().view(np.uint32), w.view(np.uint32))
    # fp64 recurrence: tolerance 1e-6 relative on the master weights (north-star bar)
    w64 = st["master"].double().numpy().copy(); m64 = st["exp_avg"].double().numpy().copy()
    v64 = st["exp_avg_sq"].double().numpy().copy()
    for i in range(5):
        oracle_lib.adamw_step_f64(bits(st["grad"]), w64, m64, v64, HP["lr"], HP["beta1"], HP["beta2"],
                                  HP["eps"], HP["weight_decay"], 98 + i)
    rel = np.abs(out["master"].double().numpy() - w64) / np.maximum(np.abs(w64), 1e-3)
    assert rel.max() <= 1e-6, rel.max()


def test_fp32_mode_bit_exact(cuda, oracle_lib):
    from optimus.optimizers import adamw_step_
    n = 100003
    st = _state(n)
    grad32 = st["grad"].float()
    w = st["master"].clone().to(cuda); g = grad32.to(cuda)
    m = st["exp_avg"].clone().to(cuda); v = st["exp_avg_sq"].clone().to(cuda)
    adamw_step_(w, g, w, m, v, 100, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"], HP["weight_decay"])
    wo = st["master"].numpy().copy(); mo = st["exp_avg"].numpy().copy(); vo = st["exp_avg_sq"].numpy().copy()
    oracle_lib.adamw_step_f32(wo, grad32.numpy(), mo, vo, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"],
                              HP["weight_decay"], 100)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), wo.view(np.uint32))
    assert np.array_equal(m.cpu().numpy().view(np.uint32), mo.view(np.uint32))
    assert np.array_equal(v.cpu().numpy().view(np.uint32), vo.view(np.uint32))


def test_optimizer_class_matches_kernel(cuda, oracle_lib):
    """MixedPrecisionAdamW: flat-buffer views, step(), zero_grad(), state_dict keys."""
    from optimus.optimizers import MixedPrecisionAdamW
    torch.manual_seed(5)
    model = torch.nn.Sequential(torch.nn.Linear(64, 96, bias=True), torch.nn.Linear(96, 33, bias=False))
    model = model.to(cuda).to(torch.bfloat16)
    ref_params = [p.detach().clone() for p in model.parameters()]
    opt = MixedPrecisionAdamW(model.parameters(), model, lr=4e-4, betas=(0.9, 0.95), eps=1e-8,
                              weight_decay=0.1, warmup_steps=10**9, dtype=torch.bfloat16, device=cuda)
    # parameters and grads are views of the flat buffers
    for p, s, sz in zip(opt.param_list, opt.param_start_inds, opt.param_sizes):
        assert p.data_ptr() == opt.flat_param.data_ptr() + 2 * s
        assert p.grad.data_ptr() == opt.flat_grad.data_ptr() + 2 * s
    assert torch.equal(opt.flat_fp32_master_param, torch.cat([r.flatten() for r in ref_params]).float())
    g = torch.Generator().manual_seed(9)
    grads = (torch.randn(opt.flat_param_size, generator=g) * 1e-3).to(torch.bfloat16)
    opt.flat_grad.copy_(grads.to(cuda))
    for pg in opt.param_groups:
        pg["lr"] = 4e-4
    norm = opt.step()
    assert abs(float(norm) - float(grads.float().norm())) < 1e-2 * float(grads.float().norm())
    assert opt.step_id == 1
    p = bits(torch.cat([r.flatten() for r in ref_params]).cpu()).copy()
    w = torch.cat([r.flatten() for r in ref_params]).float().cpu().numpy().copy()
    m = np.zeros_like(w); v = np.zeros_like(w)
    oracle_lib.adamw_step_bf16(p, bits(grads), w, m, v, 4e-4, 0.9, 0.95, 1e-8, 0.1, 1)
    assert np.array_equal(opt.flat_fp32_master_param.cpu().numpy().view(np.uint32), w.view(np.uint32))
    assert np.array_equal(bits(opt.flat_param), p)
    assert set(opt.state_dict().keys()) == {"flat_exp_avg", "flat_exp_avg_sq", "flat_fp32_master_param", "step_id"}
    opt.zero_grad()
    assert float(opt.flat_grad.abs().max()) == 0.0 and model[0].weight.grad.data_ptr() == opt.flat_grad.data_ptr()


@pytest.mark.parametrize("which", ["baseline_6.9e9", "beyond_one_launch"])
def test_full_size_int64_indexing(cuda, oracle_lib, which):
    """BASELINE size (6.9e9 elements, 110 GB of state): a CPU-generated pattern of 2^22 elements is
    tiled over the flat buffers; every tile must then equal the oracle's result on the pattern.
    Checked on tiles at the start, across the 2^31 and 2^32 element boundaries, and at the end.
    Second size: 2^33 + 2^22 + 5 elements (137 GB of state), more than one launch can take (a lane
    owns 4 elements, a launch has fewer than 2^32 lanes): the library splits the buffer, checked
    across the 2^33 boundary and on the 5-element tail."""
    import synthetic_configs as sc
    from optimus.optimizers import adamw_step_
    n = sc.ADAMW["n"] if which == "baseline_6.9e9" else (1 << 33) + (1 << 22) + 5
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    if free < 16 * n * 1.06:
        pytest.skip(f"needs {16 * n * 1.06 / 1e9:.0f} GB of free device memory")
    tile = 1 << 22
    st = _state(tile)
    reps = -(-n // tile)
    dev = {}
    for k, v in st.items():
        t = v.to(cuda)
        dev[k] = t.repeat(reps)[:n].contiguous()
        del t
    adamw_step_(dev["param"], dev["grad"], dev["master"], dev["exp_avg"], dev["exp_avg_sq"], 100,
                HP["lr"], HP["beta1"], HP["beta2"], HP["eps"], HP["weight_decay"])
    torch.cuda.synchronize()
    p, w, m, v = _run_oracle(st, 100, HP, oracle_lib)
    last_full = (n // tile - 1) * tile
    starts = [0, (1 << 31) - tile, 1 << 31, (1 << 32) - tile, 1 << 32, last_full]
    if n > (1 << 33):
        starts += [(1 << 33) - tile, 1 << 33]
    for start in starts:
        sl = slice(start, start + tile)
        assert np.array_equal(dev["master"][sl].cpu().numpy().view(np.uint32), w.view(np.uint32)), start
        assert np.array_equal(dev["exp_avg_sq"][sl].cpu().numpy().view(np.uint32), v.view(np.uint32)), start
        assert np.array_equal(bits(dev["param"][sl]), p), start
    rem = n - (n // tile) * tile
    if rem:
        assert np.array_equal(dev["master"][n - rem:].cpu().numpy().view(np.uint32), w[:rem].view(np.uint32))
    # size-independent property over the whole buffer: params are bf16(master) everywhere
    bad = 0
    for s in range(0, n, 1 << 30):
        e = min(n, s + (1 << 30))
        bad += int((dev["param"][s:e] != dev["master"][s:e].to(torch.bfloat16)).sum())
    assert bad == 0
    del dev
    torch.cuda.empty_cache()
