"""Pins the AdamW restatement (oracle/adamw_oracle.c, oracle/adamw.py).  None of these retype the
recurrence: an independent library optimizer (torch.optim.AdamW with weight_decay=0, where the two
definitions coincide), the algebraic relation that fixes WHERE the decay is applied, closed-form
special cases, and the fp64 recurrence as the distance to exact arithmetic."""
import numpy as np
import torch

from oracle import clib
from oracle.adamw import adamw_step_torch
from util import bits

HP = dict(lr=4e-4, beta1=0.9, beta2=0.95, eps=1e-8)


def _state(n, seed=0):
    g = torch.Generator().manual_seed(seed)
    grad = (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16)
    master = torch.randn(n, generator=g) * 0.02
    return grad, master, torch.zeros(n), torch.zeros(n)


def _run(grad, master, m, v, wd, steps, first_step=1):
    p = bits(master.to(torch.bfloat16)).copy()
    w = master.numpy().copy(); mm = m.numpy().copy(); vv = v.numpy().copy()
    for s in range(steps):
        clib.adamw_step_bf16(p, bits(grad), w, mm, vv, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"], wd, first_step + s)
    return p, w, mm, vv


def test_matches_torch_optim_adamw_without_decay():
    """With weight_decay = 0 the reference's update is textbook Adam; torch.optim.AdamW is an
    independent implementation of it (several steps, bias correction included)."""
    n = 4096
    grad, master, m, v = _state(n)
    param = torch.nn.Parameter(master.clone())
    opt = torch.optim.AdamW([param], lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]), eps=HP["eps"], weight_decay=0.0)
    for _ in range(5):
        param.grad = grad.float()
        opt.step()
    _, w, mm, vv = _run(grad, master, m, v, 0.0, 5)
    assert np.allclose(w, param.detach().numpy(), rtol=2e-6, atol=1e-9)
    st = opt.state[param]
    assert np.allclose(mm, st["exp_avg"].numpy(), rtol=1e-5, atol=1e-12)
    assert np.allclose(vv, st["exp_avg_sq"].numpy(), rtol=1e-5, atol=1e-15)


def test_decay_is_applied_after_the_adam_update():
    """optimizers.py:198-202: w <- (w + adam) then w <- w + (-lr*wd) w, i.e. result(wd) =
    result(0) * (1 - lr*wd).  Decaying first (torch.optim.AdamW's order) fails this."""
    grad, master, m, v = _state(2048, seed=1)
    _, w0, _, _ = _run(grad, master, m, v, 0.0, 1, first_step=100)
    _, w1, _, _ = _run(grad, master, m, v, 0.1, 1, first_step=100)
    assert np.allclose(w1, w0 * (1.0 - HP["lr"] * 0.1), rtol=3e-7, atol=0)
    wrong = master.numpy() * (1.0 - HP["lr"] * 0.1) + (w0 - master.numpy())   # decay-before-update
    assert not np.allclose(w1, wrong, rtol=3e-7, atol=0)


def test_closed_form_special_cases():
    n = 1000
    g = torch.Generator().manual_seed(2)
    grad = (torch.randn(n, generator=g) * 1e-2).to(torch.bfloat16)
    master = torch.randn(n, generator=g)
    p = bits(master.to(torch.bfloat16)).copy()
    # beta1 = beta2 = 0, wd = 0  ->  w -= lr * g / (|g| + eps)
    w = master.numpy().copy(); m = np.ones(n, np.float32); v = np.ones(n, np.float32)
    clib.adamw_step_bf16(p, bits(grad), w, m, v, 1e-3, 0.0, 0.0, 1e-8, 0.0, 7)
    gf = grad.float().numpy()
    assert np.allclose(w, master.numpy() - 1e-3 * gf / (np.abs(gf) + 1e-8), rtol=1e-6, atol=1e-9)
    assert np.allclose(m, gf) and np.allclose(v, gf * gf)
    # g = 0  ->  m, v decay geometrically
    w = master.numpy().copy(); m = np.full(n, 0.5, np.float32); v = np.full(n, 0.25, np.float32)
    zero = np.zeros(n, np.uint16)
    for s in range(3):
        clib.adamw_step_bf16(p, zero, w, m, v, 1e-3, 0.9, 0.95, 1e-8, 0.0, s + 1)
    assert np.allclose(m, 0.5 * 0.9 ** 3, rtol=1e-6) and np.allclose(v, 0.25 * 0.95 ** 3, rtol=1e-6)
    # params are the RNE bf16 rounding of the master weights
    assert np.array_equal(p, bits(torch.from_numpy(w).to(torch.bfloat16)))


def test_fp32_sequence_is_within_1e6_of_fp64():
    n = 1 << 16
    import synthetic_configs as sc
    st = sc.adamw_chunk(n)
    p = bits(st["param"]).copy(); w = st["master"].numpy().copy()
    m = st["exp_avg"].numpy().copy(); v = st["exp_avg_sq"].numpy().copy()
    w64 = w.astype(np.float64); m64 = m.astype(np.float64); v64 = v.astype(np.float64)
    clib.adamw_step_bf16(p, bits(st["grad"]), w, m, v, 4e-4, 0.9, 0.95, 1e-8, 0.1, 100)
    clib.adamw_step_f64(bits(st["grad"]), w64, m64, v64, 4e-4, 0.9, 0.95, 1e-8, 0.1, 100)
    assert (np.abs(w - w64) / np.maximum(np.abs(w64), 1e-3)).max() < 1e-6


def test_torch_op_sequence_port_agrees_with_c_restatement():
    """The PyTorch-CPU port of the reference's 13-op chunk loop (the timed cpu_baseline) and the
    scalar C restatement differ only by fused-multiply-add contraction inside torch kernels."""
    import synthetic_configs as sc
    n = 50000
    st = sc.adamw_chunk(n)
    t = {k: v.clone() for k, v in st.items()}
    adamw_step_torch(t["param"], t["grad"], t["master"], t["exp_avg"], t["exp_avg_sq"], 99, 4e-4, (0.9, 0.95),
                     1e-8, 0.1, chunk_size=16384)
    p = bits(st["param"]).copy(); w = st["master"].numpy().copy()
    m = st["exp_avg"].numpy().copy(); v = st["exp_avg_sq"].numpy().copy()
    clib.adamw_step_bf16(p, bits(st["grad"]), w, m, v, 4e-4, 0.9, 0.95, 1e-8, 0.1, 100)
    assert np.allclose(t["master"].numpy(), w, rtol=1e-6, atol=1e-10)
    assert np.allclose(t["exp_avg"].numpy(), m, rtol=1e-6, atol=1e-10)   # |m| ~ 1e-4
    assert np.allclose(t["exp_avg_sq"].numpy(), v, rtol=1e-6, atol=1e-12)   # v ~ 1e-6
    assert np.array_equal(bits(t["param"]), bits(t["master"].to(torch.bfloat16)))


# ---- float32 mode (optimizers.py:100-102: the master weights ARE the parameters, fp32 gradients) ----

def _run_f32(grad, master, m, v, wd, steps, first_step=1):
    w = master.numpy().copy(); mm = m.numpy().copy(); vv = v.numpy().copy()
    for s in range(steps):
        clib.adamw_step_f32(w, grad.numpy(), mm, vv, HP["lr"], HP["beta1"], HP["beta2"], HP["eps"], wd, first_step + s)
    return w, mm, vv


def _state_f32(n, seed=0):
    g = torch.Generator().manual_seed(seed)
    grad = torch.randn(n, generator=g) * 1e-3            # full fp32 mantissas, not bf16-representable
    master = torch.randn(n, generator=g) * 0.02
    return grad, master, torch.zeros(n), torch.zeros(n)


def test_f32_mode_matches_torch_optim_adamw_without_decay():
    """orc_adamw_step_f32 against the independent library optimizer at weight_decay = 0, several
    steps with bias correction, on gradients that use the whole fp32 mantissa (a restatement that
    rounded them to bf16 on the way in, as the bf16 form does, fails)."""
    n = 4096
    grad, master, m, v = _state_f32(n)
    param = torch.nn.Parameter(master.clone())
    opt = torch.optim.AdamW([param], lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]), eps=HP["eps"], weight_decay=0.0)
    for _ in range(5):
        param.grad = grad.clone()
        opt.step()
    w, mm, vv = _run_f32(grad, master, m, v, 0.0, 5)
    assert np.allclose(w, param.detach().numpy(), rtol=2e-6, atol=1e-9)
    st = opt.state[param]
    assert np.allclose(mm, st["exp_avg"].numpy(), rtol=1e-5, atol=1e-12)
    assert np.allclose(vv, st["exp_avg_sq"].numpy(), rtol=1e-5, atol=1e-15)
    # the same run on bf16-rounded gradients is measurably different: the fp32 form keeps all bits
    _, mm_rounded, _ = _run_f32(grad.to(torch.bfloat16).float(), master, m, v, 0.0, 5)
    assert not np.allclose(mm, mm_rounded, rtol=1e-5, atol=1e-12)


def test_f32_mode_decay_is_applied_after_the_adam_update():
    grad, master, m, v = _state_f32(2048, seed=1)
    w0, _, _ = _run_f32(grad, master, m, v, 0.0, 1, first_step=100)
    w1, _, _ = _run_f32(grad, master, m, v, 0.1, 1, first_step=100)
    assert np.allclose(w1, w0 * (1.0 - HP["lr"] * 0.1), rtol=3e-7, atol=0)
    wrong = master.numpy() * (1.0 - HP["lr"] * 0.1) + (w0 - master.numpy())
    assert not np.allclose(w1, wrong, rtol=3e-7, atol=0)


def test_f32_mode_equals_the_bf16_form_on_bf16_representable_gradients():
    """The two restatements differ only in the gradient's storage type and in the parameter copy:
    fed gradients that bf16 holds exactly they must produce the same master / m / v bit for bit
    (the bf16 form is pinned above), and the fp32 form has no separate parameter buffer."""
    import synthetic_configs as sc
    n = 30011
    st = sc.adamw_chunk(n)
    p = bits(st["param"]).copy(); w = st["master"].numpy().copy()
    m = st["exp_avg"].numpy().copy(); v = st["exp_avg_sq"].numpy().copy()
    clib.adamw_step_bf16(p, bits(st["grad"]), w, m, v, 4e-4, 0.9, 0.95, 1e-8, 0.1, 100)
    w2 = st["master"].numpy().copy(); m2 = st["exp_avg"].numpy().copy(); v2 = st["exp_avg_sq"].numpy().copy()
    clib.adamw_step_f32(w2, st["grad"].float().numpy(), m2, v2, 4e-4, 0.9, 0.95, 1e-8, 0.1, 100)
    assert np.array_equal(w.view(np.uint32), w2.view(np.uint32))
    assert np.array_equal(m.view(np.uint32), m2.view(np.uint32))
    assert np.array_equal(v.view(np.uint32), v2.view(np.uint32))


def test_f32_mode_closed_forms_and_fp64_distance():
    n = 1000
    g = torch.Generator().manual_seed(2)
    grad = torch.randn(n, generator=g) * 1e-2
    master = torch.randn(n, generator=g)
    w = master.numpy().copy(); m = np.ones(n, np.float32); v = np.ones(n, np.float32)
    clib.adamw_step_f32(w, grad.numpy(), m, v, 1e-3, 0.0, 0.0, 1e-8, 0.0, 7)
    gf = grad.numpy()
    assert np.allclose(w, master.numpy() - 1e-3 * gf / (np.abs(gf) + 1e-8), rtol=1e-6, atol=1e-9)
    assert np.array_equal(m, gf) and np.allclose(v, gf * gf, rtol=1e-7)
    # distance from exact arithmetic over one step at the benchmark's hyper-parameters
    n = 1 << 14
    grad, master, _, _ = _state_f32(n, seed=3)
    m0 = (torch.randn(n, generator=g) * 1e-4); v0 = (torch.randn(n, generator=g) * 1e-6).abs()
    w, mm, vv = _run_f32(grad, master, m0, v0, 0.1, 1, first_step=100)
    g64 = grad.double().numpy(); w64 = master.double().numpy()
    m64 = m0.double().numpy() * 0.9 + (1 - 0.9) * g64
    v64 = v0.double().numpy() * 0.95 + (1 - 0.95) * g64 * g64
    w64 = w64 - 4e-4 * (m64 / (1 - 0.9 ** 100)) / (np.sqrt(v64 / (1 - 0.95 ** 100)) + 1e-8)
    w64 = w64 - 4e-4 * 0.1 * w64
    assert (np.abs(w - w64) / np.maximum(np.abs(w64), 1e-3)).max() < 1e-6
