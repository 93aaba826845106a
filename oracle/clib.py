"""ctypes bindings of oracle/liboracle.so (moe_oracle.c, adamw_oracle.c) over numpy arrays.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).
bf16 tensors travel as numpy uint16 arrays holding the raw bit patterns.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    """Compile the C restatement (gcc, a second or two)."""
    subprocess.run(["make", "-s", "-C", _HERE, "-B", "liboracle.so"], check=True)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


I64 = ctypes.c_int64
I32 = ctypes.c_int
F64 = ctypes.c_double


def f32_to_bf16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_bf16(_p(x), _p(out), I64(x.size))
    return out


def bf16_bits_to_f32(x):
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib().orc_bf16_to_f32(_p(x), _p(out), I64(x.size))
    return out


def index_construction(selected_experts, num_local_experts, expert_start_idx, expert_end_idx,
                       tokens_per_thread=8):
    """K1 -> K2 -> K3 exactly as FastOlmoeParallelSparseMoeBlock runs them (moe.py:486-554).

    Returns a dict with every intermediate the reference materialises.
    """
    se = _c(selected_experts, np.int64)
    T, K = se.shape
    assert T % tokens_per_thread == 0
    TH = T // tokens_per_thread
    NR = num_local_experts
    partial = np.zeros((NR, TH), np.int32)
    expert_counts_ep = np.zeros(T, np.int32)
    lib().orc_compute_partial_token_counts(_p(se), _p(partial), _p(expert_counts_ep),
                                           I32(expert_start_idx), I32(expert_end_idx),
                                           I64(T), I64(K), I64(TH))
    partial_cum = np.zeros(NR * TH + 1, np.int32)
    cum_token_counts = np.zeros(NR + 1, np.int32)
    cum_expert_counts_ep = np.zeros(T + 1, np.int32)
    lib().orc_token_count_scans(_p(partial), _p(expert_counts_ep), _p(partial_cum),
                                _p(cum_token_counts), _p(cum_expert_counts_ep),
                                I64(NR), I64(TH), I64(T))
    TR = int(cum_token_counts[-1])
    incr = np.zeros((NR, TH), np.int32)
    sel_idx = np.full(TR, -1, np.int32)
    input_indices = np.full(TR, -1, np.int32)
    output_indices = np.full(TR, -1, np.int32)
    lib().orc_compute_input_and_output_indices(_p(se), _p(partial_cum), _p(incr),
                                               _p(cum_expert_counts_ep), _p(sel_idx),
                                               _p(input_indices), _p(output_indices),
                                               I32(expert_start_idx), I32(expert_end_idx),
                                               I64(T), I64(K), I64(TH))
    return dict(partial_token_counts=partial, expert_counts_ep=expert_counts_ep,
                partial_cum_token_counts=partial_cum, cum_token_counts=cum_token_counts,
                cum_expert_counts_ep=cum_expert_counts_ep, selected_experts_indices=sel_idx,
                input_indices=input_indices, output_indices=output_indices,
                num_routed_tokens=TR)


def _is_bf16(a):
    return a.dtype == np.uint16


def index_gather(inp, indices):
    indices = _c(indices, np.int32)
    O, E = indices.shape[0], inp.shape[1]
    out = np.empty((O, E), inp.dtype)
    fn = lib().orc_index_gather_bf16 if _is_bf16(inp) else lib().orc_index_gather_f32
    inp = np.ascontiguousarray(inp)
    fn(_p(inp), _p(indices), _p(out), I64(O), I64(E))
    return out


def index_add(inp, output, indices):
    """In place on `output` (a contiguous numpy array), serial in row order."""
    indices = _c(indices, np.int32)
    inp = np.ascontiguousarray(inp)
    assert output.flags.c_contiguous
    fn = lib().orc_index_add_bf16 if _is_bf16(inp) else lib().orc_index_add_f32
    fn(_p(inp), _p(output), _p(indices), I64(inp.shape[0]), I64(inp.shape[1]))
    return output


def shuffle_sub_matrix_reduce(ggemm_input_grad, cum_expert_counts_ep, output_indices, T):
    g = np.ascontiguousarray(ggemm_input_grad)
    E = g.shape[1]
    out = np.empty((T, E), g.dtype)
    fn = (lib().orc_shuffle_sub_matrix_reduce_bf16 if _is_bf16(g)
          else lib().orc_shuffle_sub_matrix_reduce_f32)
    fn(_p(g), _p(_c(cum_expert_counts_ep, np.int32)), _p(_c(output_indices, np.int32)), _p(out),
       I64(T), I64(E))
    return out


def reduce_ggemm_output(ggemm_output, routing_weights, cum_expert_counts_ep,
                        selected_experts_indices, output_indices, skip_weights_scaling=False):
    y = np.ascontiguousarray(ggemm_output)
    w = np.ascontiguousarray(routing_weights)
    T, K = w.shape
    E = y.shape[1]
    out = np.empty((T, E), y.dtype)
    ce = _c(cum_expert_counts_ep, np.int32)
    si = _c(selected_experts_indices, np.int32)
    oi = _c(output_indices, np.int32)
    if _is_bf16(y):
        lib().orc_reduce_ggemm_output_bf16(_p(y), _p(w), I32(0 if _is_bf16(w) else 1), _p(ce), _p(si),
                                           _p(oi), _p(out), I64(T), I64(K), I64(E),
                                           I32(int(skip_weights_scaling)))
    else:
        assert w.dtype == np.float32
        lib().orc_reduce_ggemm_output_f32(_p(y), _p(w), _p(ce), _p(si), _p(oi), _p(out),
                                          I64(T), I64(K), I64(E), I32(int(skip_weights_scaling)))
    return out


def reduce_ggemm_output_backward(dout, ggemm_output, routing_weights, selected_experts_indices,
                                 input_indices, output_indices):
    d = np.ascontiguousarray(dout)
    y = np.ascontiguousarray(ggemm_output)
    w = np.ascontiguousarray(routing_weights)
    T, K = w.shape
    RT, E = y.shape
    dy = np.empty_like(y)
    dw = np.zeros_like(w)
    si = _c(selected_experts_indices, np.int32)
    ii = _c(input_indices, np.int32)
    oi = _c(output_indices, np.int32)
    if _is_bf16(y):
        lib().orc_reduce_ggemm_output_backward_bf16(_p(d), _p(y), _p(w), I32(0 if _is_bf16(w) else 1),
                                                    _p(si), _p(ii), _p(oi), _p(dy), _p(dw),
                                                    I64(RT), I64(K), I64(E))
    else:
        lib().orc_reduce_ggemm_output_backward_f32(_p(d), _p(y), _p(w), _p(si), _p(ii), _p(oi),
                                                   _p(dy), _p(dw), I64(RT), I64(K), I64(E))
    return dy, dw


def swiglu_fwd(g, u):
    g = _c(g, np.float32); u = _c(u, np.float32)
    h = np.empty_like(g)
    lib().orc_swiglu_fwd_f32(_p(g), _p(u), _p(h), I64(g.size))
    return h


def swiglu_bwd(dh, g, u):
    dh = _c(dh, np.float32); g = _c(g, np.float32); u = _c(u, np.float32)
    dg = np.empty_like(g); du = np.empty_like(g)
    lib().orc_swiglu_bwd_f32(_p(dh), _p(g), _p(u), _p(dg), _p(du), I64(g.size))
    return dg, du


def adamw_step_bf16(param, grad, master, exp_avg, exp_avg_sq, lr, beta1, beta2, eps,
                    weight_decay, step):
    """In place on param (uint16 bits), master, exp_avg, exp_avg_sq. `step` is 1-based."""
    for a in (param, grad, master, exp_avg, exp_avg_sq):
        assert a.flags.c_contiguous
    assert param.dtype == np.uint16 and grad.dtype == np.uint16
    assert master.dtype == exp_avg.dtype == exp_avg_sq.dtype == np.float32
    lib().orc_adamw_step_bf16(_p(param), _p(grad), _p(master), _p(exp_avg), _p(exp_avg_sq),
                              I64(master.size), F64(lr), F64(beta1), F64(beta2), F64(eps),
                              F64(weight_decay), I64(step))


def adamw_step_f32(param_master, grad, exp_avg, exp_avg_sq, lr, beta1, beta2, eps,
                   weight_decay, step):
    for a in (param_master, grad, exp_avg, exp_avg_sq):
        assert a.flags.c_contiguous and a.dtype == np.float32
    lib().orc_adamw_step_f32(_p(param_master), _p(grad), _p(exp_avg), _p(exp_avg_sq),
                             I64(param_master.size), F64(lr), F64(beta1), F64(beta2), F64(eps),
                             F64(weight_decay), I64(step))


def adamw_step_f64(grad, master, exp_avg, exp_avg_sq, lr, beta1, beta2, eps, weight_decay, step):
    assert grad.dtype == np.uint16
    for a in (master, exp_avg, exp_avg_sq):
        assert a.flags.c_contiguous and a.dtype == np.float64
    lib().orc_adamw_step_f64(_p(grad), _p(master), _p(exp_avg), _p(exp_avg_sq), I64(master.size),
                             F64(lr), F64(beta1), F64(beta2), F64(eps), F64(weight_decay),
                             I64(step))


def grad_norm_clip(grad, starts, sizes, max_norm=1.0):
    """Per-parameter norms, total norm and clip coefficient of a flat gradient buffer
    (uint16 bf16 bits or float32).  Returns (seg_norms float32[P], total_norm, clip_coef)."""
    assert grad.flags.c_contiguous and grad.dtype in (np.uint16, np.float32)
    starts = np.ascontiguousarray(starts, dtype=np.int64)
    sizes = np.ascontiguousarray(sizes, dtype=np.int64)
    seg = np.zeros(len(sizes), dtype=np.float32)
    total = np.zeros(1, dtype=np.float32)
    coef = np.zeros(1, dtype=np.float32)
    fn = lib().orc_grad_norm_clip_bf16 if grad.dtype == np.uint16 else lib().orc_grad_norm_clip_f32
    fn(_p(grad), _p(starts), _p(sizes), I64(len(sizes)), F64(max_norm), _p(seg), _p(total), _p(coef))
    return seg, float(total[0]), float(coef[0])


def scale_grads(grad, coef):
    """In place: grad = cast(float(grad) * coef)."""
    assert grad.flags.c_contiguous and grad.dtype in (np.uint16, np.float32)
    fn = lib().orc_scale_grads_bf16 if grad.dtype == np.uint16 else lib().orc_scale_grads_f32
    fn(_p(grad), I64(grad.size), ctypes.c_float(coef))


def shard_clip_multiplier(value, mode, grad_is_bf16, max_norm=1.0):
    """(grad_norm, multiplier) of the sharded optimizer's clip decision; `value` is the shard norm
    (mode 0) or the summed squared shard norms (mode 1)."""
    norm = np.zeros(1, dtype=np.float32)
    mult = np.zeros(1, dtype=np.float32)
    lib().orc_shard_clip_multiplier(ctypes.c_float(value), ctypes.c_int(mode), ctypes.c_int(int(grad_is_bf16)),
                                    F64(max_norm), _p(norm), _p(mult))
    return float(norm[0]), float(mult[0])
