"""Router auxiliary (load-balancing) losses with the reference's signatures
(optimus/models/common/ral_functions.py:6-35 and optimus/models/olmoe/modeling_olmoe.py:29-85),
computed from per-layer statistics that one HIP pass over the logits produces
(om_router_balance_stats) instead of softmax + topk + one_hot + two means over [L*T, K, N] tensors.

For every layer: c[e] = fraction of tokens whose top-K holds expert e, P[e] = mean softmax
probability of e.  The reference's expressions reduce to
    global      : N * sum_e c[e] * P[e]     with c, P averaged over ALL tokens of all layers,
    layer-level : N * sum_layers sum_e c_l[e] * P_l[e].
Differences kept on purpose: probabilities stay in fp32 (the reference rounds the softmax of bf16
logits to bf16 before taking the mean), and the top-K order is (probability desc, index asc) where
torch.topk leaves ties implementation-defined; attention masks are not supported."""
import torch

from optimus import _native as _n


class RouterBalanceStatsFunction(torch.autograd.Function):
    """(prob_mean [N], count_frac [N]) of logits [T,N]; only prob_mean carries a gradient."""

    @staticmethod
    def forward(ctx, logits, top_k):
        _n.require_cuda_contiguous(logits)
        T, N = logits.shape
        dev = logits.device
        out = torch.empty((2, N), dtype=torch.float32, device=dev)
        ws_bytes = _n.lib().om_router_balance_workspace_bytes(T, N)
        ws = torch.empty(max(ws_bytes, 8), dtype=torch.uint8, device=dev)
        _n.check(_n.lib().om_router_balance_stats(
            _n.ptr(logits), _n.dtype_code(logits), T, N, int(top_k), _n.ptr(out), _n.ptr(out) + 4 * N,
            _n.ptr(ws), ws_bytes, _n.stream()), "om_router_balance_stats")
        ctx.save_for_backward(logits)
        ctx.T = T
        prob_mean, count_frac = out[0] / T, out[1] / T
        ctx.mark_non_differentiable(count_frac)
        return prob_mean, count_frac

    @staticmethod
    def backward(ctx, g_prob_mean, _g_count):
        (logits,) = ctx.saved_tensors
        T, N = logits.shape
        g = (g_prob_mean.float() / ctx.T).contiguous()
        dlogits = torch.empty_like(logits)
        _n.check(_n.lib().om_router_balance_bwd(_n.ptr(logits), _n.dtype_code(logits), _n.ptr(g), T, N,
                                                _n.ptr(dlogits), _n.stream()), "om_router_balance_bwd")
        return dlogits, None


def _layer_stats(gate_logits, top_k):
    return [RouterBalanceStatsFunction.apply(lg.reshape(-1, lg.shape[-1]).contiguous(), top_k)
            for lg in gate_logits]


def single_input_load_balancing_loss_func(gate_logits, num_experts, top_k):
    """Reference ral_functions.py:6-15 (one layer's logits [T,N])."""
    prob_mean, count_frac = RouterBalanceStatsFunction.apply(gate_logits.contiguous(), top_k)
    return torch.sum(count_frac * prob_mean) * num_experts


def layer_level_load_balancing_loss_func(gate_logits, num_experts=None, top_k=2, attention_mask=None):
    """Reference ral_functions.py:18-35: the per-layer losses summed over the layers."""
    if gate_logits is None or not isinstance(gate_logits, tuple):
        return 0
    assert attention_mask is None
    total = None
    for prob_mean, count_frac in _layer_stats(gate_logits, top_k):
        term = torch.sum(count_frac * prob_mean)
        total = term if total is None else total + term
    return total * num_experts


def load_balancing_loss_func(gate_logits, num_experts=None, top_k=2, attention_mask=None):
    """Reference modeling_olmoe.py:29-85 without a mask: statistics over the tokens of all layers
    together (the reference concatenates the layers' logits)."""
    if gate_logits is None or not isinstance(gate_logits, tuple):
        return 0
    if attention_mask is not None:
        raise NotImplementedError("load_balancing_loss_func: attention_mask is not supported")
    tokens = [lg.reshape(-1, lg.shape[-1]).shape[0] for lg in gate_logits]
    total = float(sum(tokens))
    prob = count = None
    for (prob_mean, count_frac), t in zip(_layer_stats(gate_logits, top_k), tokens):
        prob = prob_mean * (t / total) if prob is None else prob + prob_mean * (t / total)
        count = count_frac * (t / total) if count is None else count + count_frac * (t / total)
    return torch.sum(count * prob) * num_experts
