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
torch.topk leaves ties implementation-defined."""
import torch

from optimus import _native as _n


class RouterBalanceStatsFunction(torch.autograd.Function):
    """(prob_sum [N], count [N]) of logits [T,N]: the sums over the tokens, each weighted by
    `token_weight` [T] (fp32, or None for 1), of the softmax probabilities and of the top-K
    membership.  Only prob_sum carries a gradient."""

    @staticmethod
    def forward(ctx, logits, top_k, token_weight):
        _n.require_cuda_contiguous(logits, token_weight)
        T, N = logits.shape
        dev = logits.device
        out = torch.empty((2, N), dtype=torch.float32, device=dev)
        ws_bytes = _n.lib().om_router_balance_workspace_bytes(T, N)
        ws = torch.empty(max(ws_bytes, 8), dtype=torch.uint8, device=dev)
        _n.check(_n.lib().om_router_balance_stats_masked(
            _n.ptr(logits), _n.dtype_code(logits), _n.ptr(token_weight), T, N, int(top_k), _n.ptr(out),
            _n.ptr(out) + 4 * N, _n.ptr(ws), ws_bytes, _n.stream()), "om_router_balance_stats_masked")
        ctx.save_for_backward(logits, token_weight)
        prob_sum, count = out[0], out[1]
        ctx.mark_non_differentiable(count)
        return prob_sum, count

    @staticmethod
    def backward(ctx, g_prob_sum, _g_count):
        logits, token_weight = ctx.saved_tensors
        T, N = logits.shape
        g = g_prob_sum.float().contiguous()
        dlogits = torch.empty_like(logits)
        _n.check(_n.lib().om_router_balance_bwd_masked(
            _n.ptr(logits), _n.dtype_code(logits), _n.ptr(g), _n.ptr(token_weight), T, N, _n.ptr(dlogits),
            _n.stream()), "om_router_balance_bwd_masked")
        return dlogits, None, None


def _layer_sums(gate_logits, top_k, token_weight=None):
    """Per layer: (prob_sum, count, weight of the layer's tokens)."""
    out = []
    for lg in gate_logits:
        flat = lg.reshape(-1, lg.shape[-1]).contiguous()
        if token_weight is not None and token_weight.numel() != flat.shape[0]:
            raise ValueError(f"attention_mask has {token_weight.numel()} entries, a layer's router logits "
                             f"have {flat.shape[0]} tokens")
        prob_sum, count = RouterBalanceStatsFunction.apply(flat, top_k, token_weight)
        out.append((prob_sum, count, float(flat.shape[0])))
    return out


def single_input_load_balancing_loss_func(gate_logits, num_experts, top_k):
    """Reference ral_functions.py:6-15 (one layer's logits [T,N])."""
    T = gate_logits.shape[0]
    prob_sum, count = RouterBalanceStatsFunction.apply(gate_logits.contiguous(), top_k, None)
    return torch.sum((count / T) * (prob_sum / T)) * num_experts


def layer_level_load_balancing_loss_func(gate_logits, num_experts=None, top_k=2, attention_mask=None):
    """Reference ral_functions.py:18-35: the per-layer losses summed over the layers (the reference
    asserts that no mask is given here)."""
    if gate_logits is None or not isinstance(gate_logits, tuple):
        return 0
    assert attention_mask is None
    total = None
    for prob_sum, count, t in _layer_sums(gate_logits, top_k):
        term = torch.sum((count / t) * (prob_sum / t))
        total = term if total is None else total + term
    return total * num_experts


def load_balancing_loss_func(gate_logits, num_experts=None, top_k=2, attention_mask=None):
    """Reference modeling_olmoe.py:29-85: statistics over the tokens of all layers together (the
    reference concatenates the layers' logits).  With `attention_mask` [batch, sequence] every
    token's contribution is multiplied by its mask entry and the means are taken over the sum of the
    mask (modeling_olmoe.py:58-83); every layer's logits then hold batch * sequence tokens in the
    mask's order."""
    if gate_logits is None or not isinstance(gate_logits, tuple):
        return 0
    weight = None
    if attention_mask is not None:
        weight = attention_mask.to(device=gate_logits[0].device, dtype=torch.float32).reshape(-1).contiguous()
    sums = _layer_sums(gate_logits, top_k, weight)
    if weight is None:
        norm = float(sum(t for _, _, t in sums))
    else:
        norm = weight.sum() * len(sums)
    prob = count = None
    for prob_sum, cnt, _ in sums:
        prob = prob_sum if prob is None else prob + prob_sum
        count = cnt if count is None else count + cnt
    return torch.sum((count / norm) * (prob / norm)) * num_experts
