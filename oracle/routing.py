"""Router restatements in PyTorch-CPU.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

* olmoe_router        — optimus/models/common/moe.py:467-471
                        (= optimus/models/olmoe/modeling_olmoe.py:295-299)
* dsv3_topk_indices   — optimus/models/deepseek_v3/modeling_deepseek_v3.py:164-180
* dsv3_router         — optimus/models/deepseek_v3/modeling_deepseek_v3.py:182-192

Tie-break.  The reference calls torch.topk, whose order among equal values is an
implementation property.  The oracle fixes it: among equal scores the lower expert
index comes first (a stable descending sort).  On rows without ties this is exactly
torch.topk(sorted=True); tests/test_oracle_routing.py checks that against the library
call.  For the DeepSeek router the reference asks for sorted=False, so the order of a
token's K experts is unspecified there; the oracle returns them in descending
score-for-choice order and parity on that path is per-token *sets* plus weights.
"""
import torch


def _topk_stable(values, k):
    """Top-k along the last dim, descending, lower index first among equals."""
    s = torch.sort(values, dim=-1, descending=True, stable=True)
    return s.values[..., :k].contiguous(), s.indices[..., :k].contiguous()


def olmoe_router(router_logits, top_k, norm_topk_prob, out_dtype):
    """-> (routing_weights [T,K] out_dtype, selected_experts [T,K] int64, probs [T,N] fp32)."""
    probs = torch.softmax(router_logits, dim=1, dtype=torch.float)       # moe.py:467
    routing_weights, selected_experts = _topk_stable(probs, top_k)       # moe.py:468
    if norm_topk_prob:
        routing_weights = routing_weights / routing_weights.sum(dim=-1, keepdim=True)  # :469-470
    return routing_weights.to(out_dtype), selected_experts, probs        # :471


def min_topk_gap_ulps(scores, top_k):
    """Smallest gap, in units of fp32 ulp of the larger neighbour, between adjacent entries
    of each row's top-(K+1) scores.  Fixtures are valid for bit-exact index parity when this
    exceeds a few ulp: a last-ulp difference between two exp() implementations cannot then
    reorder a row."""
    k1 = min(top_k + 1, scores.shape[-1])
    top = torch.sort(scores.float(), dim=-1, descending=True).values[..., :k1]
    gap = top[..., :-1] - top[..., 1:]
    ulp = torch.abs(top[..., :-1]) * (2.0 ** -23)
    return float((gap / ulp.clamp_min(1e-45)).min())


def dsv3_topk_indices(scores, bias, n_group, topk_group, top_k):
    """Group-limited selection, modeling_deepseek_v3.py:164-180 (sorted=False there)."""
    T, N = scores.shape
    scores_for_choice = scores.view(-1, N) + bias.unsqueeze(0)                        # :164
    per_group = scores_for_choice.view(-1, n_group, N // n_group)
    group_scores = _topk_stable(per_group, 2)[0].sum(dim=-1)                          # :165-169
    group_idx = _topk_stable(group_scores, topk_group)[1]                             # :170
    group_mask = torch.zeros_like(group_scores)
    group_mask.scatter_(1, group_idx, 1)                                              # :171-172
    score_mask = (group_mask.unsqueeze(-1).expand(-1, n_group, N // n_group).reshape(-1, N))
    scores_for_choice = scores_for_choice.masked_fill(~score_mask.bool(), 0.0)        # :178
    return _topk_stable(scores_for_choice, top_k)[1], scores_for_choice               # :179


def dsv3_selection_margin(scores, bias, n_group, topk_group, top_k):
    """Per token, the smallest gap that the group-limited selection (modeling_deepseek_v3.py:164-180)
    rests on: between the last kept and the first dropped group score, and between the K-th and
    the (K+1)-th choice value among the kept groups.  A fixture whose margins all exceed the
    difference two fp32 evaluations of the logits can have (summation order: ~1e-7) selects the
    same expert SETS on the CPU and the GPU, which is what makes set-exact parity a fair demand."""
    T, N = scores.shape
    choice = scores.view(-1, N) + bias.unsqueeze(0)
    group_scores = _topk_stable(choice.view(-1, n_group, N // n_group), 2)[0].sum(dim=-1)
    gs = torch.sort(group_scores, dim=-1, descending=True).values
    group_gap = gs[:, topk_group - 1] - gs[:, topk_group] if topk_group < n_group else torch.full((T,), float("inf"))
    _, masked = dsv3_topk_indices(scores, bias, n_group, topk_group, top_k)
    ms = torch.sort(masked, dim=-1, descending=True).values
    choice_gap = ms[:, top_k - 1] - ms[:, top_k]
    return torch.minimum(group_gap, choice_gap)


def dsv3_router(hidden_states, weight, bias, n_group, topk_group, top_k, norm_topk_prob,
                routed_scaling_factor):
    """-> (topk_indices [T,K] int64, topk_weights [T,K] fp32, router_logits fp32)."""
    x = hidden_states.reshape(-1, hidden_states.shape[-1])
    router_logits = torch.nn.functional.linear(x.type(torch.float32), weight.type(torch.float32))
    scores = router_logits.sigmoid()                                                  # :185
    with torch.no_grad():
        topk_indices, _ = dsv3_topk_indices(scores, bias.float(), n_group, topk_group, top_k)
    topk_weights = scores.gather(1, topk_indices)                                     # :187
    if norm_topk_prob:
        denominator = topk_weights.sum(dim=-1, keepdim=True) + 1e-20                  # :189
        topk_weights = topk_weights / denominator
    topk_weights = topk_weights * routed_scaling_factor                               # :191
    return topk_indices, topk_weights, router_logits


def load_balancing_loss(gate_logits, num_experts, top_k, attention_mask=None):
    """The reference's global auxiliary loss, optimus/models/olmoe/modeling_olmoe.py:39-85, as the
    torch expressions it uses (softmax, topk, one_hot, means or masked sums), in the dtype of the
    logits.  `gate_logits` is a tuple of per-layer [T,N] tensors; `attention_mask` [batch, sequence]
    with batch * sequence == T selects the masked branch (:58-83)."""
    cat = torch.cat(list(gate_logits), dim=0)                                        # :41
    routing_weights = torch.nn.functional.softmax(cat, dim=-1)                       # :43
    _, selected = torch.topk(routing_weights, top_k, dim=-1)                         # :45
    expert_mask = torch.nn.functional.one_hot(selected, num_experts)                 # :47
    if attention_mask is None:
        tokens_per_expert = torch.mean(expert_mask.float(), dim=0)                   # :51
        router_prob_per_expert = torch.mean(routing_weights, dim=0)                  # :54
    else:
        batch_size, sequence_length = attention_mask.shape                           # :56
        num_hidden_layers = cat.shape[0] // (batch_size * sequence_length)           # :57
        expert_attention_mask = (attention_mask[None, :, :, None, None]
                                 .expand((num_hidden_layers, batch_size, sequence_length, top_k, num_experts))
                                 .reshape(-1, top_k, num_experts))                   # :60-65
        tokens_per_expert = torch.sum(expert_mask.float() * expert_attention_mask, dim=0) / torch.sum(
            expert_attention_mask, dim=0)                                            # :68-70
        router_mask = (attention_mask[None, :, :, None]
                       .expand((num_hidden_layers, batch_size, sequence_length, num_experts))
                       .reshape(-1, num_experts))                                    # :73-78
        router_prob_per_expert = torch.sum(routing_weights * router_mask, dim=0) / torch.sum(
            router_mask, dim=0)                                                      # :81-83
    return torch.sum(tokens_per_expert * router_prob_per_expert.unsqueeze(0)) * num_experts   # :84-85


def layer_level_load_balancing_loss(gate_logits, num_experts, top_k):
    """optimus/models/common/ral_functions.py:18-35: the same per layer, summed over the layers."""
    stacked = torch.stack(list(gate_logits), dim=0)
    routing_weights = torch.nn.functional.softmax(stacked, dim=-1)
    _, selected = torch.topk(routing_weights, top_k, dim=-1)
    expert_mask = torch.nn.functional.one_hot(selected, num_experts)
    tokens_per_expert = torch.mean(expert_mask.float(), dim=1)
    router_prob_per_expert = torch.mean(routing_weights, dim=1)
    return torch.sum(tokens_per_expert * router_prob_per_expert.unsqueeze(1)) * num_experts
