"""optimus.models.deepseek_v3.modeling_deepseek_v3 — the MoE part of the reference file
(optimus/models/deepseek_v3/modeling_deepseek_v3.py:79-282): DeepseekV3ParallelMLP,
DeepseekV3ParallelTopkRouter, DeepseekV3ParallelMoE.

The reference has no fast path for this block: it loops over the local experts in Python with an
fp32 [T,H] accumulator.  Here the same modules run the grouped HIP kernels: sigmoid /
group-limited top-K router kernel, the counting-sort permutation restricted to this rank's expert
window, the merged-MLP GEMMs over the per-expert weights (strided view, no copies) and the fp32
weighted combine with fp32 routing weights; the shared expert is the same GEMM with one group.
With expert_parallelism > 1 only this rank's window of experts is computed; the token exchange
with the other ranks is not performed (one GPU's share).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.utils.checkpoint import checkpoint as torch_activation_checkpoint

from optimus import _native as _n
from optimus.models.common import moe as _moe
from optimus.models.common.norm import ParallelRMSNorm


class DeepseekV3ParallelMLP(nn.Module):
    """SwiGLU MLP (reference modeling_deepseek_v3.py:79-129)."""

    def __init__(self, config, hidden_size=None, intermediate_size=None, pmap=None):
        super().__init__()
        self.config = config
        self.pmap = pmap
        self.hidden_size = config.hidden_size if hidden_size is None else hidden_size
        self.intermediate_size = config.intermediate_size if intermediate_size is None else intermediate_size
        if self.pmap is None:
            self.intermediate_size_per_rank = self.intermediate_size
        else:
            self.intermediate_size_per_rank = config.intermediate_size // self.pmap.expert_parallelism
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size_per_rank, bias=False)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size_per_rank, bias=False)
        self.down_proj = nn.Linear(self.intermediate_size_per_rank, self.hidden_size, bias=False)
        self.act_fn = nn.SiLU()

    def forward(self, hidden_states):
        lead = hidden_states.shape[:-1]
        x2 = hidden_states.reshape(-1, hidden_states.shape[-1]).contiguous()
        cum = _moe.single_segment_counts(x2.shape[0], x2.device)
        y = _moe.MergedMLPFunction.apply(x2, self.gate_proj.weight, self.up_proj.weight,
                                         self.down_proj.weight, cum)
        return y.reshape(*lead, -1)

    def set_parameters_from_full_module(self, module):
        self.load_state_dict(module.state_dict())


class SigmoidGroupTopkRouterFunction(torch.autograd.Function):
    """(topk_indices, topk_weights) from fp32 router logits: reference
    modeling_deepseek_v3.py:150-180 (selection, no grad) and :185-191 (weights).  Index order
    within a token is (choice score desc, expert index asc); the reference leaves it unspecified
    (torch.topk(sorted=False))."""

    @staticmethod
    def forward(ctx, router_logits, bias, n_group, topk_group, top_k, norm_topk_prob, scale):
        _n.require_cuda_contiguous(router_logits, bias)
        T, N = router_logits.shape
        experts = torch.empty((T, top_k), dtype=torch.int64, device=router_logits.device)
        weights = torch.empty((T, top_k), dtype=torch.float32, device=router_logits.device)
        _n.check(_n.lib().om_route_sigmoid_group_topk(
            _n.ptr(router_logits), _n.ptr(bias), T, N, n_group, topk_group, top_k,
            int(bool(norm_topk_prob)), float(scale), _n.ptr(experts), _n.ptr(weights), _n.stream()),
            "om_route_sigmoid_group_topk")
        ctx.save_for_backward(router_logits, experts)
        ctx.cfg = (bool(norm_topk_prob), float(scale))
        ctx.mark_non_differentiable(experts)
        return experts, weights

    @staticmethod
    def backward(ctx, _experts_grad, weights_grad):
        router_logits, experts = ctx.saved_tensors
        norm, scale = ctx.cfg
        T, N = router_logits.shape
        dlogits = torch.empty_like(router_logits)
        _n.check(_n.lib().om_route_sigmoid_topk_bwd(
            _n.ptr(router_logits), _n.ptr(experts), _n.ptr(weights_grad.contiguous().float()), T, N,
            experts.shape[1], int(norm), scale, _n.ptr(dlogits), _n.stream()),
            "om_route_sigmoid_topk_bwd")
        return dlogits, None, None, None, None, None, None


class DeepseekV3ParallelTopkRouter(nn.Module):
    """Reference modeling_deepseek_v3.py:131-192."""

    def __init__(self, config, pmap=None):
        super().__init__()
        self.config = config
        self.pmap = pmap
        self.top_k = config.num_experts_per_tok
        self.n_routed_experts = config.n_routed_experts
        self.routed_scaling_factor = config.routed_scaling_factor
        self.n_group = config.n_group
        self.topk_group = config.topk_group
        self.norm_topk_prob = config.norm_topk_prob
        self.weight = nn.Parameter(torch.empty((self.n_routed_experts, config.hidden_size)))
        self.register_buffer("e_score_correction_bias", torch.zeros(self.n_routed_experts))
        if getattr(config, "force_uniform_routing", False):
            raise NotImplementedError("force_uniform_routing is not part of this build")

    def forward(self, hidden_states):
        return self.forward_with_passthrough(hidden_states)[:2]

    def forward_with_passthrough(self, hidden_states):
        """(topk_indices, topk_weights, hidden_states [T,H]): the third result is the gate
        projection's pass-through of its input; experts fed from it get their input gradient added
        to the gate's inside the gate's input-gradient kernel (GateLogitsFunction)."""
        hidden_states = hidden_states.reshape(-1, self.config.hidden_size)
        router_logits, hidden_states = _moe.fp32_logits_with_passthrough(hidden_states, self.weight)
        topk_indices, topk_weights = SigmoidGroupTopkRouterFunction.apply(
            router_logits.contiguous(), self.e_score_correction_bias.float().contiguous(),
            self.n_group, self.topk_group, self.top_k, self.norm_topk_prob,
            self.routed_scaling_factor)
        return topk_indices, topk_weights, hidden_states


class DeepseekV3ParallelMoE(nn.Module):
    """Reference modeling_deepseek_v3.py:194-282.  forward(x [B,S,H]) -> [B,S,H]."""

    def __init__(self, config, pmap=None):
        super().__init__()
        self.config = config
        self.pmap = pmap
        self.n_routed_experts_per_rank = config.n_routed_experts // config.expert_parallelism
        self.expert_start_idx = self.pmap.ep_ind * self.n_routed_experts_per_rank
        self.expert_end_idx = (self.pmap.ep_ind + 1) * self.n_routed_experts_per_rank
        self.experts = nn.ModuleList([
            DeepseekV3ParallelMLP(config, intermediate_size=config.moe_intermediate_size)
            for _ in range(self.n_routed_experts_per_rank)])
        self.gate = DeepseekV3ParallelTopkRouter(config, pmap=self.pmap)
        self.shared_experts = DeepseekV3ParallelMLP(
            config=config, intermediate_size=config.moe_intermediate_size * config.n_shared_experts)
        self.use_activation_checkpointing_for_moe = False
        if config.use_activation_checkpointing:
            self.use_activation_checkpointing_for_moe = config.activation_checkpointing_level & (1 << 0)

    def _experts_fn(self, ggemm_input, cum_token_counts):
        _moe.pack_expert_weights(self.experts)   # no-op once the weights share a buffer
        params = []
        for expert in self.experts:
            params += [expert.gate_proj.weight, expert.up_proj.weight, expert.down_proj.weight]
        return _moe.GroupMLPFunction.apply(ggemm_input, cum_token_counts, False, *params)

    def _gathered_experts_fn(self, hidden_states, input_indices, cum_expert_counts_ep, output_indices,
                             cum_token_counts):
        _moe.pack_expert_weights(self.experts)
        params = []
        for expert in self.experts:
            params += [expert.gate_proj.weight, expert.up_proj.weight, expert.down_proj.weight]
        return _moe.GatheredGroupMLPFunction.apply(hidden_states, input_indices, cum_expert_counts_ep,
                                                   output_indices, cum_token_counts, *params)

    def _routed_kernels_fit(self, hidden_states, routing_weights):
        w0, d0 = self.experts[0].gate_proj.weight, self.experts[0].down_proj.weight
        return _moe.routed_mlp_kernel_fits(hidden_states, routing_weights, w0.unsqueeze(0), d0.unsqueeze(0))

    def _routed_experts_fn(self, hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                           output_indices, selected_experts_indices, cum_token_counts, residual,
                           rows_is_bound=False, with_shared=False):
        _moe.pack_expert_weights(self.experts)
        w0, d0 = self.experts[0].gate_proj.weight, self.experts[0].down_proj.weight
        why = _moe.routed_mlp_unfit_reason(hidden_states, routing_weights, w0.unsqueeze(0), d0.unsqueeze(0))
        if why is not None:
            if hidden_states.dtype == torch.bfloat16:    # (float32 modules run unfused by design)
                _moe.note_unfused_path("routing weight inside the expert MLP", why)
            return None
        params = []
        for expert in self.experts:
            params += [expert.gate_proj.weight, expert.up_proj.weight, expert.down_proj.weight]
        if with_shared:
            sh = self.shared_experts
            return _moe.RoutedAndSharedMLPFunction.apply(
                hidden_states, routing_weights, input_indices, cum_expert_counts_ep, output_indices,
                selected_experts_indices, cum_token_counts, rows_is_bound, *params, sh.gate_proj.weight,
                sh.up_proj.weight, sh.down_proj.weight)
        return _moe.RoutedMLPFunction.apply(hidden_states, routing_weights, input_indices,
                                            cum_expert_counts_ep, output_indices, selected_experts_indices,
                                            cum_token_counts, residual,
                                            "per_expert_bound" if rows_is_bound else False, *params)

    def _fuses_routing_weights(self):
        return getattr(self.config, "fuse_input_gather", True) and \
            getattr(self.config, "fuse_routing_weights", True)

    def moe(self, hidden_states, topk_indices, topk_weights, residual=None, with_shared=False):
        """Routed part for [T,H] hidden_states (reference :221-244): fp32 weights, fp32 sum over a
        token's local experts, one rounding to the activation dtype.  The local experts read their
        tokens through the permutation index (no gathered copy of the activations) and apply the
        routing weight themselves (RoutedMLPFunction) unless the config switches that off.
        `residual` [T,H] is added to the rounded result inside the combine kernel.  `with_shared`
        (needs the fused path): the shared experts run inside the same function and their output
        is that residual (RoutedAndSharedMLPFunction)."""
        gathered = self._gathered_experts_fn if getattr(self.config, "fuse_input_gather", True) else None
        routed = None
        if self._fuses_routing_weights():
            routed = self._routed_experts_fn
            if with_shared:
                routed = lambda *a, **kw: self._routed_experts_fn(*a, with_shared=True, **kw)
        elif with_shared:
            raise ValueError("with_shared needs the fused routing-weight path")
        return _moe.expert_computation(hidden_states, topk_weights, topk_indices,
                                       self.expert_start_idx, self.expert_end_idx, self._experts_fn,
                                       self.config.n_routed_experts, gathered_experts_fn=gathered,
                                       residual=residual, routed_experts_fn=routed,
                                       sync_free_window=getattr(self.config, "sync_free_expert_window", False))

    def forward(self, hidden_states):
        # the experts are fed from the gate projection's pass-through of the hidden states, so that
        # their input gradient and the gate's are added inside one kernel
        topk_indices, topk_weights, flat = self.gate.forward_with_passthrough(hidden_states)
        hidden_states = flat.view(hidden_states.shape)

        def expert_computation_block(hidden_states, topk_indices, topk_weights):
            residuals = hidden_states
            orig_shape = hidden_states.shape
            flat = hidden_states.reshape(-1, hidden_states.shape[-1])
            # routed + shared (reference :265): the shared experts' output goes into the combine
            # kernel as its residual, which rounds the routed sum first and then adds: the same two
            # roundings as `moe(...) + shared_experts(...)`
            if self._fuses_routing_weights() and self._routed_kernels_fit(flat, topk_weights):
                return self.moe(flat, topk_indices, topk_weights, with_shared=True).view(*orig_shape)
            shared = self.shared_experts(residuals).reshape(flat.shape)
            return self.moe(flat, topk_indices, topk_weights, residual=shared).view(*orig_shape)

        args = [hidden_states, topk_indices, topk_weights]
        if self.use_activation_checkpointing_for_moe:
            return torch_activation_checkpoint(expert_computation_block, *args, use_reentrant=False)
        return expert_computation_block(*args)

    def set_parameters_from_full_module(self, module):
        self.gate.load_state_dict(module.gate.state_dict())
        for local_expert_idx in range(self.n_routed_experts_per_rank):
            self.experts[local_expert_idx].load_state_dict(
                module.experts[self.expert_start_idx + local_expert_idx].state_dict())
        self.shared_experts.load_state_dict(module.shared_experts.state_dict())


class DeepseekV3ParallelRMSNorm(ParallelRMSNorm):
    """Reference modeling_deepseek_v3.py:29-44 (eps default 1e-6)."""

    def __init__(self, hidden_size, eps=1e-6):
        super().__init__(hidden_size, eps)

