"""optimus.models.olmoe.modeling_olmoe — the MoE part of the reference file
(optimus/models/olmoe/modeling_olmoe.py:239-359): OlmoeParallelMLP and
OlmoeParallelSparseMoeBlock with a ModuleList of per-expert MLPs.

The reference's block loops over experts in Python (one-hot mask, where, three Linear calls,
index_add_).  Here the same module interface and parameter names run on the grouped HIP kernels:
the per-expert weights are kept at a constant pitch inside one buffer per projection
(pack_expert_weights) and handed to the kernels as a strided [NR, out, in] view, so there is one
code path for both layouts.  Sums over a token's K experts are taken in fp32 with one rounding,
where the reference's index_add_ rounds to the model dtype after every expert.
"""
import torch
import torch.nn as nn
from torch.utils.checkpoint import checkpoint as torch_activation_checkpoint

from optimus.models.common import moe as _moe
from optimus.models.common.norm import ParallelRMSNorm
from optimus.models.common.ral_functions import (  # noqa: F401  (same names as the reference module)
    layer_level_load_balancing_loss_func, load_balancing_loss_func)


class OlmoeParallelMLP(nn.Module):
    """SwiGLU MLP of one expert (reference modeling_olmoe.py:239-251)."""

    def __init__(self, config):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=False)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        """x [rows, H] -> [rows, H] through the grouped kernels with a single group."""
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        cum = _moe.single_segment_counts(x2.shape[0], x2.device)
        y = _moe.MergedMLPFunction.apply(x2, self.gate_proj.weight, self.up_proj.weight,
                                         self.down_proj.weight, cum)
        return y.reshape(*lead, -1)


class OlmoeParallelSparseMoeBlock(nn.Module):
    """Reference modeling_olmoe.py:254-359; same constructor, parameters and return value."""

    def __init__(self, config, pmap=None):
        super().__init__()
        self.pmap = pmap
        self.num_experts_per_rank = config.num_experts // config.expert_parallelism
        self.expert_start_idx = self.pmap.ep_ind * self.num_experts_per_rank
        self.expert_end_idx = (self.pmap.ep_ind + 1) * self.num_experts_per_rank

        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        self.num_experts = config.num_experts
        self.num_experts_per_tok = config.num_experts_per_tok
        self.norm_topk_prob = config.norm_topk_prob
        self.output_router_logits = config.output_router_logits

        self.gate = nn.Linear(self.hidden_size, self.num_experts, bias=False)
        self.experts = nn.ModuleList([OlmoeParallelMLP(config) for _ in range(self.num_experts_per_rank)])

        self.use_activation_checkpointing_for_moe = False
        if config.use_activation_checkpointing:
            self.use_activation_checkpointing_for_moe = config.activation_checkpointing_level & (1 << 0)
        if getattr(config, "force_uniform_routing", False):
            raise NotImplementedError("force_uniform_routing is not part of this build")

    def _expert_weights(self):
        params = []
        for expert in self.experts:
            params += [expert.gate_proj.weight, expert.up_proj.weight, expert.down_proj.weight]
        return params

    def _experts_fn(self, ggemm_input, cum_token_counts):
        _moe.pack_expert_weights(self.experts)   # no-op once the weights share a buffer
        return _moe.GroupMLPFunction.apply(ggemm_input, cum_token_counts, False,
                                           *self._expert_weights())

    def forward(self, hidden_states):
        batch_size, sequence_length, hidden_dim = hidden_states.shape
        router_logits, flat = _moe.gate_logits_with_passthrough(hidden_states.reshape(-1, hidden_dim), self.gate)
        hidden_states = flat.view(batch_size, sequence_length, hidden_dim)    # see gate_logits_with_passthrough
        routing_weights, selected_experts = _moe.SoftmaxTopkRouterFunction.apply(
            router_logits.contiguous(), self.num_experts_per_tok, self.norm_topk_prob,
            hidden_states.dtype)

        def expert_computation_block(hidden_states, selected_experts, routing_weights):
            b, s, h = hidden_states.shape
            out = _moe.expert_computation(hidden_states.reshape(-1, h), routing_weights,
                                          selected_experts, self.expert_start_idx,
                                          self.expert_end_idx, self._experts_fn, self.num_experts)
            return out.reshape(b, s, h)

        args = [hidden_states, selected_experts, routing_weights]
        if self.use_activation_checkpointing_for_moe:
            final_hidden_states = torch_activation_checkpoint(expert_computation_block, *args,
                                                              use_reentrant=False)
        else:
            final_hidden_states = expert_computation_block(*args)
        if self.output_router_logits:
            return final_hidden_states, router_logits
        return final_hidden_states, None

    def set_parameters_from_full_module(self, module):
        self.gate.load_state_dict(module.gate.state_dict())
        for local_expert_idx in range(self.num_experts_per_rank):
            self.experts[local_expert_idx].load_state_dict(
                module.experts[self.expert_start_idx + local_expert_idx].state_dict())


class OlmoeParallelRMSNorm(ParallelRMSNorm):
    """Reference modeling_olmoe.py:93-104 (eps default 1e-5)."""

    def __init__(self, hidden_size, eps=1e-5):
        super().__init__(hidden_size, eps)

