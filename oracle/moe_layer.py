"""Whole-layer restatements in PyTorch-CPU.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

* expert_mlp / olmoe_slow_block — optimus/models/olmoe/modeling_olmoe.py:239-251, :282-354
  (the reference's per-expert one-hot / where / index_add_ loop; backward by autograd).
* dsv3_moe_block                — optimus/models/deepseek_v3/modeling_deepseek_v3.py:221-275.
* fast_block_restatement        — optimus/models/common/moe.py:454-621 with the K1..K6
  operators taken from the C restatement of the SYCL kernels (oracle/clib.py) and the expert
  GEMMs as per-expert torch.matmul on slices (moe.py:174-178).
* fast_block_sequence           — the same block forward AND backward in the tensors' own dtype
  (bf16 keeps every rounding the reference's sequence of operators has: moe.py:163-215, :396-405,
  :217-377 and the SYCL kernels behind them); the yardstick for what the reference's own bf16
  path loses against float32.
* dense_formula                 — the textbook statement out[t] = sum_k w[t,k] MLP_{e[t,k]}(x[t]),
  evaluated token by token; used on tiny shapes to pin the two loops above.

All functions take plain tensors (no nn.Module) so the tests read as data in / data out.
"""
import numpy as np
import torch
import torch.nn.functional as F

from . import clib
from . import routing


def expert_mlp(x, w_gate, w_up, w_down):
    """down(silu(gate(x)) * up(x)); weights are [out, in] like nn.Linear (modeling_olmoe.py:249-251)."""
    return F.linear(F.silu(F.linear(x, w_gate)) * F.linear(x, w_up), w_down)


def olmoe_slow_block(hidden_states, gate_weight, w_gate, w_up, w_down, top_k, norm_topk_prob,
                     expert_start_idx=0, router_logits=None):
    """modeling_olmoe.py:282-354 with expert_parallelism == 1 semantics for the window.

    hidden_states [T,H]; gate_weight [N,H]; w_gate/w_up [NR,I,H]; w_down [NR,H,I].
    Accumulates in hidden_states.dtype via index_add_ in expert order, like the reference.
    Returns (final_hidden_states [T,H], router_logits [T,N]).
    """
    T, H = hidden_states.shape
    N = gate_weight.shape[0]
    NR = w_gate.shape[0]
    if router_logits is None:
        router_logits = F.linear(hidden_states, gate_weight)                       # :284
    routing_weights, selected_experts, _ = routing.olmoe_router(
        router_logits, top_k, norm_topk_prob, hidden_states.dtype)                 # :295-299
    final = torch.zeros((T, H), dtype=hidden_states.dtype)                         # :311-313
    expert_mask = F.one_hot(selected_experts, num_classes=N).permute(2, 1, 0)      # :316
    for local_expert_idx in range(NR):                                             # :322
        expert_idx = expert_start_idx + local_expert_idx
        idx, top_x = torch.where(expert_mask[expert_idx])                          # :325
        current_state = hidden_states[None, top_x].reshape(-1, H)                  # :330
        current = expert_mlp(current_state, w_gate[local_expert_idx], w_up[local_expert_idx],
                             w_down[local_expert_idx]) * routing_weights[top_x, idx, None]  # :331
        final.index_add_(0, top_x, current)                                        # :336
    return final, router_logits


def dsv3_moe_block(hidden_states, router_weight, bias, w_gate, w_up, w_down,
                   ws_gate, ws_up, ws_down, n_group, topk_group, top_k, norm_topk_prob,
                   routed_scaling_factor, expert_start_idx=0):
    """modeling_deepseek_v3.py:221-275 for one rank's window of routed experts + shared expert.

    The routed part accumulates in the routing-weight dtype (fp32) and is cast once (:222, :244).
    """
    T, H = hidden_states.shape
    N = router_weight.shape[0]
    NR = w_gate.shape[0]
    topk_indices, topk_weights, _ = routing.dsv3_router(
        hidden_states, router_weight, bias, n_group, topk_group, top_k, norm_topk_prob,
        routed_scaling_factor)
    final = torch.zeros((T, H), dtype=topk_weights.dtype)                          # :222
    expert_mask = F.one_hot(topk_indices, num_classes=N).permute(2, 0, 1)          # :224-225
    for local_expert_idx in range(NR):
        expert_idx = expert_start_idx + local_expert_idx
        token_indices, weight_indices = torch.where(expert_mask[expert_idx])       # :232
        if token_indices.numel() > 0:
            expert_weights = topk_weights[token_indices, weight_indices]
            expert_output = expert_mlp(hidden_states[token_indices], w_gate[local_expert_idx],
                                       w_up[local_expert_idx], w_down[local_expert_idx])
            final.index_add_(0, token_indices, expert_output * expert_weights.unsqueeze(-1))  # :239
    out = final.type(hidden_states.dtype)                                          # :244
    out = out + expert_mlp(hidden_states, ws_gate, ws_up, ws_down)                 # :265
    return out, topk_indices, topk_weights


def dense_formula(hidden_states, routing_weights, selected_experts, w_gate, w_up, w_down,
                  expert_start_idx=0):
    """out[t] = sum over k with a local expert of w[t,k] * MLP_{e[t,k]}(x[t]); token-by-token loop."""
    T, H = hidden_states.shape
    NR = w_gate.shape[0]
    rows = []
    for t in range(T):
        acc = torch.zeros(H, dtype=hidden_states.dtype)
        for k in range(selected_experts.shape[1]):
            ln = int(selected_experts[t, k]) - expert_start_idx
            if 0 <= ln < NR:
                acc = acc + routing_weights[t, k] * expert_mlp(hidden_states[t:t + 1], w_gate[ln],
                                                                w_up[ln], w_down[ln])[0]
        rows.append(acc)
    return torch.stack(rows)


def _np(t):
    """torch tensor -> numpy (bf16 as raw uint16 bits)."""
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)
    return t.contiguous().numpy()


def _pt(a, dtype):
    if dtype == torch.bfloat16:
        return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
    return torch.from_numpy(a)


def fast_block_restatement(hidden_states, routing_weights, selected_experts, w_gate, w_up, w_down,
                           expert_start_idx=0):
    """Forward of expert_computation_block (moe.py:473-610) for EP == 1 style windows.

    hidden_states [T,H] fp32 or bf16; selected_experts [T,K] int64; merged weights [NR,*,*].
    K1..K3, K4f and K6f come from the C restatement of the SYCL kernels; the grouped GEMM is
    the reference's loop of per-expert matmuls (moe.py:174-178) and SwiGLU the two torch ops of
    MergedMLP.forward (moe.py:401-402).  Returns (final [T,H], dict of intermediates).
    """
    dt = hidden_states.dtype
    NR = w_gate.shape[0]
    idx = clib.index_construction(selected_experts.numpy(), NR, expert_start_idx,
                                  expert_start_idx + NR)
    ggemm_input = _pt(clib.index_gather(_np(hidden_states), idx["input_indices"]), dt)
    cum = idx["cum_token_counts"]
    g = torch.empty((ggemm_input.shape[0], w_gate.shape[1]), dtype=dt)
    u = torch.empty_like(g)
    for n in range(NR):
        s, e = int(cum[n]), int(cum[n + 1])
        torch.matmul(ggemm_input[s:e], w_gate[n].t(), out=g[s:e])
        torch.matmul(ggemm_input[s:e], w_up[n].t(), out=u[s:e])
    h = F.silu(g) * u
    y = torch.empty((ggemm_input.shape[0], w_down.shape[1]), dtype=dt)
    for n in range(NR):
        s, e = int(cum[n]), int(cum[n + 1])
        torch.matmul(h[s:e], w_down[n].t(), out=y[s:e])
    final = _pt(clib.reduce_ggemm_output(_np(y), _np(routing_weights), idx["cum_expert_counts_ep"],
                                         idx["selected_experts_indices"], idx["output_indices"]), dt)
    idx.update(ggemm_input=ggemm_input, g=g, u=u, h=h, ggemm_output=y)
    return final, idx


class _SegmentMatmul(torch.autograd.Function):
    """GroupedGemmFunction with use_triton_path=False (moe.py:163-215): per expert segment
    out = in @ W[n].T; backward din = dout @ W[n], dW[n] = dout.T @ in.  Every product accumulates in
    float32 and is rounded once to the operands' dtype, which is what a bf16 GEMM with fp32
    accumulation (oneDNN on the reference's device, MFMA here) returns."""

    @staticmethod
    def forward(ctx, inp, weight, cum):
        out = torch.empty((inp.shape[0], weight.shape[1]), dtype=inp.dtype)
        for n in range(weight.shape[0]):
            s, e = int(cum[n]), int(cum[n + 1])
            out[s:e] = (inp[s:e].float() @ weight[n].float().t()).to(inp.dtype)            # :178
        ctx.save_for_backward(inp, weight)
        ctx.cum = cum
        return out

    @staticmethod
    def backward(ctx, dout):
        inp, weight = ctx.saved_tensors
        cum = ctx.cum
        din = torch.empty_like(inp)
        dw = torch.empty_like(weight)
        for n in range(weight.shape[0]):
            s, e = int(cum[n]), int(cum[n + 1])
            din[s:e] = (dout[s:e].float() @ weight[n].float()).to(inp.dtype)               # :208
            dw[n] = (dout[s:e].float().t() @ inp[s:e].float()).to(weight.dtype)            # :210
        return din, dw, None


class _GatherRows(torch.autograd.Function):
    """PrepareInputForGroupGemmFunction (moe.py:217-282): index_gather forward,
    shuffle_sub_matrix_reduce backward (sparse_moe_block.sycl:56-106, :478-532)."""

    @staticmethod
    def forward(ctx, hidden_states, idx):
        ctx.idx, ctx.T = idx, hidden_states.shape[0]
        return _pt(clib.index_gather(_np(hidden_states), idx["input_indices"]), hidden_states.dtype)

    @staticmethod
    def backward(ctx, grad):
        idx = ctx.idx
        return _pt(clib.shuffle_sub_matrix_reduce(_np(grad), idx["cum_expert_counts_ep"],
                                                  idx["output_indices"], ctx.T), grad.dtype), None


class _CombineRows(torch.autograd.Function):
    """GroupGemmOutputReductionFunction (moe.py:284-377): reduce_ggemm_output forward,
    reduce_ggemm_output_backward backward (sparse_moe_block.sycl:282-475)."""

    @staticmethod
    def forward(ctx, y, routing_weights, idx):
        ctx.idx = idx
        ctx.save_for_backward(y, routing_weights)
        return _pt(clib.reduce_ggemm_output(_np(y), _np(routing_weights), idx["cum_expert_counts_ep"],
                                            idx["selected_experts_indices"], idx["output_indices"]), y.dtype)

    @staticmethod
    def backward(ctx, dfinal):
        y, routing_weights = ctx.saved_tensors
        idx = ctx.idx
        dy, dw = clib.reduce_ggemm_output_backward(_np(dfinal.contiguous()), _np(y), _np(routing_weights),
                                                   idx["selected_experts_indices"], idx["input_indices"],
                                                   idx["output_indices"])
        return _pt(dy, y.dtype), _pt(dw, routing_weights.dtype), None


def fast_block_sequence(hidden_states, routing_weights, selected_experts, w_gate, w_up, w_down, dfinal,
                        expert_start_idx=0):
    """expert_computation_block of the fast block (moe.py:473-610), forward and backward, as the
    reference runs it: K4 gather -> MergedMLP.forward (three GroupedGemmFunction calls, torch's silu
    and multiply, moe.py:396-405) -> K6 combine, gradients by autograd through exactly those
    operators.  In bfloat16 every operator rounds its result to bfloat16 as on the reference's
    device (g, u, silu(g), h, y, dy, dh, d silu, dg, du, the two dx terms and their sum), with
    fp32 accumulation inside every product and inside K4's and K6's sums.

    All tensors in one dtype (float32 or bfloat16); selected_experts [T,K] int64.
    Returns (final [T,H], {"x", "routing_weights", "w_gate", "w_up", "w_down"} gradients)."""
    NR = w_gate.shape[0]
    idx = clib.index_construction(selected_experts.numpy(), NR, expert_start_idx, expert_start_idx + NR)
    cum = idx["cum_token_counts"]
    leaves = {"x": hidden_states, "routing_weights": routing_weights, "w_gate": w_gate, "w_up": w_up,
              "w_down": w_down}
    leaves = {k: v.detach().clone().requires_grad_(True) for k, v in leaves.items()}
    ggemm_input = _GatherRows.apply(leaves["x"], idx)
    g = _SegmentMatmul.apply(ggemm_input, leaves["w_gate"], cum)            # moe.py:398
    u = _SegmentMatmul.apply(ggemm_input, leaves["w_up"], cum)              # moe.py:399
    h = F.silu(g) * u                                                       # moe.py:401-402
    y = _SegmentMatmul.apply(h, leaves["w_down"], cum)                      # moe.py:404
    final = _CombineRows.apply(y, leaves["routing_weights"], idx)
    final.backward(dfinal)
    return final.detach(), {k: v.grad for k, v in leaves.items()}


def rmsnorm(hidden_states, weight, eps, residual=None):
    """OlmoeParallelRMSNorm.forward, optimus/models/olmoe/modeling_olmoe.py:98-104, preceded by the
    residual add of the layer body (:402) when `residual` is given.  Returns (y, h)."""
    if residual is not None:
        hidden_states = hidden_states + residual                                   # :402
    input_dtype = hidden_states.dtype
    h32 = hidden_states.to(torch.float32)                                          # :100
    variance = h32.pow(2).mean(-1, keepdim=True)                                   # :101
    h32 = h32 * torch.rsqrt(variance + eps)                                        # :102
    return weight * h32.to(input_dtype), hidden_states                             # :103
